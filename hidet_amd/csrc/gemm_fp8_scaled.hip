// Block-scaled FP8 e4m3 GEMM (DeepSeek-style): for every K block of 128
//   c[m, n] += (sum_{k in block} a[m, k] * b[n, k]) * scale_a[kb, m] * scale_b[n / 128, kb]
// with scale_a float32 [K/128, M] (M contiguous) and scale_b float32 [N/128, K/128].
//
// Each k block is multiplied into a scratch accumulator (one 16x16x128 MFMA per 16 x 16 block, C = 0) and folded into
// the running sum with its two scales on the vector ALU: one fma per accumulator element and k block, which the MFMA
// cannot absorb (its built-in block scales are powers of two).
//
// gemm_fp8_scaled_kernel8 (tensors below 1 GiB, 16-byte aligned): workgroup tile 256 x 128 (one scale_b entry per k
// block), eight waves of 64 x 64 - two per SIMD, so that one wave's folding overlaps the other's MFMAs; in a single
// wave the two do not overlap - operand tiles straight into a three-slot LDS ring (buffer_load ... lds) two k blocks
// ahead, one barrier per k block, hand-placed fragment reads, the scratch accumulator double-buffered per row block so
// that the fold of row block i runs behind the MFMAs of row block i + 1. The running sums live in VGPRs (the VALU cannot
// read accumulation registers). gemm_fp8_scaled_kernel (128 x 128 tile, register-staged double-buffered LDS) takes
// the rest.
#include "common.h"
#include "gemm_tiling.h"
#include "numeric.h"

namespace qmm {
namespace {

constexpr int kT = 128;  // tile rows, tile columns and k-step bytes
constexpr int kThreads = 256;
constexpr int kStageChunks = 2 * kT * 8;
constexpr int kChunksPerThread = kStageChunks / kThreads;  // 8
constexpr int kLdsBytes = 2 * kStageChunks * 16;           // 64 KiB

template <int OUT>
__device__ __forceinline__ void store4_scaled(void *c, int64_t o, float4_t v) {
    if (OUT == HIDET_QMM_F32) {
        *reinterpret_cast<float4_t *>(static_cast<float *>(c) + o) = v;
    } else if (OUT == HIDET_QMM_BF16) {
        uint2 w2;
        w2.x = uint32_t(f32_to_bf16_bits(v[0])) | (uint32_t(f32_to_bf16_bits(v[1])) << 16);
        w2.y = uint32_t(f32_to_bf16_bits(v[2])) | (uint32_t(f32_to_bf16_bits(v[3])) << 16);
        *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(c) + o) = w2;
    } else if (OUT == HIDET_QMM_F16) {
        uint2 w2;
        w2.x = uint32_t(f32_to_f16_bits(v[0])) | (uint32_t(f32_to_f16_bits(v[1])) << 16);
        w2.y = uint32_t(f32_to_f16_bits(v[2])) | (uint32_t(f32_to_f16_bits(v[3])) << 16);
        *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(c) + o) = w2;
    } else if (OUT == HIDET_QMM_E5M2) {
        *reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(c) + o) =
            uint32_t(f32_to_e5m2(v[0])) | (uint32_t(f32_to_e5m2(v[1])) << 8) | (uint32_t(f32_to_e5m2(v[2])) << 16) |
            (uint32_t(f32_to_e5m2(v[3])) << 24);
    } else {
        *reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(c) + o) =
            uint32_t(f32_to_e4m3(v[0])) | (uint32_t(f32_to_e4m3(v[1])) << 8) | (uint32_t(f32_to_e4m3(v[2])) << 16) |
            (uint32_t(f32_to_e4m3(v[3])) << 24);
    }
}

// FMT: operand format of the MFMA, 0 = float8 e4m3, 1 = float8 e5m2 (both operands the same).
template <int OUT, int FMT = 0>
__global__ __launch_bounds__(kThreads, 1) void gemm_fp8_scaled_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                                      const float *__restrict__ scale_a,
                                                                      const float *__restrict__ scale_b, void *__restrict__ c,
                                                                      int m, int n, int k, int tiles_m) {
    extern __shared__ uint4 lds[];
    const int m0 = (blockIdx.x % tiles_m) * kT;
    const int nb = blockIdx.x / tiles_m;
    const int n0 = nb * kT;
    const int kblocks = k / 128;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int kg = lane >> 4, ls = lane & 15;

    float4_t total[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) total[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    uint4 stage[kChunksPerThread];
    auto load_stage = [&](int kbase) {
#pragma unroll
        for (int j = 0; j < kChunksPerThread; ++j) {
            const int id = j * kThreads + tid;
            const int row = id >> 3, pos = id & 7;
            const int kb = kbase + (pos ^ (row & 7)) * 16;
            stage[j] = uint4{0u, 0u, 0u, 0u};
            if (j < kChunksPerThread / 2) {
                if (m0 + row < m) stage[j] = *reinterpret_cast<const uint4 *>(a + int64_t(m0 + row) * k + kb);
            } else {
                if (n0 + row - kT < n) stage[j] = *reinterpret_cast<const uint4 *>(b + int64_t(n0 + row - kT) * k + kb);
            }
        }
    };
    auto store_stage = [&](int buf) {
#pragma unroll
        for (int j = 0; j < kChunksPerThread; ++j) lds[buf * kStageChunks + j * kThreads + tid] = stage[j];
    };

    load_stage(0);
    store_stage(0);
    __syncthreads();

    for (int s = 0; s < kblocks; ++s) {
        const int buf = s & 1;
        const bool more = s + 1 < kblocks;
        if (more) load_stage((s + 1) * 128);
        // scale of this k block for the lane's 4 rows (one per row block) and the tile's column block
        const float sb = scale_b[int64_t(nb) * kblocks + s];
        float f[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = m0 + wm * 64 + i * 16 + ls;
            f[i] = row < m ? scale_a[int64_t(s) * m + row] * sb : 0.f;
        }
        const uint4 *la = lds + buf * kStageChunks;
        const uint4 *lb = la + kT * 8;
        uint4 bf[4][2];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = wn * 64 + j * 16 + ls;
            bf[j][0] = lb[r * 8 + ((2 * kg) ^ (r & 7))];
            bf[j][1] = lb[r * 8 + ((2 * kg + 1) ^ (r & 7))];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = wm * 64 + i * 16 + ls;
            const uint4 a0 = la[r * 8 + ((2 * kg) ^ (r & 7))];
            const uint4 a1 = la[r * 8 + ((2 * kg + 1) ^ (r & 7))];
            int8v_t cv;
            cv[0] = int(a0.x); cv[1] = int(a0.y); cv[2] = int(a0.z); cv[3] = int(a0.w);
            cv[4] = int(a1.x); cv[5] = int(a1.y); cv[6] = int(a1.z); cv[7] = int(a1.w);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int8v_t rv;
                rv[0] = int(bf[j][0].x); rv[1] = int(bf[j][0].y); rv[2] = int(bf[j][0].z); rv[3] = int(bf[j][0].w);
                rv[4] = int(bf[j][1].x); rv[5] = int(bf[j][1].y); rv[6] = int(bf[j][1].z); rv[7] = int(bf[j][1].w);
                const float4_t part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    rv, cv, float4_t{0.f, 0.f, 0.f, 0.f}, FMT, FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
#pragma unroll
                for (int v = 0; v < 4; ++v) total[i][j][v] += part[v] * f[i];
            }
        }
        if (more) store_stage(buf ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = m0 + wm * 64 + i * 16 + ls;
        if (row >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + wn * 64 + j * 16 + 4 * kg;
            if (col >= n) continue;
            const int64_t o = int64_t(row) * n + col;
            const float4_t v = total[i][j];
            store4_scaled<OUT>(c, o, v);
        }
    }
}


// ---- fast path ---------------------------------------------------------------------------------------------------------

constexpr int kM8 = 256, kN8 = 128;           // workgroup tile
constexpr int kThreads8 = 512;
constexpr int kSlotChunks8 = (kM8 + kN8) * 8;  // 16-byte chunks of one k block: A rows then B rows
constexpr int kLoads8 = kSlotChunks8 / kThreads8;  // 6 direct-to-LDS loads per thread and k block
constexpr int kRingBytes8 = 3 * kSlotChunks8 * 16;  // 144 KiB
constexpr int kLdsBytes8 = kRingBytes8 + 16;       // + the K-split fix-up's flag; the ring must start at LDS address 0

template <int FMT>
__device__ __forceinline__ float4_t mfma_fp8_k128_fresh(const int4v_t &r0, const int4v_t &r1, const int4v_t &c0, const int4v_t &c1) {
    const int8v_t rv = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
    const int8v_t cv = __builtin_shufflevector(c0, c1, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rv, cv, float4_t{0.f, 0.f, 0.f, 0.f}, FMT, FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
}

// SCALED: scale_a / scale_b are the block scales described at the top of the file. !SCALED: plain a x b^T with optional
// per-tensor scales (one float each, may be null), applied to the sums in the epilogue.
template <int OUT, bool SCALED, int FMT = 0>
__global__ __launch_bounds__(kThreads8, 1) void gemm_fp8_kernel8(const uint8_t *__restrict__ a, int64_t lda,
                                                                 const uint8_t *__restrict__ b, int64_t ldb,
                                                                 const float *__restrict__ scale_a,
                                                                 const float *__restrict__ scale_b, void *__restrict__ c,
                                                                 int m, int n, int k, int tiles_m, int tiles_n, int xm, int xn,
                                                                 int tail_parts, int tail_stride, float *__restrict__ partials,
                                                                 uint32_t *__restrict__ counters) {
    extern __shared__ uint4 lds[];  // [3][kSlotChunks8]; no static LDS: fragment reads address the ring from 0
    int &s_last = *reinterpret_cast<int *>(lds + kRingBytes8 / 16);
    GemmWorkItem item;
    if (!gemm_work_item(tiles_m, tiles_n, xm, xn, 32, tail_parts, tail_stride, &item)) return;
    const int tile_m = item.tile_m, tile_n = item.tile_n;
    const int m0 = tile_m * kM8, n0 = tile_n * kN8;
    const int kblocks = k / 128;
    // this workgroup's K range (the whole of K unless the launch splits tail tiles)
    const int kb_begin = (kblocks * item.part) / item.parts, kb_end = (kblocks * (item.part + 1)) / item.parts;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int kg = lane >> 4, ls = lane & 15;

    float4_t total[4][4];  // [row block][column block] of this wave's 64 x 64
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) total[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    const __amdgpu_buffer_rsrc_t rsrc_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(a), 0, int(int64_t(m - 1) * lda + k), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(b), 0, int(int64_t(n - 1) * ldb + k), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_sa = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(scale_a), 0, SCALED ? int(int64_t(kblocks) * m * 4) : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_sb = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(scale_b), 0, SCALED ? int(int64_t(n / 128) * kblocks * 4) : 0, 0x00020000);

    // Load instruction j of a wave fills chunk slots j * 512 + wave * 64 .. + 63 of a k block: tile row j * 64 + tid / 8
    // (A rows for j < 4, B rows after), position tid % 8, which holds chunk (tid % 8) ^ key(row). Rows past the end of a
    // tensor get an offset outside the buffer and read as zero.
    constexpr int kOutside = 0x7FFFFFF0;
    const int chunk = (tid & 7) ^ lds_swizzle_key_step2(tid >> 3);
    int voff[kLoads8];
#pragma unroll
    for (int j = 0; j < kLoads8; ++j) {
        const int r = j * 64 + (tid >> 3);
        if (j < 4) voff[j] = m0 + r < m ? int(int64_t(m0 + r) * lda) + chunk * 16 : kOutside;
        else voff[j] = n0 + r - kM8 < n ? int(int64_t(n0 + r - kM8) * ldb) + chunk * 16 : kOutside;
    }
    // A short matrix leaves most of the 256 tile rows empty: load instructions whose 64 rows all lie past M are left
    // out (a_cnt of the 4 stay; the same for every wave), and a wave whose 64 output rows do skips its fragment reads
    // and MFMAs.
    int a_cnt = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) a_cnt += int(m0 + j * 64 < m);
    const bool wave_active = m0 + wm * 64 < m;
    // (all_tag: the tile is full - no conditions in the loop)
    auto load_tiles = [&](int kb, int slot, auto all_tag) {
        // the scalar offset is not part of the buffer's range check: a prefetch past the end of K re-reads the last block
        const int kbc = kb < kblocks ? kb : kblocks - 1;
        uint4 *dst = lds + slot * kSlotChunks8 + wave * 64;
#pragma unroll
        for (int j = 0; j < kLoads8; ++j)
            if (decltype(all_tag)::value || j >= 4 || j < a_cnt)
                buffer_load_to_lds_b128(j < 4 ? rsrc_a : rsrc_b, dst + j * kThreads8, voff[j], kbc * 128);
    };
    auto load_tile_one = [&](auto j_tag, int kb, int slot) {  // one of the kLoads8 instructions of load_tiles, full tiles
        constexpr int J = decltype(j_tag)::value;
        const int kbc = kb < kblocks ? kb : kblocks - 1;
        buffer_load_to_lds_b128(J < 4 ? rsrc_a : rsrc_b, lds + slot * kSlotChunks8 + wave * 64 + J * kThreads8, voff[J], kbc * 128);
    };
    auto wait_older_tiles = [&](auto all_tag) {  // everything but the loads of the last load_scales + load_tiles has landed
        constexpr int kScaleLoads = SCALED ? 5 : 0;
        if (decltype(all_tag)::value) {
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(kScaleLoads + kLoads8));
            return;
        }
        switch (a_cnt) {
            case 1: __builtin_amdgcn_s_waitcnt(waitcnt_vm(kScaleLoads + 3)); break;
            case 2: __builtin_amdgcn_s_waitcnt(waitcnt_vm(kScaleLoads + 4)); break;
            case 3: __builtin_amdgcn_s_waitcnt(waitcnt_vm(kScaleLoads + 5)); break;
            default: __builtin_amdgcn_s_waitcnt(waitcnt_vm(kScaleLoads + 6)); break;
        }
    };
    // scales of a k block: the lane's 4 rows (one per row block) and the tile's column block
    int sa_off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = m0 + wm * 64 + i * 16 + ls;
        sa_off[i] = row < m ? row * 4 : kOutside;
    }
    const int sb_off = tile_n * kblocks * 4;
    float sa_next[4] = {1.f, 1.f, 1.f, 1.f}, sb_next = 1.f;
    auto load_scales = [&](int kb) {
        if constexpr (!SCALED) return;
        const int kbc = kb < kblocks ? kb : kblocks - 1;  // scalar offsets are not range-checked: stay inside
#pragma unroll
        for (int i = 0; i < 4; ++i) sa_next[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_sa, sa_off[i], kbc * m * 4, 0));
        sb_next = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_sb, sb_off, kbc * 4, 0));
    };

    // LDS byte addresses of this lane's two 16-byte fragment halves in block 0 of its wave, ring slot 0; block i adds
    // i * 16 rows = i * 2048 bytes
    uint32_t a_addr[2], b_addr[2];
    {
        const int ra = wm * 64 + ls, rb = kM8 + wn * 64 + ls;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            a_addr[h] = uint32_t((ra * 8 + ((2 * kg + h) ^ lds_swizzle_key_step2(ra))) * 16);
            b_addr[h] = uint32_t((rb * 8 + ((2 * kg + h) ^ lds_swizzle_key_step2(rb))) * 16);
        }
    }
    constexpr uint32_t kSlotBytes = kSlotChunks8 * 16;

    load_scales(kb_begin);
    load_tiles(kb_begin, 0, std::false_type());
    load_tiles(kb_begin + 1, 1, std::false_type());
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __builtin_amdgcn_s_barrier();

    auto k_loop = [&](auto all_tag) {
    for (int s = kb_begin, slot = 0; s < kb_end; ++s) {
        float f[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = sa_next[i] * sb_next;
        load_scales(s + 1);                           // issued before the tile loads: waiting for them later does not
        // wait for these. Slot (s + 2) % 3 was last read in k block s - 1. Full tiles issue the six load instructions two,
        // two, one and one at a time between the row blocks instead of in one burst behind the barrier (every wave of the
        // workgroup would queue its burst at the same moment, in front of its MFMAs).
        constexpr bool kSpread = decltype(all_tag)::value;
        const int slot_in = slot >= 1 ? slot - 1 : 2;
        if constexpr (kSpread) {
            load_tile_one(std::integral_constant<int, 0>(), s + 2, slot_in);
            load_tile_one(std::integral_constant<int, 1>(), s + 2, slot_in);
        } else {
            load_tiles(s + 2, slot_in, all_tag);
        }
        if (decltype(all_tag)::value || wave_active) {
        const uint32_t so = uint32_t(slot) * kSlotBytes;
        const uint32_t aa0 = a_addr[0] + so, aa1 = a_addr[1] + so, ba0 = b_addr[0] + so, ba1 = b_addr[1] + so;
        int4v_t bf[4][2], af[4][2];
        bf[0][0] = lds_read_b128_early<0>(ba0);        bf[0][1] = lds_read_b128_early<0>(ba1);
        af[0][0] = lds_read_b128_early<0>(aa0);        af[0][1] = lds_read_b128_early<0>(aa1);
        bf[1][0] = lds_read_b128_early<2048>(ba0);     bf[1][1] = lds_read_b128_early<2048>(ba1);
        bf[2][0] = lds_read_b128_early<4096>(ba0);     bf[2][1] = lds_read_b128_early<4096>(ba1);
        bf[3][0] = lds_read_b128_early<6144>(ba0);     bf[3][1] = lds_read_b128_early<6144>(ba1);
        af[1][0] = lds_read_b128_early<2048>(aa0);     af[1][1] = lds_read_b128_early<2048>(aa1);
        af[2][0] = lds_read_b128_early<4096>(aa0);     af[2][1] = lds_read_b128_early<4096>(aa1);
        af[3][0] = lds_read_b128_early<6144>(aa0);     af[3][1] = lds_read_b128_early<6144>(aa1);
        __builtin_amdgcn_sched_barrier(0);
        float4_t part[2][4];  // scratch accumulators of two consecutive row blocks
        // row block 0: fragments arrive in issue order b0, a0, b1, b2, b3 (then a1 .. a3: 6 reads)
        lds_wait_keep_newer<12>(bf[0][0], bf[0][1]);
        lds_wait_keep_newer<12>(af[0][0], af[0][1]);
        auto mm = [&](float4_t &dst_scaled, float4_t &dst_plain, const int4v_t &r0, const int4v_t &r1, const int4v_t &c0, const int4v_t &c1) {
            if constexpr (SCALED) dst_scaled = mfma_fp8_k128_fresh<FMT>(r0, r1, c0, c1);
            else {
                const int8v_t rv = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
                const int8v_t cv = __builtin_shufflevector(c0, c1, 0, 1, 2, 3, 4, 5, 6, 7);
                dst_plain = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rv, cv, dst_plain, FMT, FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
            }
        };
        mm(part[0][0], total[0][0], bf[0][0], bf[0][1], af[0][0], af[0][1]);
        lds_wait_keep_newer<10>(bf[1][0], bf[1][1]);
        mm(part[0][1], total[0][1], bf[1][0], bf[1][1], af[0][0], af[0][1]);
        lds_wait_keep_newer<8>(bf[2][0], bf[2][1]);
        mm(part[0][2], total[0][2], bf[2][0], bf[2][1], af[0][0], af[0][1]);
        lds_wait_keep_newer<6>(bf[3][0], bf[3][1]);
        mm(part[0][3], total[0][3], bf[3][0], bf[3][1], af[0][0], af[0][1]);
        if constexpr (kSpread) {
            load_tile_one(std::integral_constant<int, 2>(), s + 2, slot_in);
            load_tile_one(std::integral_constant<int, 3>(), s + 2, slot_in);
        }
        __builtin_amdgcn_sched_barrier(0);
        auto row_block = [&](auto i_tag) {  // MFMAs of row block I, then the fold of row block I - 1 behind them
            constexpr int I = decltype(i_tag)::value;
            lds_wait_keep_newer<2 * (3 - I)>(af[I][0], af[I][1]);
#pragma unroll
            for (int j = 0; j < 4; ++j) mm(part[I & 1][j], total[I][j], bf[j][0], bf[j][1], af[I][0], af[I][1]);
            if constexpr (kSpread && I <= 2) load_tile_one(std::integral_constant<int, 3 + I>(), s + 2, slot_in);
            if constexpr (SCALED) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) total[I - 1][j][v] = __builtin_fmaf(part[(I - 1) & 1][j][v], f[I - 1], total[I - 1][j][v]);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        row_block(std::integral_constant<int, 1>());
        row_block(std::integral_constant<int, 2>());
        row_block(std::integral_constant<int, 3>());
        if constexpr (SCALED) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) total[3][j][v] = __builtin_fmaf(part[1][j][v], f[3], total[3][j][v]);
        }
        }
        // the tiles of k block s + 1 (issued one block ago) must have landed before anyone reads them; the scale loads
        // and tile loads issued in this block may stay in flight
        wait_older_tiles(all_tag);
        __builtin_amdgcn_s_barrier();
        slot = slot == 2 ? 0 : slot + 1;
    }
    };
    if (a_cnt == 4) k_loop(std::true_type());
    else k_loop(std::false_type());
    // LDS must not be released with tile loads in flight
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));

    if (item.parts > 1) {
        uint32_t rows_valid = 0;  // row blocks of this wave that reach into the matrix
#pragma unroll
        for (int i = 0; i < 4; ++i) rows_valid |= uint32_t(m0 + wm * 64 + i * 16 < m) << i;
        if (!gemm_k_split_fixup<kThreads8>(total, item, partials, counters, &s_last, rows_valid)) return;
    }

    float alpha = 1.0f;
    if constexpr (!SCALED) {
        if (scale_a != nullptr) alpha *= *scale_a;
        if (scale_b != nullptr) alpha *= *scale_b;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = m0 + wm * 64 + i * 16 + ls;
        if (row >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + wn * 64 + j * 16 + 4 * kg;
            if (col >= n) continue;  // n % 4 == 0
            float4_t v = total[i][j];
            if constexpr (!SCALED) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] *= alpha;
            }
            store4_scaled<OUT>(c, int64_t(row) * n + col, v);
        }
    }
}

}  // namespace

// Launch of the 8-wave kernel; SCALED selects block scales (scale_a [K/128, M], scale_b [N/128, K/128]) or optional
// per-tensor scales.
template <bool SCALED, int FMT = 0>
static void launch_kernel8(const void *a, int64_t lda, const void *b, int64_t ldb, const void *scale_a, const void *scale_b,
                           void *c, int64_t m, int64_t n, int64_t k, int out_dtype, void *workspace, int64_t workspace_bytes,
                           hipStream_t stream) {
    const int tiles_m = int(cdiv(m, kM8)), tiles_n = int(cdiv(n, kN8));
    const GemmTiling tiling = make_gemm_tiling(tiles_m, tiles_n, 32);
    // Tail split (tiles that do not fill a round of one workgroup per CU are computed in K ranges and summed in range
    // order by the last workgroup to arrive): at most 4 ranges of at least 4 k blocks, and only with a workspace that
    // holds the partial tiles (8 XCDs x their tail tiles x parts) in its scratch part.
    GemmTail tail = make_gemm_tail(tiling, 32, 32, 4);
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    if (ws.scratch == nullptr) tail.parts = 1;
    while (tail.parts > 1 &&
           (k / 128 < 4 * tail.parts || ws.scratch_bytes < int64_t(8) * tail.max_tiles * tail.parts * kM8 * kN8 * 4))
        --tail.parts;
    const int64_t grid = gemm_grid_with_tail(tiling, 32, tail);
    QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
    auto go = [&](auto kern) {
        allow_dynamic_lds(reinterpret_cast<const void *>(kern), kLdsBytes8);
        launch(kern, dim3(uint32_t(grid)), dim3(kThreads8), size_t(kLdsBytes8), stream, static_cast<const uint8_t *>(a), lda,
               static_cast<const uint8_t *>(b), ldb, static_cast<const float *>(scale_a), static_cast<const float *>(scale_b), c,
               int(m), int(n), int(k), tiles_m, tiles_n, tiling.xm, tiling.xn, tail.parts, tail.max_tiles,
               reinterpret_cast<float *>(ws.scratch), ws.counters);
    };
    constexpr int kOut8 = FMT == 1 ? HIDET_QMM_E5M2 : HIDET_QMM_E4M3;  // the 8-bit output type is the operands' own
    if (out_dtype == HIDET_QMM_F32) go(gemm_fp8_kernel8<HIDET_QMM_F32, SCALED, FMT>);
    else if (out_dtype == HIDET_QMM_F16) go(gemm_fp8_kernel8<HIDET_QMM_F16, SCALED, FMT>);
    else if (out_dtype == HIDET_QMM_BF16) go(gemm_fp8_kernel8<HIDET_QMM_BF16, SCALED, FMT>);
    else if (out_dtype == kOut8) go(gemm_fp8_kernel8<kOut8, SCALED, FMT>);
    else QMM_FAIL("unsupported output dtype code " << out_dtype);
}

// a x b^T with optional per-tensor scales on the 256 x 128, 8-wave kernel. The caller has checked: K a multiple of 128,
// 16-byte aligned rows and pointers, N a multiple of 4, tensors below 1 GiB.
void gemm_fp8_kernel8_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                             int out_dtype, const void *scale_a, const void *scale_b, void *workspace, int64_t workspace_bytes,
                             hipStream_t stream) {
    launch_kernel8<false>(a, lda, b, ldb, scale_a, scale_b, c, m, n, k, out_dtype, workspace, workspace_bytes, stream);
}

template <int FMT>
static void scaled_launch(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m, int64_t n,
                          int64_t k, int out_dtype, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    const bool fast = m * k <= (int64_t(1) << 30) && n * k <= (int64_t(1) << 30) && (k / 128) * m * 4 < (int64_t(1) << 31) &&
                      aligned(a, 16) && aligned(b, 16) && aligned(c, 16);
    if (fast) {
        launch_kernel8<true, FMT>(a, k, b, k, scale_a, scale_b, c, m, n, k, out_dtype, workspace, workspace_bytes, stream);
        return;
    }
    const int tiles_m = int(cdiv(m, kT)), tiles_n = int(n / 128);
    const int64_t grid = int64_t(tiles_m) * tiles_n;
    QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
    auto go = [&](auto kern) {
        launch(kern, dim3(uint32_t(grid)), dim3(kThreads), size_t(kLdsBytes), stream, static_cast<const uint8_t *>(a),
               static_cast<const uint8_t *>(b), static_cast<const float *>(scale_a), static_cast<const float *>(scale_b), c,
               int(m), int(n), int(k), tiles_m);
    };
    constexpr int kOut8 = FMT == 1 ? HIDET_QMM_E5M2 : HIDET_QMM_E4M3;
    if (out_dtype == HIDET_QMM_F32) go(gemm_fp8_scaled_kernel<HIDET_QMM_F32, FMT>);
    else if (out_dtype == HIDET_QMM_F16) go(gemm_fp8_scaled_kernel<HIDET_QMM_F16, FMT>);
    else if (out_dtype == HIDET_QMM_BF16) go(gemm_fp8_scaled_kernel<HIDET_QMM_BF16, FMT>);
    else if (out_dtype == kOut8) go(gemm_fp8_scaled_kernel<kOut8, FMT>);
    else QMM_FAIL("unsupported output dtype code " << out_dtype);
}

// `e5m2`: both operands are float8_e5m2 (the 8-bit output type is then e5m2 as well), else e4m3.
void gemm_fp8_scaled_launch(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m,
                            int64_t n, int64_t k, int out_dtype, bool e5m2, void *workspace, int64_t workspace_bytes,
                            hipStream_t stream) {
    if (e5m2) scaled_launch<1>(a, b, scale_a, scale_b, c, m, n, k, out_dtype, workspace, workspace_bytes, stream);
    else scaled_launch<0>(a, b, scale_a, scale_b, c, m, n, k, out_dtype, workspace, workspace_bytes, stream);
}

}  // namespace qmm
