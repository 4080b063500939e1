// FP8 e4m3 GEMM: c[m, n] = cast(alpha * sum_k a[m, k] * b[n, k]), both operands K-contiguous, fp32
// accumulation on the CDNA4 block-scaled MFMA (v_mfma_scale_f32_16x16x128_f8f6f4 with unit block
// scales, the form that runs fp8 at twice the rate of the plain fp8 MFMA).  alpha = scale_a * scale_b
// (per-tensor float32 scales read from device memory) or 1.
//
// Workgroup tile 256 x 256, four waves of 128 x 128, k-step 128 bytes.  Both operand tiles are staged
// through LDS as rows of 128 bytes = eight 16-byte chunks, XOR-swizzled by row so that the 32-byte
// fragment reads of 16 consecutive rows spread over all banks; two buffers, one barrier per k-step,
// the next step's global loads in flight during the 64 MFMAs of the current one.  The MFMA is issued
// with the b tile as its row operand: a lane then holds 4 consecutive output columns of one row and
// stores them together.
#include "common.h"
#include "gemm_tiling.h"
#include "numeric.h"

namespace qmm {
namespace {

constexpr int kBM = 256, kBN = 256, kBKB = 128;  // tile and k-step in bytes (= fp8 elements)
constexpr int kThreads = 256;
constexpr int kStageChunks = (kBM + kBN) * 8;      // 16-byte chunks per stage (A rows then B rows)
constexpr int kChunksPerThread = kStageChunks / kThreads;  // 16
constexpr int kLdsBytes = 2 * kStageChunks * 16;   // 128 KiB

template <int FMT = kFmtE4M3>
__device__ __forceinline__ float4_t mfma_fp8_k128(const uint4 &r0, const uint4 &r1, const uint4 &c0, const uint4 &c1, float4_t acc) {
    int8v_t rv, cv;
    rv[0] = int(r0.x); rv[1] = int(r0.y); rv[2] = int(r0.z); rv[3] = int(r0.w);
    rv[4] = int(r1.x); rv[5] = int(r1.y); rv[6] = int(r1.z); rv[7] = int(r1.w);
    cv[0] = int(c0.x); cv[1] = int(c0.y); cv[2] = int(c0.z); cv[3] = int(c0.w);
    cv[4] = int(c1.x); cv[5] = int(c1.y); cv[6] = int(c1.z); cv[7] = int(c1.w);
    // formats FMT / FMT: 0 = e4m3, 1 = e5m2 for both operands; block scales 0x7F = 2^0
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rv, cv, acc, FMT, FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
}

template <int OUT>
__device__ __forceinline__ void store4(void *c, int64_t idx, float4_t v) {
    if (OUT == HIDET_QMM_F32) {
        *reinterpret_cast<float4_t *>(static_cast<float *>(c) + idx) = v;
    } else if (OUT == HIDET_QMM_BF16) {
        uint2 o;
        o.x = uint32_t(f32_to_bf16_bits(v[0])) | (uint32_t(f32_to_bf16_bits(v[1])) << 16);
        o.y = uint32_t(f32_to_bf16_bits(v[2])) | (uint32_t(f32_to_bf16_bits(v[3])) << 16);
        *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(c) + idx) = o;
    } else if (OUT == HIDET_QMM_F16) {
        uint2 o;
        o.x = uint32_t(f32_to_f16_bits(v[0])) | (uint32_t(f32_to_f16_bits(v[1])) << 16);
        o.y = uint32_t(f32_to_f16_bits(v[2])) | (uint32_t(f32_to_f16_bits(v[3])) << 16);
        *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(c) + idx) = o;
    } else if (OUT == HIDET_QMM_E5M2) {
        const uint32_t o = uint32_t(f32_to_e5m2(v[0])) | (uint32_t(f32_to_e5m2(v[1])) << 8) |
                           (uint32_t(f32_to_e5m2(v[2])) << 16) | (uint32_t(f32_to_e5m2(v[3])) << 24);
        *reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(c) + idx) = o;
    } else {
        const uint32_t o = uint32_t(f32_to_e4m3(v[0])) | (uint32_t(f32_to_e4m3(v[1])) << 8) |
                           (uint32_t(f32_to_e4m3(v[2])) << 16) | (uint32_t(f32_to_e4m3(v[3])) << 24);
        *reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(c) + idx) = o;
    }
}

template <int OUT, int FMT = kFmtE4M3>
__global__ __launch_bounds__(kThreads, 1) void gemm_fp8_staged_kernel(const uint8_t *__restrict__ a, int64_t lda,
                                                               const uint8_t *__restrict__ b, int64_t ldb,
                                                               void *__restrict__ c, int m, int n, int k,
                                                               const float *__restrict__ scale_a,
                                                               const float *__restrict__ scale_b, int tiles_m, int tiles_n, int xm, int xn) {
    extern __shared__ uint4 lds[];  // [2][kStageChunks]

    int tile_m, tile_n;
    if (!gemm_tile_of_block(tiles_m, tiles_n, xm, xn, &tile_m, &tile_n)) return;
    const int m0 = tile_m * kBM, n0 = tile_n * kBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int kg = lane >> 4, ls = lane & 15;

    float4_t acc[8][8];  // [row block of a][column block of b]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    // staging: chunk id = j * 256 + tid -> tile row id / 8 (A rows 0..255, then B rows 256..511),
    // LDS position id % 8 holds the row's chunk (position ^ (row & 7))
    uint4 stage[kChunksPerThread];
    auto load_stage = [&](int kbase) {
#pragma unroll
        for (int j = 0; j < kChunksPerThread; ++j) {
            const int id = j * kThreads + tid;
            const int row = id >> 3, pos = id & 7;
            const int chunk = pos ^ (row & 7);
            const int kb = kbase + chunk * 16;
            stage[j] = uint4{0u, 0u, 0u, 0u};
            if (j < kChunksPerThread / 2) {
                const int r = m0 + row;
                if (r < m && kb < k) stage[j] = *reinterpret_cast<const uint4 *>(a + int64_t(r) * lda + kb);
            } else {
                const int r = n0 + row - kBM;
                if (r < n && kb < k) stage[j] = *reinterpret_cast<const uint4 *>(b + int64_t(r) * ldb + kb);
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

    const int steps = (k + kBKB - 1) / kBKB;
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        const bool more = s + 1 < steps;
        if (more) load_stage((s + 1) * kBKB);
        const uint4 *la = lds + buf * kStageChunks;
        const uint4 *lb = la + kBM * 8;
        uint4 bf[8][2];  // the 8 column-block fragments of b
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int r = wn * 128 + j * 16 + ls;
            bf[j][0] = lb[r * 8 + ((2 * kg) ^ (r & 7))];
            bf[j][1] = lb[r * 8 + ((2 * kg + 1) ^ (r & 7))];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = wm * 128 + i * 16 + ls;
            const uint4 a0 = la[r * 8 + ((2 * kg) ^ (r & 7))];
            const uint4 a1 = la[r * 8 + ((2 * kg + 1) ^ (r & 7))];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[i][j] = mfma_fp8_k128<FMT>(bf[j][0], bf[j][1], a0, a1, acc[i][j]);
        }
        if (more) store_stage(buf ^ 1);
        __syncthreads();
    }

    // acc[i][j][v] = c[m0 + wm*128 + i*16 + ls][n0 + wn*128 + j*16 + 4*kg + v]
    float alpha = 1.0f;
    if (scale_a != nullptr) alpha *= *scale_a;
    if (scale_b != nullptr) alpha *= *scale_b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = m0 + wm * 128 + i * 16 + ls;
        if (row < m) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int col = n0 + wn * 128 + j * 16 + 4 * kg;
                if (col < n) {  // n % 4 == 0
                    float4_t v = acc[i][j];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] *= alpha;
                    store4<OUT>(c, int64_t(row) * n + col, v);
                }
            }
        }
    }
}

// ---- fast path: K a multiple of 128, 16-byte aligned rows, tensors below 1 GiB -------------------------------
// Same 256x256 tile and swizzled LDS layout, eight waves of 128 x 64 (two per SIMD), and:
//  * both operand tiles go global -> LDS directly (buffer_load ... lds: no staging registers, no ds_write; the
//    chunk swizzle is applied on the global side);
//  * LDS holds a ring of three A tiles and two B tiles (160 KiB). A wave reads all its B fragments of a k-step
//    up front, so a B slot is free again after the first of the eight row blocks; A fragments stream through
//    the step. With two barriers per step - P after row block 0 (B slot free -> issue B of step s+2) and L before
//    the MFMAs of row block 7 (A slot free -> issue A of step s+3; loads of step s+1 confirmed landed) - every
//    load is issued about two k-steps (~4000 MFMA cycles) before its first use;
//  * fragment reads are issued by hand in order of first use, the next step's first fragments during row block
//    7 of the current one, and each wait is tied to the registers it guards.
constexpr int kTileChunks = kBM * 8;  // 16-byte chunks of one 256 x 128-byte operand tile
constexpr int kASlots = 3, kBSlots = 2;
constexpr int kFastLdsBytes = (kASlots + kBSlots) * kTileChunks * 16;  // 160 KiB
static_assert(kBM == kBN, "A and B tiles share the slot size");

// acc += r (8 dwords of 32 fp8 per lane) x c, in place in accumulation registers. Written as asm so that the 256
// accumulator registers of a wave stay where they are (the register allocator otherwise rotates some of them
// through temporaries, with the wait states that costs) and the MFMAs keep their program order. The scale operand
// holds E8M0 ones (0x7F bytes); operand formats default to e4m3.
__device__ __forceinline__ void mfma_fp8_k128v(const int4v_t &r0, const int4v_t &r1, const int4v_t &c0, const int4v_t &c1, float4_t &acc, int unit_scales) {
    const int8v_t rv = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
    const int8v_t cv = __builtin_shufflevector(c0, c1, 0, 1, 2, 3, 4, 5, 6, 7);
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0]" : "+a"(acc) : "v"(rv), "v"(cv), "v"(unit_scales));
}

// Compile-time loop: f(std::integral_constant<int, I>()) for I = BEGIN .. END - 1, in order.
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>());
        static_for<BEGIN + 1, END>(f);
    }
}

// WAVES = 4: waves of 128 x 128 (2 x 2), one per SIMD. WAVES = 8: waves of 128 x 64 (2 x 4), two per SIMD, so that a
// wave stalled on a barrier, an LDS read or a tile load leaves the MFMA unit to the other.
template <int OUT, int WAVES>
__global__ __launch_bounds__(WAVES * 64, 1) void gemm_fp8_kernel(const uint8_t *__restrict__ a, int64_t lda,
                                                                 const uint8_t *__restrict__ b, int64_t ldb,
                                                                 void *__restrict__ c, int m, int n, int k,
                                                                 const float *__restrict__ scale_a,
                                                                 const float *__restrict__ scale_b, int tiles_m, int tiles_n, int xm, int xn) {
    static_assert(WAVES == 4 || WAVES == 8, "2 x 2 or 2 x 4 waves");
    constexpr int kThr = WAVES * 64;
    constexpr int WN = WAVES / 2;          // waves along N
    constexpr int NB = 16 / WN;            // 16-column blocks (B fragments) per wave
    constexpr int kLoads = 2048 / kThr;    // direct-to-LDS loads per thread and operand tile
    extern __shared__ uint4 lds[];  // [kASlots][kTileChunks] A ring, then [kBSlots][kTileChunks] B ring

    int tile_m, tile_n;
    if (!gemm_tile_of_block(tiles_m, tiles_n, xm, xn, &tile_m, &tile_n)) return;
    const int m0 = tile_m * kBM, n0 = tile_n * kBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int kg = lane >> 4, ls = lane & 15;

    float4_t acc[8][NB];  // [row block of a][column block of b]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(a), 0, int(int64_t(m - 1) * lda + k), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(b), 0, int(int64_t(n - 1) * ldb + k), 0x00020000);
    // Load instruction j of a wave fills chunk slots j * kThr + wave * 64 .. + 63 of a tile: tile row
    // j * kThr / 8 + tid / 8, position tid % 8, which holds chunk (tid % 8) ^ lds_swizzle_key_step2(row). Rows past the
    // end of the tensor get an offset outside the buffer and read as zero.
    constexpr int kOutside = 0x7FFFFFF0;
    const int chunk = (tid & 7) ^ lds_swizzle_key_step2(tid >> 3);  // j * kThr / 8 is a multiple of 16: same key
    int voff_a[kLoads], voff_b[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
        const int ra = m0 + j * (kThr / 8) + (tid >> 3), rb = n0 + j * (kThr / 8) + (tid >> 3);
        voff_a[j] = ra < m ? int(int64_t(ra) * lda) + chunk * 16 : kOutside;
        voff_b[j] = rb < n ? int(int64_t(rb) * ldb) + chunk * 16 : kOutside;
    }
    const int steps = k / kBKB;
    // The scalar offset is not part of the buffer's range check: a prefetch past the end of K re-reads the last step
    // (what it fetches is never used). A tile load is kLoads instructions per wave; the loop issues them one quarter
    // (QUARTER = 0 .. 3) at a time, one quarter per row block, so that no wave ever queues a burst of loads in front of
    // its MFMAs (issued as a burst right behind a barrier, when all eight waves do the same, the loads cost a quarter
    // of the kernel's time in issue stalls).
    static_assert(kLoads % 4 == 0, "tile loads are issued in quarters");
    auto load_a_quarter = [&](auto quarter_tag, int step, int slot) {
        constexpr int Q = decltype(quarter_tag)::value;
        const int soff = (step < steps ? step : steps - 1) * kBKB;
        uint4 *dst = lds + slot * kTileChunks + wave * 64;
#pragma unroll
        for (int j = Q * (kLoads / 4); j < (Q + 1) * (kLoads / 4); ++j) buffer_load_to_lds_b128(rsrc_a, dst + j * kThr, voff_a[j], soff);
    };
    auto load_b_quarter = [&](auto quarter_tag, int step, int slot) {
        constexpr int Q = decltype(quarter_tag)::value;
        const int soff = (step < steps ? step : steps - 1) * kBKB;
        uint4 *dst = lds + (kASlots + slot) * kTileChunks + wave * 64;
#pragma unroll
        for (int j = Q * (kLoads / 4); j < (Q + 1) * (kLoads / 4); ++j) buffer_load_to_lds_b128(rsrc_b, dst + j * kThr, voff_b[j], soff);
    };
    auto load_a = [&](int step, int slot) {
        static_for<0, 4>([&](auto qt) { load_a_quarter(qt, step, slot); });
    };
    auto load_b = [&](int step, int slot) {
        static_for<0, 4>([&](auto qt) { load_b_quarter(qt, step, slot); });
    };

    // LDS byte addresses of this lane's two 16-byte fragment halves in block 0 of its wave, slot 0 of each ring;
    // block i adds i * 16 rows = i * 2048 bytes
    uint32_t a_addr[2], b_addr[2];
    {
        const int ra = wm * 128 + ls, rb = wn * (NB * 16) + ls;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            a_addr[h] = uint32_t((ra * 8 + ((2 * kg + h) ^ lds_swizzle_key_step2(ra))) * 16);
            b_addr[h] = uint32_t(((kASlots * kBM + rb) * 8 + ((2 * kg + h) ^ lds_swizzle_key_step2(rb))) * 16);
        }
    }
    constexpr uint32_t kSlotBytes = kTileChunks * 16;

    // Issue order of the tile loads (A ring: 3 slots, B ring: 2): the A tile of step s + 3 goes out one quarter each in
    // row block 7 of step s (behind barrier L, which frees its slot) and row blocks 0, 1, 2 of step s + 1; the B tile of
    // step s + 2 one quarter each in row blocks 3 .. 6 of step s (behind barrier P, which frees its slot).
    load_a(0, 0);
    load_b(0, 0);
    load_a(1, 1);
    load_b(1, 1);
    load_a_quarter(std::integral_constant<int, 0>(), 2, 2);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * kLoads + kLoads / 4));
    __builtin_amdgcn_s_barrier();

    int4v_t bf[NB][2], af[3][2];
    // row block i of a step keeps its A fragment in af[i % 3]. First reads in order of first use: b0, a0, b1 ..
    bf[0][0] = lds_read_b128_early<0>(b_addr[0]);
    bf[0][1] = lds_read_b128_early<0>(b_addr[1]);
    af[0][0] = lds_read_b128_early<0>(a_addr[0]);
    af[0][1] = lds_read_b128_early<0>(a_addr[1]);
    static_for<1, NB>([&](auto jt) {
        constexpr int J = decltype(jt)::value;
        bf[J][0] = lds_read_b128_early<J * 2048>(b_addr[0]);
        bf[J][1] = lds_read_b128_early<J * 2048>(b_addr[1]);
    });

    int unit_scales;
    asm volatile("v_mov_b32 %0, 0x7f7f7f7f" : "=v"(unit_scales));
    int a_slot = 0, b_slot = 0;  // ring slots of the current step
    for (int s = 0; s < steps; ++s) {
        const uint32_t aa0 = a_addr[0] + uint32_t(a_slot) * kSlotBytes, aa1 = a_addr[1] + uint32_t(a_slot) * kSlotBytes;
        const int a_next = a_slot == kASlots - 1 ? 0 : a_slot + 1, b_next = b_slot ^ 1;
        const int a_prev = a_slot == 0 ? kASlots - 1 : a_slot - 1;  // freed by barrier L of the previous step: takes step s + 2

        // ---- row block 0: the reads outstanding are a0, b0 .. b(NB-1) of this step (in either order of a0 and b0);
        // the B fragments arrive one by one, a1 is requested behind the first MFMA
        lds_wait_keep_newer<2 * (NB - 1)>(bf[0][0], bf[0][1]);
        lds_wait_keep_newer<2 * (NB - 1)>(af[0][0], af[0][1]);
        mfma_fp8_k128v(bf[0][0], bf[0][1], af[0][0], af[0][1], acc[0][0], unit_scales);
        load_a_quarter(std::integral_constant<int, 1>(), s + 2, a_prev);
        af[1][0] = lds_read_b128_early<1 * 2048>(aa0);
        af[1][1] = lds_read_b128_early<1 * 2048>(aa1);
        static_for<1, NB>([&](auto jt) {
            constexpr int J = decltype(jt)::value;
            lds_wait_keep_newer<2 * (NB - 1 - J) + 2>(bf[J][0], bf[J][1]);
            mfma_fp8_k128v(bf[J][0], bf[J][1], af[0][0], af[0][1], acc[0][J], unit_scales);
            __builtin_amdgcn_sched_barrier(0);
        });
        // barrier P: every wave holds all B fragments of this step, so its B slot can take step s + 2
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        // ---- row blocks 1 .. 6
        static_for<1, 7>([&](auto it) {
            constexpr int I = decltype(it)::value;
            af[(I + 1) % 3][0] = lds_read_b128_early<(I + 1) * 2048>(aa0);
            af[(I + 1) % 3][1] = lds_read_b128_early<(I + 1) * 2048>(aa1);
            lds_wait_keep_newer<2>(af[I % 3][0], af[I % 3][1]);
            mfma_fp8_k128v(bf[0][0], bf[0][1], af[I % 3][0], af[I % 3][1], acc[I][0], unit_scales);
            if constexpr (I <= 2) load_a_quarter(std::integral_constant<int, I + 1>(), s + 2, a_prev);
            else load_b_quarter(std::integral_constant<int, I - 3>(), s + 2, b_slot);
#pragma unroll
            for (int j = 1; j < NB; ++j) mfma_fp8_k128v(bf[j][0], bf[j][1], af[I % 3][0], af[I % 3][1], acc[I][j], unit_scales);
            __builtin_amdgcn_sched_barrier(0);
        });

        // ---- row block 7. Barrier L: every wave has read all of this step's A slot, so it can take step s + 3,
        // and every wave's loads of step s + 1 have landed (the newer ones, A of s + 2 and B of s + 2, may still be
        // in flight), so the first fragments of step s + 1 can be fetched behind this block's MFMAs.
        lds_wait_keep_newer<0>(af[1][0], af[1][1]);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * kLoads));
        __builtin_amdgcn_s_barrier();
        load_a_quarter(std::integral_constant<int, 0>(), s + 3, a_slot);
        __builtin_amdgcn_sched_barrier(0);
        {
            const uint32_t na0 = a_addr[0] + uint32_t(a_next) * kSlotBytes, na1 = a_addr[1] + uint32_t(a_next) * kSlotBytes;
            const uint32_t nb0 = b_addr[0] + uint32_t(b_next) * kSlotBytes, nb1 = b_addr[1] + uint32_t(b_next) * kSlotBytes;
            af[0][0] = lds_read_b128_early<0>(na0);
            af[0][1] = lds_read_b128_early<0>(na1);
            static_for<0, NB>([&](auto jt) {
                constexpr int J = decltype(jt)::value;
                mfma_fp8_k128v(bf[J][0], bf[J][1], af[1][0], af[1][1], acc[7][J], unit_scales);
                bf[J][0] = lds_read_b128_early<J * 2048>(nb0);
                bf[J][1] = lds_read_b128_early<J * 2048>(nb1);
            });
        }
        __builtin_amdgcn_sched_barrier(0);
        a_slot = a_next;
        b_slot = b_next;
    }
    // drain: the look-ahead fragment reads of the step past the end are never used, but their destination
    // registers must not be reused before they have landed (the waits name every one of them), and LDS must
    // not be released with tile loads in flight
    lds_wait_keep_newer<0>(af[0][0], af[0][1]);
#pragma unroll
    for (int j = 0; j < NB; ++j) lds_wait_keep_newer<0>(bf[j][0], bf[j][1]);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    // the compiler does not see the MFMAs inside the asm: let the last ones retire before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    // acc[i][j][v] = c[m0 + wm*128 + i*16 + ls][n0 + wn*NB*16 + j*16 + 4*kg + v]
    float alpha = 1.0f;
    if (scale_a != nullptr) alpha *= *scale_a;
    if (scale_b != nullptr) alpha *= *scale_b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = m0 + wm * 128 + i * 16 + ls;
        if (row < m) {
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int col = n0 + wn * (NB * 16) + j * 16 + 4 * kg;
                if (col < n) {  // n % 4 == 0
                    float4_t v = acc[i][j];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] *= alpha;
                    store4<OUT>(c, int64_t(row) * n + col, v);
                }
            }
        }
    }
}

// Fallback for shapes the tiled kernel cannot take: one thread per output element.
template <int OUT, int FMT = kFmtE4M3>
__global__ __launch_bounds__(256) void naive_fp8_kernel(const uint8_t *__restrict__ a, int64_t lda, const uint8_t *__restrict__ b,
                                                        int64_t ldb, void *__restrict__ c, int64_t m, int64_t n, int64_t k,
                                                        const float *__restrict__ scale_a, const float *__restrict__ scale_b) {
    const int64_t o = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (o >= m * n) return;
    const int64_t i = o / n, j = o - i * n;
    float acc = 0.f;
    for (int64_t kk = 0; kk < k; ++kk) acc += fp8_to_f32<FMT>(a[i * lda + kk]) * fp8_to_f32<FMT>(b[j * ldb + kk]);
    if (scale_a != nullptr) acc *= (*scale_a) * (scale_b != nullptr ? *scale_b : 1.0f);
    else if (scale_b != nullptr) acc *= *scale_b;
    store_out<OUT>(c, o, acc);
}

template <typename F>
void dispatch_out(int out_dtype, F &&f) {
    switch (out_dtype) {
        case HIDET_QMM_F32: f(std::integral_constant<int, HIDET_QMM_F32>()); break;
        case HIDET_QMM_F16: f(std::integral_constant<int, HIDET_QMM_F16>()); break;
        case HIDET_QMM_BF16: f(std::integral_constant<int, HIDET_QMM_BF16>()); break;
        case HIDET_QMM_E4M3: f(std::integral_constant<int, HIDET_QMM_E4M3>()); break;
        default: QMM_FAIL("unsupported output dtype code " << out_dtype);
    }
}

// float8_e5m2 operands: the register-staged tile kernel with the MFMA's bf8 format, or the element-wise kernel
template <typename F>
void dispatch_out_e5m2(int out_dtype, F &&f) {
    switch (out_dtype) {
        case HIDET_QMM_F32: f(std::integral_constant<int, HIDET_QMM_F32>()); break;
        case HIDET_QMM_F16: f(std::integral_constant<int, HIDET_QMM_F16>()); break;
        case HIDET_QMM_BF16: f(std::integral_constant<int, HIDET_QMM_BF16>()); break;
        case HIDET_QMM_E5M2: f(std::integral_constant<int, HIDET_QMM_E5M2>()); break;
        default: QMM_FAIL("unsupported output dtype code " << out_dtype << " for float8_e5m2 operands");
    }
}

}  // namespace

void gemm_fp8_e5m2_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                          int out_dtype, const void *scale_a, const void *scale_b, hipStream_t stream) {
    const uint8_t *ap = static_cast<const uint8_t *>(a), *bp = static_cast<const uint8_t *>(b);
    const float *sa = static_cast<const float *>(scale_a), *sb = static_cast<const float *>(scale_b);
    const bool tiled = (k % 16 == 0) && (lda % 16 == 0) && (ldb % 16 == 0) && (n % 4 == 0) && aligned(a, 16) &&
                       aligned(b, 16) && aligned(c, 16) && k > 0;
    dispatch_out_e5m2(out_dtype, [&](auto o) {
        constexpr int OUT = decltype(o)::value;
        if (!tiled) {
            launch(naive_fp8_kernel<OUT, kFmtE5M2>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap, lda, bp, ldb, c, m, n, k, sa, sb);
            return;
        }
        const int tiles_m = int(cdiv(m, kBM)), tiles_n = int(cdiv(n, kBN));
        const GemmTiling tiling = make_gemm_tiling(tiles_m, tiles_n, 32);
        const int64_t grid = tiling.grid();
        QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
        allow_dynamic_lds(reinterpret_cast<const void *>(gemm_fp8_staged_kernel<OUT, kFmtE5M2>), kLdsBytes);
        launch(gemm_fp8_staged_kernel<OUT, kFmtE5M2>, dim3(uint32_t(grid)), dim3(kThreads), size_t(kLdsBytes), stream, ap, lda, bp,
               ldb, c, int(m), int(n), int(k), sa, sb, tiles_m, tiles_n, tiling.xm, tiling.xn);
    });
}

void gemm_fp8_kernel8_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                             int out_dtype, const void *scale_a, const void *scale_b, void *workspace, int64_t workspace_bytes,
                             hipStream_t stream);

void gemm_fp8_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                     int out_dtype, const void *scale_a, const void *scale_b, void *workspace, int64_t workspace_bytes,
                     hipStream_t stream) {
    const uint8_t *ap = static_cast<const uint8_t *>(a), *bp = static_cast<const uint8_t *>(b);
    const float *sa = static_cast<const float *>(scale_a), *sb = static_cast<const float *>(scale_b);
    const bool tiled = (k % 16 == 0) && (lda % 16 == 0) && (ldb % 16 == 0) && (n % 4 == 0) && aligned(a, 16) &&
                       aligned(b, 16) && aligned(c, 16) && k > 0;
    dispatch_out(out_dtype, [&](auto o) {
        constexpr int OUT = decltype(o)::value;
        if (!tiled) {
            launch(naive_fp8_kernel<OUT>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap, lda, bp, ldb, c, m, n, k, sa, sb);
            return;
        }
        const int tiles_m = int(cdiv(m, kBM)), tiles_n = int(cdiv(n, kBN));
        const GemmTiling tiling = make_gemm_tiling(tiles_m, tiles_n, 32);
        const int64_t grid = tiling.grid();
        QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
        const bool fast = (k % kBKB == 0) && (m - 1) * lda + k <= (int64_t(1) << 30) &&
                          (n - 1) * ldb + k <= (int64_t(1) << 30);
        if (fast) {
            // 256 x 256 tiles move the fewest bytes per flop; 256 x 128 tiles cost about 15 % more per flop but come in
            // twice as many pieces. Take whichever needs less time in rounds of one workgroup per CU (measured: 4096^3 60
            // vs 70 us, 2048 x 4096 x 11008 108 vs 101 us, 1024 x 8192 x 8192 91 vs 65 us).
            const int64_t t256 = int64_t(tiles_m) * tiles_n, t128 = int64_t(tiles_m) * cdiv(n, 128);
            const double cost256 = double(cdiv(t256, 256)), cost128 = double(cdiv(t128, 256)) * 0.5 * 1.15;
            if (cost128 < cost256) {
                gemm_fp8_kernel8_launch(a, b, c, m, n, k, lda, ldb, out_dtype, scale_a, scale_b, workspace, workspace_bytes, stream);
                return;
            }
            allow_dynamic_lds(reinterpret_cast<const void *>(gemm_fp8_kernel<OUT, 8>), kFastLdsBytes);
            launch(gemm_fp8_kernel<OUT, 8>, dim3(uint32_t(grid)), dim3(512), size_t(kFastLdsBytes), stream, ap, lda, bp, ldb, c,
                   int(m), int(n), int(k), sa, sb, tiles_m, tiles_n, tiling.xm, tiling.xn);
            return;
        }
        allow_dynamic_lds(reinterpret_cast<const void *>(gemm_fp8_staged_kernel<OUT>), kLdsBytes);
        launch(gemm_fp8_staged_kernel<OUT>, dim3(uint32_t(grid)), dim3(kThreads), size_t(kLdsBytes), stream, ap, lda, bp, ldb, c,
               int(m), int(n), int(k), sa, sb, tiles_m, tiles_n, tiling.xm, tiling.xn);
    });
}

}  // namespace qmm
