// W8A16 prefill GEMM (M > 16): c[m, n] = (sum_k a[m, k] * w[k, n]) * scale[n] on fp16 MFMA with fp32
// accumulation.
//
// The int8 weights never pass through LDS.  Lane (kg, ns) of a wave (kg = lane / 16, ns = lane % 16)
// loads rows 8kg .. 8kg+7 of a 32-row k-step at columns 4ns .. 4ns+3 (one dword per row); that 8x4
// byte block holds, for each of its 4 columns, the 8 consecutive k values a 16x16x32 MFMA wants as
// the B operand of output column slot ns.  Byte t of two rows is gathered with one v_perm_b32, one
// v_xor_b32 turns the pair into two float16 values (0x6400 | (q ^ 0x80) == 1152 + q) and one packed
// subtract removes the 1152, so the dequantisation is exact and costs 3 VALU ops per 2 weights.  A
// wave owns 128 rows x 64 columns of the output (128 accumulator registers, two workgroups per CU, so
// that the second wave of each SIMD runs its MFMAs while the first one dequantises or waits); every
// dequantised fragment is reused for 8 row blocks.
//
// The inner loop is laid out by hand in blocks of 4 MFMAs: each block issues the LDS read of the A
// fragment three blocks ahead (inline ds_read_b128 + a wait tied to the destination registers), does its
// share of the next k-step's dequantisation (two column pairs) and weight refills, and runs its MFMAs.
// All global reads are buffer loads (scalar base + per-lane constant offset + scalar k offset): no address
// arithmetic in the loop, and out-of-range rows read as zero.  Weight rows are refilled one stage (64 k)
// ahead into the registers they were just dequantised from.  The activation tile goes global -> LDS
// directly (buffer_load ... lds, no registers) into a three-slot ring of 16-byte chunks XOR-swizzled by
// row (the swizzle is applied on the global side), two stages ahead; one barrier per 64 k.  The per-column
// scale is applied to the fp32 accumulators in the epilogue.  Matrices of at most 96 rows run the same tile with the
// row blocks that cannot hold a row left out at compile time (template parameter RBA).
#include "common.h"
#include "gemm_tiling.h"

namespace qmm {
namespace {

constexpr int kBK = 64;  // k extent of one pipeline stage (four 16-deep MFMA steps)

template <int RB, int WM, int WN>
struct GemmW8Cfg16 {
    static constexpr int kBM = WM * RB * 16;
    static constexpr int kBN = WN * 64;
    static constexpr int kThreads = WM * WN * 64;
    static constexpr int kAChunks = kBM * 8 / kThreads;
    static constexpr int kRingBytes = 3 * kBM * 128;  // three-slot ring filled by direct-to-LDS loads
    static constexpr int kLdsBytes = kRingBytes + 16;  // + the fix-up's flag; the ring must start at LDS address 0
};

// RBA <= RB: row blocks (of 16 rows) per wave that can hold rows of the matrix. A short matrix (M <= 16 RBA) runs the same
// tile with the activation loads, fragment reads and MFMAs of the other row blocks left out.
// W_NK: the weight is stored K-contiguous, w[col * ldw + k] (the [N, K] storage of nn.Linear); a lane then loads the 8
// consecutive k of one of its 4 columns with one 8-byte load and widens byte pairs instead of gathering rows.
template <int RB, int WM, int WN, int MIN_BLOCKS, int RBA, bool W_NK = false>
__global__ __launch_bounds__(WM * WN * 64, MIN_BLOCKS) void gemm_w8a16_kernel16(const _Float16 *__restrict__ a, int64_t lda,
                                                                                 const int8_t *__restrict__ w, int64_t ldw,
                                                                                 const _Float16 *__restrict__ scale,
                                                                                 const _Float16 *__restrict__ bias,
                                                                                 _Float16 *__restrict__ c, int m, int k, int n,
                                                                                 int tiles_m, int tiles_n, int xm, int xn,
                                                                                 int concurrent, int tail_parts, int tail_stride,
                                                                                 float *__restrict__ partials,
                                                                                 uint32_t *__restrict__ counters) {
    using Cfg = GemmW8Cfg16<RB, WM, WN>;
    extern __shared__ uint4 lds[];  // no static LDS in this kernel: fragment reads address the ring from 0
    int &s_last = *reinterpret_cast<int *>(lds + Cfg::kRingBytes / 16);

    GemmWorkItem item;
    if (!gemm_work_item(tiles_m, tiles_n, xm, xn, concurrent, tail_parts, tail_stride, &item)) return;
    const int tile_m = item.tile_m, tile_n = item.tile_n, part = item.part, parts = item.parts;
    const int m0 = tile_m * Cfg::kBM;
    const int n0 = tile_n * Cfg::kBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int kg = lane >> 4, ns = lane & 15;
    const int col = n0 + wn * 64 + ns * 4;
    const bool col_ok = col < n;

    float4_t acc[RB][4];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[rb][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(w), 0, W_NK ? int(int64_t(n - 1) * ldw + k) : int(int64_t(k) * n), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(a), 0, int((int64_t(m - 1) * lda + k) * 2), 0x00020000);

    // A staging by direct-to-LDS loads: instruction j of a wave fills the 64 consecutive 16-byte LDS slots
    // (j * kThreads + wave * 64 .. + 63); slot id holds chunk ((id % 8) ^ lds_swizzle_key_step1(row)) of tile row id / 8, so
    // the swizzle is applied on the global side.  Rows past M point outside the buffer and read as zero.
    int a_off[Cfg::kAChunks];
#pragma unroll
    for (int j = 0; j < Cfg::kAChunks; ++j) {
        const int id = j * Cfg::kThreads + tid;
        const int r = id >> 3;
        const int row = m0 + r;
        a_off[j] = row < m ? int((int64_t(row) * lda + ((id & 7) ^ lds_swizzle_key_step1(r)) * 8) * 2) : 0x7FFFFFF0;
    }
    // row-major: row 8 kg + j of a k-step, 4 columns; K-contiguous: column col + t, the 8 k of lane group kg
    int w_off[W_NK ? 4 : 8];
#pragma unroll
    for (int j = 0; j < (W_NK ? 4 : 8); ++j)
        w_off[j] = !col_ok ? 0x7FFFFFF0 : W_NK ? int(int64_t(col + j) * ldw) + kg * 8 : (kg * 8 + j) * n + col;
    constexpr int kWLoadsPerStage = W_NK ? 8 : 16;  // weight load instructions of one stage
    constexpr uint32_t kPairLo = 0x0c010c00u, kPairHi = 0x0c030c02u;  // bytes (0, 1) / (2, 3) of a dword into two halves

    const int stages = k / kBK;
    const int s_begin = (stages * part) / parts, s_end = (stages * (part + 1)) / parts;

    uint32_t w_raw[2][8];  // raw rows of the two k-steps of a stage; each slot is refilled one stage ahead once dequantised
    union BFrag {
        uint32_t u[4];
        half2_t h2[4];
        half8_t h8;
    };
    BFrag bq[2][4];

    // instruction j brings tile rows j * kThreads / 8 ..: only those below 16 RBA are needed
    static_assert(WM == 1 && (RBA * 16 * 8) % Cfg::kThreads == 0, "whole load instructions per active row range");
    constexpr int kAChunksActive = RBA * 16 * 8 / Cfg::kThreads;
    auto load_a = [&](int st, int slot) {
#pragma unroll
        for (int j = 0; j < kAChunksActive; ++j)
            buffer_load_to_lds_b128(rsrc_a, lds + slot * Cfg::kBM * 8 + j * Cfg::kThreads + wave * 64, a_off[j],
                                    (st < stages ? st : stages - 1) * (kBK * 2));  // the scalar offset is not range-checked
    };
    auto load_w = [&](int st, int q, uint32_t (&dst)[8]) {
        if constexpr (W_NK) {
            const int soff = (st < stages ? st : stages - 1) * kBK + q * 32;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, w_off[t], soff, 0);
                dst[2 * t] = v[0];
                dst[2 * t + 1] = v[1];
            }
        } else {
            const int soff = ((st < stages ? st : stages - 1) * kBK + q * 32) * n;
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[j] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_w, w_off[j], soff, 0);
        }
    };
    auto dequant = [&](const uint32_t (&raw)[8], BFrag (&dst)[4]) {
        if constexpr (W_NK) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const uint32_t src = raw[2 * t + p / 2];
                    dst[t].u[p] = __builtin_amdgcn_perm(src, src, (p & 1) ? kPairHi : kPairLo) ^ 0x64806480u;
                    dst[t].h2[p] = dst[t].h2[p] - half2_t{_Float16(1152.0f), _Float16(1152.0f)};
                }
            return;
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            constexpr uint32_t kZero = 0x0c;
            const uint32_t sel = (kZero << 24) | (uint32_t(4 + t) << 16) | (kZero << 8) | uint32_t(t);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                dst[t].u[p] = __builtin_amdgcn_perm(raw[2 * p + 1], raw[2 * p], sel) ^ 0x64806480u;
                dst[t].h2[p] = dst[t].h2[p] - half2_t{_Float16(1152.0f), _Float16(1152.0f)};
            }
        }
    };

    // LDS byte address of this lane's A fragment for row block 0 of its wave, k-step 0 / 1, in ring slot 0; row block
    // rb adds rb * 16 rows = rb * 2048 bytes (the row swizzle repeats every 8 rows), slot adds slot * kBM * 128
    uint32_t af_addr[2];
    {
        const int r = wm * RB * 16 + ns;
#pragma unroll
        for (int q = 0; q < 2; ++q) af_addr[q] = uint32_t((r * 8 + ((q * 4 + kg) ^ lds_swizzle_key_step1(r))) * 16);
    }
    auto stage = [&](int s, int slot) {
        load_a(s + 2, slot >= 1 ? slot - 1 : 2);  // slot (s + 2) % 3: last read in stage s - 1
        const uint32_t slot_off = uint32_t(slot * Cfg::kBM * 128);
        const uint32_t addr0 = af_addr[0] + slot_off, addr1 = af_addr[1] + slot_off;
        // A fragments are read from LDS three fragments (12 MFMAs) ahead of their use, through a ring of four
        // (fragment index = k-step * RBA + row block, over the active row blocks only)
        int4v_t af[4];
        auto issue = [&](auto idx_tag) {
            constexpr int IDX = decltype(idx_tag)::value;
            if constexpr (IDX < 2 * RBA) af[IDX & 3] = lds_read_b128_early<(IDX % RBA) * 2048>(IDX / RBA ? addr1 : addr0);
        };
        issue(std::integral_constant<int, 0>());
        issue(std::integral_constant<int, 1>());
        issue(std::integral_constant<int, 2>());
        // One block = one A fragment: issue the LDS read three fragments ahead, do this block's share of the next
        // k-step's dequantisation (two column pairs) and weight refills, then wait for the fragment and run its 4 MFMAs.
        auto block = [&](auto idx_tag) {
            constexpr int IDX = decltype(idx_tag)::value;
            constexpr int Q = IDX / RB, RBI = IDX % RB;
            constexpr int AI = Q * RBA + RBI;  // fragment index, if the row block is active
            if constexpr (RBI < RBA) issue(std::integral_constant<int, AI + 3>());
            if constexpr (W_NK) {
                constexpr int T = RBI / 2;  // column of the next k-step's block; this block widens one of its two dwords
                const uint32_t src = w_raw[Q ^ 1][2 * T + (RBI & 1)];
                BFrag &dst = bq[Q ^ 1][T];
#pragma unroll
                for (int pp = 0; pp < 2; ++pp) {
                    constexpr int kFirst = 2 * (RBI & 1);
                    dst.u[kFirst + pp] = __builtin_amdgcn_perm(src, src, pp ? kPairHi : kPairLo) ^ 0x64806480u;
                    dst.h2[kFirst + pp] = dst.h2[kFirst + pp] - half2_t{_Float16(1152.0f), _Float16(1152.0f)};
                }
                if constexpr (RBI & 1) {  // both dwords of column T are consumed: refill them one stage ahead
                    const int st = Q == 0 ? s + 1 : s + 2;
                    const int soff = (st < stages ? st : stages - 1) * kBK + (Q ^ 1) * 32;
                    const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, w_off[T], soff, 0);
                    w_raw[Q ^ 1][2 * T] = v[0];
                    w_raw[Q ^ 1][2 * T + 1] = v[1];
                }
            } else {
                constexpr int P = RBI / 2;  // row pair of the next k-step's raw block
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    constexpr uint32_t kZero = 0x0c;
                    const int t = 2 * (RBI & 1) + tt;
                    const uint32_t sel = (kZero << 24) | (uint32_t(4 + t) << 16) | (kZero << 8) | uint32_t(t);
                    BFrag &dst = bq[Q ^ 1][t];
                    dst.u[P] = __builtin_amdgcn_perm(w_raw[Q ^ 1][2 * P + 1], w_raw[Q ^ 1][2 * P], sel) ^ 0x64806480u;
                    dst.h2[P] = dst.h2[P] - half2_t{_Float16(1152.0f), _Float16(1152.0f)};
                }
                if constexpr (RBI & 1) {  // rows 2P and 2P+1 are consumed: refill them with the rows one stage ahead
                    // the scalar offset is not part of the buffer's range check: a prefetch for a stage past the end
                    // re-reads the last stage instead (its values are not used)
                    const int st = Q == 0 ? s + 1 : s + 2;
                    const int soff = ((st < stages ? st : stages - 1) * kBK + (Q ^ 1) * 32) * n;
                    w_raw[Q ^ 1][2 * P] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_w, w_off[2 * P], soff, 0);
                    w_raw[Q ^ 1][2 * P + 1] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_w, w_off[2 * P + 1], soff, 0);
                }
            }
            if constexpr (RBI < RBA) {
                constexpr int NEWER = (2 * RBA - 1 - AI) < 3 ? (2 * RBA - 1 - AI) : 3;
                lds_wait_keep_newer<NEWER>(af[AI & 3]);
                const half8_t afrag = __builtin_bit_cast(half8_t, af[AI & 3]);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc[RBI][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag, bq[Q][t].h8, acc[RBI][t], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        auto kstep = [&](auto q_tag) {
            constexpr int Q = decltype(q_tag)::value;
            static_assert(RB == 8, "the dequantisation is spread over 8 blocks per k-step");
            block(std::integral_constant<int, Q * RB + 0>());
            block(std::integral_constant<int, Q * RB + 1>());
            block(std::integral_constant<int, Q * RB + 2>());
            block(std::integral_constant<int, Q * RB + 3>());
            block(std::integral_constant<int, Q * RB + 4>());
            block(std::integral_constant<int, Q * RB + 5>());
            block(std::integral_constant<int, Q * RB + 6>());
            block(std::integral_constant<int, Q * RB + 7>());
        };
        kstep(std::integral_constant<int, 0>());
        kstep(std::integral_constant<int, 1>());
        // the loads of stage s + 1 (issued one stage ago) must have landed in LDS before anyone reads them; the
        // loads issued during this stage (kAChunksActive + kWLoadsPerStage of them) may stay in flight
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(kAChunksActive + kWLoadsPerStage));
        __syncthreads();
    };

    load_a(s_begin, 0);
    load_a(s_begin + 1, 1);
    load_w(s_begin, 0, w_raw[0]);
    load_w(s_begin, 1, w_raw[1]);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    dequant(w_raw[0], bq[0]);
    load_w(s_begin + 1, 0, w_raw[0]);
    __syncthreads();

    for (int s = s_begin, slot = 0; s < s_end; ++s) {
        stage(s, slot);
        slot = slot == 2 ? 0 : slot + 1;
    }
    // the activation loads issued for stages past the end are never read, but LDS must not be released with them in flight
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));

    // a tile computed in K ranges is finished by the part that arrives last (gemm_k_split_fixup)
    if (parts > 1) {
        uint32_t rows_valid = 0;  // row blocks of this wave that reach into the matrix
#pragma unroll
        for (int rb = 0; rb < RBA; ++rb) rows_valid |= uint32_t(m0 + (wm * RB + rb) * 16 < m) << rb;
        // only the active row blocks take part (every workgroup of a launch has the same RBA)
        if (!gemm_k_split_fixup<Cfg::kThreads>(reinterpret_cast<float4_t(&)[RBA][4]>(acc), item, partials, counters, &s_last,
                                               rows_valid))
            return;
    }

    // acc[rb][t][v] = c[m0 + (wm*RB + rb)*16 + 4*kg + v][col + t]
    if (!col_ok) return;
    float sc[4], bs[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        sc[t] = float(scale[col + t]);
        bs[t] = bias != nullptr ? float(bias[col + t]) : -0.0f;
    }
#pragma unroll
    for (int rb = 0; rb < RBA; ++rb)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = m0 + (wm * RB + rb) * 16 + kg * 4 + v;
            if (row < m) {
                half4_t o;
#pragma unroll
                for (int t = 0; t < 4; ++t) o[t] = scaled_biased_f16(acc[rb][t][v], sc[t], bs[t]);
                *reinterpret_cast<half4_t *>(c + int64_t(row) * n + col) = o;
            }
        }
}

template <int RB, int WM, int WN, int MIN_BLOCKS, int RBA, bool W_NK = false>
void launch_cfg16(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k, int64_t n,
                  int64_t lda, int64_t ldw, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    using Cfg = GemmW8Cfg16<RB, WM, WN>;
    const int tiles_m = int(cdiv(m, Cfg::kBM)), tiles_n = int(cdiv(n, Cfg::kBN));
    constexpr int kConcurrent = 32 * MIN_BLOCKS;  // workgroups an XCD (32 CUs) runs at a time
    const GemmTiling tiling = make_gemm_tiling(tiles_m, tiles_n, kConcurrent);
    // Tail split: at most 4 K ranges of at least 8 stages each, and only with workspace for the partial tiles
    // (8 XCDs x their tail tiles x parts) in the scratch part of the workspace.
    // (light workgroups - at most 4 active row blocks - are worth up to 8 ranges: measured)
    GemmTail tail = make_gemm_tail(tiling, kConcurrent, 32, RBA <= 4 ? 8 : 4);
    // Full tiles: count rounds of one workgroup per CU. The tiles past a whole number of such rounds share their CUs
    // with another workgroup or run in a round of their own; cut into K ranges they finish sooner when they are few
    // (K = 4096, N = 11008: M = 768 / 896 / 1024: 96 / 94.5 / 96 -> 88 / 84 / 91.5 us, M = 1536 / 1792: 149.5 / 153 -> 133 /
    // 140 us; up to 8 ranges instead of 4: no further gain).
    int split_unit = kConcurrent;
    if (RBA == 8 && tail.parts == 1) {
        tail = make_gemm_tail_by_rounds(tiling, 32, 4, 0.00085 * 4096.0 / double(k));
        split_unit = 32;
    }
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    while (tail.parts > 1 &&
           (k / kBK < 8 * tail.parts || ws.scratch_bytes < int64_t(8) * tail.max_tiles * tail.parts * Cfg::kBM * Cfg::kBN * 4))
        --tail.parts;
    static_assert(8 * kConcurrent * 4 <= kCounterBytes, "one counter per tail tile");
    const int64_t grid = gemm_grid_with_tail(tiling, split_unit, tail);
    QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
    allow_dynamic_lds(reinterpret_cast<const void *>(gemm_w8a16_kernel16<RB, WM, WN, MIN_BLOCKS, RBA, W_NK>), Cfg::kLdsBytes);
    launch(gemm_w8a16_kernel16<RB, WM, WN, MIN_BLOCKS, RBA, W_NK>, dim3(uint32_t(grid)), dim3(Cfg::kThreads), size_t(Cfg::kLdsBytes), stream,
           static_cast<const _Float16 *>(a), lda, static_cast<const int8_t *>(w), ldw, static_cast<const _Float16 *>(scale),
           static_cast<const _Float16 *>(bias), static_cast<_Float16 *>(c), int(m), int(k), int(n), tiles_m, tiles_n, tiling.xm, tiling.xn, split_unit, tail.parts, tail.max_tiles,
           reinterpret_cast<float *>(ws.scratch), ws.counters);
}

}  // namespace

// The MFMA kernel takes K in whole 64-deep stages, 16-byte aligned activation rows, N a multiple of 4 and
// tensors addressable with 31-bit byte offsets; everything else goes to the row-pass kernel.
bool gemm_w8a16_supported(const void *a, const void *w, const void *c, int64_t m, int64_t k, int64_t n, int64_t lda) {
    return (k % kBK == 0) && (lda % 8 == 0) && (n % 4 == 0) && aligned(a, 16) && aligned(w, 4) && aligned(c, 8) &&
           k * n < (int64_t(1) << 31) - (1 << 20) && (m * lda + k) * 2 < (int64_t(1) << 31) - (1 << 20);
}

void gemm_w8a16_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                       int64_t n, int64_t lda, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    // waves 128 x 64, workgroup tile 128 x 256; a matrix of at most 32 / 64 / 96 rows leaves the empty row blocks out
    if (m <= 32) launch_cfg16<8, 1, 4, 2, 2>(a, w, scale, bias, c, m, k, n, lda, n, workspace, workspace_bytes, stream);
    else if (m <= 64) launch_cfg16<8, 1, 4, 2, 4>(a, w, scale, bias, c, m, k, n, lda, n, workspace, workspace_bytes, stream);
    else if (m <= 96) launch_cfg16<8, 1, 4, 2, 6>(a, w, scale, bias, c, m, k, n, lda, n, workspace, workspace_bytes, stream);
    else launch_cfg16<8, 1, 4, 2, 8>(a, w, scale, bias, c, m, k, n, lda, n, workspace, workspace_bytes, stream);
}

// The same kernel on a weight stored K-contiguous (w_nk[col * ldw + k]): 8-byte loads, so rows of w_nk 8-byte aligned.
bool gemm_w8a16_nk_supported(const void *a, const void *w, const void *c, int64_t m, int64_t k, int64_t n, int64_t lda,
                             int64_t ldw) {
    return (k % kBK == 0) && (lda % 8 == 0) && (n % 4 == 0) && (ldw % 8 == 0) && aligned(a, 16) && aligned(w, 8) &&
           aligned(c, 8) && (n - 1) * ldw + k < (int64_t(1) << 31) - (1 << 20) &&
           (m * lda + k) * 2 < (int64_t(1) << 31) - (1 << 20);
}

void gemm_w8a16_nk_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                          int64_t n, int64_t lda, int64_t ldw, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    if (m <= 32) launch_cfg16<8, 1, 4, 2, 2, true>(a, w, scale, bias, c, m, k, n, lda, ldw, workspace, workspace_bytes, stream);
    else if (m <= 64) launch_cfg16<8, 1, 4, 2, 4, true>(a, w, scale, bias, c, m, k, n, lda, ldw, workspace, workspace_bytes, stream);
    else if (m <= 96) launch_cfg16<8, 1, 4, 2, 6, true>(a, w, scale, bias, c, m, k, n, lda, ldw, workspace, workspace_bytes, stream);
    else launch_cfg16<8, 1, 4, 2, 8, true>(a, w, scale, bias, c, m, k, n, lda, ldw, workspace, workspace_bytes, stream);
}

}  // namespace qmm
