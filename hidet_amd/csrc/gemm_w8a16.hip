// W8A16 prefill GEMM (M >= 32): c[m, n] = (sum_k a[m, k] * w[k, n]) * scale[n] on fp16 MFMA with fp32
// accumulation.
//
// The int8 weights never pass through LDS.  Lane (kg, ns) of a wave (kg = lane / 16, ns = lane % 16)
// loads rows 8kg .. 8kg+7 of a 32-row k-step at columns 4ns .. 4ns+3 (one dword per row); that 8x4
// byte block holds, for each of its 4 columns, the 8 consecutive k values a 16x16x32 MFMA wants as
// the B operand of output column slot ns.  Byte t of two rows is gathered with one v_perm_b32, one
// v_xor_b32 turns the pair into two float16 values (0x6400 | (q ^ 0x80) == 1152 + q) and one packed
// subtract removes the 1152, so the dequantisation is exact and costs 3 VALU ops per 2 weights,
// hidden under the MFMAs.  A wave owns RB*16 rows x 64 columns of the output; every dequantised
// fragment is reused for RB row blocks.  The activation tile of the workgroup is staged through LDS
// (16-byte chunks, XOR-swizzled so the fragment reads are conflict free), double buffered, with the
// next stage's global loads in flight during the MFMAs.  The per-column scale is applied to the fp32
// accumulators in the epilogue.
#include "common.h"

namespace qmm {
namespace {

constexpr int kBK = 64;  // k extent of one pipeline stage (two 32-deep MFMA steps)

template <int RB, int WN>
struct GemmW8Cfg {
    static constexpr int kBM = RB * 16;
    static constexpr int kBN = WN * 64;
    static constexpr int kThreads = WN * 64;
    static constexpr int kAChunks = kBM * 8 / kThreads;  // 16-byte chunks of the A stage per thread
    static constexpr int kLdsBytes = 2 * kBM * 128;
};

template <int RB, int WN, int MIN_BLOCKS>
__global__ __launch_bounds__(WN * 64, MIN_BLOCKS) void gemm_w8a16_kernel(const _Float16 *__restrict__ a, int64_t lda,
                                                                          const int8_t *__restrict__ w,
                                                                          const _Float16 *__restrict__ scale,
                                                                          _Float16 *__restrict__ c, int m, int k, int n,
                                                                          int tiles_m, int tiles_n) {
    using Cfg = GemmW8Cfg<RB, WN>;
    extern __shared__ uint4 lds[];  // [2][kBM * 8] chunks

    // ---- tile of this workgroup: every XCD owns a contiguous range of tile columns and walks it
    // row-block first, so the workgroups resident on one XCD share a few weight tile columns in L2.
    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int cb_begin = (tiles_n * xcd) / 8, cb_end = (tiles_n * (xcd + 1)) / 8;
    if (local >= (cb_end - cb_begin) * tiles_m) return;
    const int cb = cb_begin + local / tiles_m;
    const int rbk = local % tiles_m;
    const int m0 = rbk * Cfg::kBM;
    const int n0 = cb * Cfg::kBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 4, ns = lane & 15;
    const int col = n0 + wave * 64 + ns * 4;  // first of this lane's 4 columns
    const bool col_ok = col < n;               // n % 4 == 0: the 4 columns are in or out together

    float4_t acc[RB][4];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[rb][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    // A staging: thread -> chunk (row = tid / 8 + j * kThreads / 8, chunk = tid % 8)
    const int a_row = tid >> 3, a_chunk = tid & 7;
    const _Float16 *a_base = a + int64_t(m0 + a_row) * lda + a_chunk * 8;
    const int8_t *w_base = w + col;

    uint4 a_regs[Cfg::kAChunks];
    uint32_t w_raw[2][8];  // raw int8 rows of the two k-steps of a stage; reloaded in place once consumed

    auto load_a = [&](int kbase) {
#pragma unroll
        for (int j = 0; j < Cfg::kAChunks; ++j) {
            const int row = m0 + a_row + j * (Cfg::kThreads / 8);
            a_regs[j] = uint4{0u, 0u, 0u, 0u};
            if (row < m && kbase + a_chunk * 8 < k)
                a_regs[j] = *reinterpret_cast<const uint4 *>(a_base + int64_t(j * (Cfg::kThreads / 8)) * lda + kbase);
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int j = 0; j < Cfg::kAChunks; ++j) {
            const int r = a_row + j * (Cfg::kThreads / 8);
            lds[buf * Cfg::kBM * 8 + r * 8 + (a_chunk ^ (r & 7))] = a_regs[j];
        }
    };
    auto load_w = [&](int kbase, int ks) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int row = kbase + ks * 32 + kg * 8 + j;
            w_raw[ks][j] = 0u;
            if (col_ok && row < k) w_raw[ks][j] = *reinterpret_cast<const uint32_t *>(w_base + int64_t(row) * n);
        }
    };

    load_a(0);
    load_w(0, 0);
    load_w(0, 1);
    store_a(0);
    __syncthreads();

    const int stages = (k + kBK - 1) / kBK;
    for (int s = 0; s < stages; ++s) {
        const int buf = s & 1;
        const bool more = s + 1 < stages;
        if (more) load_a((s + 1) * kBK);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            union BFrag {
                uint32_t u[4];
                half2_t h2[4];
                half8_t h8;
            } b[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                constexpr uint32_t kZero = 0x0c;
                const uint32_t sel = (kZero << 24) | (uint32_t(4 + t) << 16) | (kZero << 8) | uint32_t(t);
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    b[t].u[p] = __builtin_amdgcn_perm(w_raw[ks][2 * p + 1], w_raw[ks][2 * p], sel) ^ 0x64806480u;
                    b[t].h2[p] = b[t].h2[p] - half2_t{_Float16(1152.0f), _Float16(1152.0f)};
                }
            }
            if (more) load_w((s + 1) * kBK, ks);  // the raw rows of this k-step are consumed: prefetch in place
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int r = rb * 16 + ns;
                const uint4 v = lds[buf * Cfg::kBM * 8 + r * 8 + ((ks * 4 + kg) ^ (r & 7))];
                const half8_t afrag = __builtin_bit_cast(half8_t, v);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc[rb][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag, b[t].h8, acc[rb][t], 0, 0, 0);
            }
        }
        if (more) store_a(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: scale the fp32 accumulators per column, round to float16, 8-byte stores -----------
    if (!col_ok) return;
    float sc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) sc[t] = float(scale[col + t]);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = m0 + rb * 16 + kg * 4 + v;
            if (row < m) {
                half4_t o;
#pragma unroll
                for (int t = 0; t < 4; ++t) o[t] = _Float16(acc[rb][t][v] * sc[t]);
                *reinterpret_cast<half4_t *>(c + int64_t(row) * n + col) = o;
            }
        }
}

}  // namespace

bool gemm_w8a16_supported(const void *a, const void *w, const void *c, int64_t k, int64_t n, int64_t lda) {
    return (k % 8 == 0) && (lda % 8 == 0) && (n % 4 == 0) && aligned(a, 16) && aligned(w, 4) && aligned(c, 8);
}

void gemm_w8a16_launch(const void *a, const void *w, const void *scale, void *c, int64_t m, int64_t k, int64_t n,
                       int64_t lda, hipStream_t stream) {
    constexpr int RB = 8, WN = 4;
    using Cfg = GemmW8Cfg<RB, WN>;
    const int tiles_m = int(cdiv(m, Cfg::kBM)), tiles_n = int(cdiv(n, Cfg::kBN));
    // every XCD gets floor/ceil(tiles_n / 8) tile columns: size the grid for the largest share
    const int max_cols = int(cdiv(tiles_n, 8));
    const int64_t grid = int64_t(8) * max_cols * tiles_m;
    QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
    launch(gemm_w8a16_kernel<RB, WN, 2>, dim3(uint32_t(grid)), dim3(Cfg::kThreads), size_t(Cfg::kLdsBytes), stream,
           static_cast<const _Float16 *>(a), lda, static_cast<const int8_t *>(w), static_cast<const _Float16 *>(scale),
           static_cast<_Float16 *>(c), int(m), int(k), int(n), tiles_m, tiles_n);
}

}  // namespace qmm
