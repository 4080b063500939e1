// FP8 e4m3 decode GEMV / skinny GEMM (M <= 16): c[m, n] = cast(alpha * sum_k a[m, k] * b[n, k]).
//
// b is [N, K] with K contiguous, so the reduction runs along the lanes' own loads: lane (kg, ls) of a
// wave reads 32 consecutive bytes of row n0 + ls at k = kbase + 32 kg; the 16 lanes x 4 k-groups of one
// k-step cover 16 rows x 128 contiguous bytes.  Those 32 bytes are directly the column operand of
// the CDNA4 block-scaled MFMA 16x16x128 (unit scales): the matrix core does both the multiply and the
// cross-lane reduction, and M = 1 costs the same as M = 16.  The 4 waves of a workgroup split K and
// meet in LDS; a workgroup owns 16 output columns, so N / 16 workgroups stream b exactly once.
#include "common.h"
#include "numeric.h"

namespace qmm {
namespace {

constexpr int kWaves = 4;
constexpr int kEightWaveTiles = 512;  // fewer column tiles than this: eight waves per workgroup (8192 x 4096: 9.4 -> 7.2 us)
constexpr int kDepth = 8;  // k-steps (of 128 bytes) whose loads are issued together

template <int OUT, bool ALIGNED_A, int FMT = kFmtE4M3>
__global__ __launch_bounds__(256) void skinny_fp8_kernel(const uint8_t *__restrict__ a, int64_t lda,
                                                         const uint8_t *__restrict__ b, int64_t ldb, void *__restrict__ c,
                                                         int m, int n, int k, const float *__restrict__ scale_a,
                                                         const float *__restrict__ scale_b) {
    __shared__ float red[kWaves][16][17];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 4, ls = lane & 15;
    const int n0 = blockIdx.x * 16;
    const int nrow = n0 + ls;
    const bool n_ok = nrow < n;

    // K is cut into 128-byte steps dealt to the waves in contiguous runs
    const int steps = (k + 127) >> 7;
    const int steps_per_wave = (steps + kWaves - 1) / kWaves;
    const int s_begin = wave * steps_per_wave, s_end = min(steps, s_begin + steps_per_wave);

    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    const uint8_t *bp = b + int64_t(nrow) * ldb + 32 * kg;
    const uint8_t *ap = a + int64_t(ls) * lda + 32 * kg;

    for (int s0 = s_begin; s0 < s_end; s0 += kDepth) {
        uint4 wv[kDepth][2], xv[kDepth][2];
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int kb = (s0 + d) * 128 + 32 * kg;
            wv[d][0] = wv[d][1] = uint4{0u, 0u, 0u, 0u};
            if (n_ok && s0 + d < s_end) {
                if (kb < k) wv[d][0] = *reinterpret_cast<const uint4 *>(bp + int64_t(s0 + d) * 128);
                if (kb + 16 < k) wv[d][1] = *reinterpret_cast<const uint4 *>(bp + int64_t(s0 + d) * 128 + 16);
            }
        }
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int kb = (s0 + d) * 128 + 32 * kg;
            xv[d][0] = xv[d][1] = uint4{0u, 0u, 0u, 0u};
            if (ls < m && s0 + d < s_end) {
                if (ALIGNED_A) {
                    if (kb < k) xv[d][0] = *reinterpret_cast<const uint4 *>(ap + int64_t(s0 + d) * 128);
                    if (kb + 16 < k) xv[d][1] = *reinterpret_cast<const uint4 *>(ap + int64_t(s0 + d) * 128 + 16);
                } else {
                    uint8_t tmp[32];
#pragma unroll
                    for (int e = 0; e < 32; ++e) tmp[e] = (kb + e < k) ? ap[int64_t(s0 + d) * 128 + e] : uint8_t(0);
                    uint32_t wds[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        wds[e] = uint32_t(tmp[4 * e]) | (uint32_t(tmp[4 * e + 1]) << 8) | (uint32_t(tmp[4 * e + 2]) << 16) |
                                 (uint32_t(tmp[4 * e + 3]) << 24);
                    xv[d][0] = uint4{wds[0], wds[1], wds[2], wds[3]};
                    xv[d][1] = uint4{wds[4], wds[5], wds[6], wds[7]};
                }
            }
        }
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            int8v_t rv, cv;
            rv[0] = int(xv[d][0].x); rv[1] = int(xv[d][0].y); rv[2] = int(xv[d][0].z); rv[3] = int(xv[d][0].w);
            rv[4] = int(xv[d][1].x); rv[5] = int(xv[d][1].y); rv[6] = int(xv[d][1].z); rv[7] = int(xv[d][1].w);
            cv[0] = int(wv[d][0].x); cv[1] = int(wv[d][0].y); cv[2] = int(wv[d][0].z); cv[3] = int(wv[d][0].w);
            cv[4] = int(wv[d][1].x); cv[5] = int(wv[d][1].y); cv[6] = int(wv[d][1].z); cv[7] = int(wv[d][1].w);
            // rows = activation rows, columns = rows of b; both operands in format FMT, unit block scales
            acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rv, cv, acc, FMT, FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
        }
    }
    // acc[v] = partial c[4 kg + v][n0 + ls]
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][4 * kg + v][ls] = acc[v];
    __syncthreads();
    const int row = tid >> 4, cn = tid & 15;
    if (row < m && n0 + cn < n) {
        float v = red[0][row][cn] + red[1][row][cn] + red[2][row][cn] + red[3][row][cn];
        if (scale_a != nullptr) v *= *scale_a;
        if (scale_b != nullptr) v *= *scale_b;
        store_out<OUT>(c, int64_t(row) * n + n0 + cn, v);
    }
}

// 3 to 16 rows, K a multiple of 128, aligned activations.  Fetching the activation operand straight from memory (lane =
// 16 bytes at a 32-byte stride of one of 16 rows) touches every cache line of a step's 16 x 128-byte block twice and once
// per row, and the time grew with M (8192 x 8192: 13.3 us for one row, 19.6 us for 16).  Here a wave fetches the block
// with two fully coalesced loads (8 rows x 128 bytes each) and reads its operand back from a private LDS tile of
// 16 rows x (128 + 16) bytes, two slots; no barrier, one wave's LDS operations execute in order.  The loop has no
// conditions: lanes of rows >= M and columns >= N read a clamped row and their results are dropped.
// BLOCK_SCALED: scale_a is [K / 128, M] and scale_b [N / 128, K / 128] (one factor per 128-deep step and row, and per step
// and 128 output columns): every step's products are accumulated from zero and added to the total times both factors.
// The 16 row factors of a step are fetched by the 16 lanes of a group like one more operand and turned into the four
// each lane needs (rows 4 kg .. 4 kg + 3) through LDS, per step, as the activations are.
// FMT: operand format of the MFMA, 0 = float8 e4m3, 1 = float8 e5m2.
template <int OUT, int WAVES, bool BLOCK_SCALED = false, int FMT = 0>
__global__ __launch_bounds__(64 * WAVES) void skinny_fp8_staged_kernel(const uint8_t *__restrict__ a, int64_t lda,
                                                                const uint8_t *__restrict__ b, int64_t ldb,
                                                                void *__restrict__ c, int m, int n, int k,
                                                                const float *__restrict__ scale_a,
                                                                const float *__restrict__ scale_b) {
    __shared__ float red[WAVES][16][17];
    __shared__ uint4 stage[WAVES][2][16 * 9];
    __shared__ float4_t factor_stage[BLOCK_SCALED ? WAVES : 1][2][4];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 4, ls = lane & 15;
    const int n0 = blockIdx.x * 16;

    const int steps = k >> 7;
    const int steps_per_wave = (steps + WAVES - 1) / WAVES;
    const int s_begin = wave * steps_per_wave, s_end = min(steps, s_begin + steps_per_wave);

    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    const float *sa_col = BLOCK_SCALED ? scale_a + min(ls, m - 1) : nullptr;
    const float *sb_row = BLOCK_SCALED ? scale_b + int64_t(n0 >> 7) * steps : nullptr;  // 16 columns lie in one 128-column block
    const uint8_t *bp = b + int64_t(min(n0 + ls, n - 1)) * ldb + 32 * kg;
    const uint8_t *ap0 = a + int64_t(min(lane >> 3, m - 1)) * lda + 16 * (lane & 7);
    const uint8_t *ap1 = a + int64_t(min(8 + (lane >> 3), m - 1)) * lda + 16 * (lane & 7);

    for (int s0 = s_begin; s0 < s_end; s0 += kDepth) {
        uint4 wv[kDepth][2], ax[kDepth][2];
        float fr[BLOCK_SCALED ? kDepth : 1];
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int st = min(s0 + d, s_end - 1);  // a step past the wave's range re-reads its last one; not used
            wv[d][0] = *reinterpret_cast<const uint4 *>(bp + int64_t(st) * 128);
            wv[d][1] = *reinterpret_cast<const uint4 *>(bp + int64_t(st) * 128 + 16);
            if (BLOCK_SCALED) fr[d] = sa_col[int64_t(st) * m] * sb_row[st];
        }
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int st = min(s0 + d, s_end - 1);
            ax[d][0] = *reinterpret_cast<const uint4 *>(ap0 + int64_t(st) * 128);
            ax[d][1] = *reinterpret_cast<const uint4 *>(ap1 + int64_t(st) * 128);
        }
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            // One block per step (wave-uniform branch): the compiler moves each step's loads down into its block, so a
            // wave has one step in flight at a time and the many waves per CU hide the latency.  Measured against the
            // same loop without the branch, where all eight steps' loads really are issued up front: 8192 x 8192, one
            // row: 12 us against 18 us.
            if (s0 + d >= s_end) break;
            uint4 *tile = stage[wave][d & 1];
            tile[(lane >> 3) * 9 + (lane & 7)] = ax[d][0];
            tile[(8 + (lane >> 3)) * 9 + (lane & 7)] = ax[d][1];
            const uint4 x0 = tile[ls * 9 + 2 * kg], x1 = tile[ls * 9 + 2 * kg + 1];
            int8v_t rv, cv;
            rv[0] = int(x0.x); rv[1] = int(x0.y); rv[2] = int(x0.z); rv[3] = int(x0.w);
            rv[4] = int(x1.x); rv[5] = int(x1.y); rv[6] = int(x1.z); rv[7] = int(x1.w);
            cv[0] = int(wv[d][0].x); cv[1] = int(wv[d][0].y); cv[2] = int(wv[d][0].z); cv[3] = int(wv[d][0].w);
            cv[4] = int(wv[d][1].x); cv[5] = int(wv[d][1].y); cv[6] = int(wv[d][1].z); cv[7] = int(wv[d][1].w);
            if (BLOCK_SCALED) {
                float *ft = reinterpret_cast<float *>(factor_stage[wave][d & 1]);
                ft[ls] = fr[d];  // the four lane groups store the same 16 values
                const float4_t f = factor_stage[wave][d & 1][kg];
                const float4_t part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rv, cv, zero, FMT, FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[v] = fmaf(part[v], f[v], acc[v]);
            } else {
                acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rv, cv, acc, FMT, FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
            }
        }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][4 * kg + v][ls] = acc[v];
    __syncthreads();
    const int row = tid >> 4, cn = tid & 15;
    if (row < m && n0 + cn < n) {  // row < 16: threads of the first four waves
        float v = 0.f;
#pragma unroll
        for (int p = 0; p < WAVES; ++p) v += red[p][row][cn];
        if (!BLOCK_SCALED && scale_a != nullptr) v *= *scale_a;
        if (!BLOCK_SCALED && scale_b != nullptr) v *= *scale_b;
        const int64_t o = int64_t(row) * n + n0 + cn;
        if (OUT == HIDET_QMM_F32) static_cast<float *>(c)[o] = v;
        else if (OUT == HIDET_QMM_BF16) static_cast<uint16_t *>(c)[o] = f32_to_bf16_bits(v);
        else if (OUT == HIDET_QMM_F16) static_cast<uint16_t *>(c)[o] = f32_to_f16_bits(v);
        else if (OUT == HIDET_QMM_E5M2) static_cast<uint8_t *>(c)[o] = f32_to_e5m2(v);
        else static_cast<uint8_t *>(c)[o] = f32_to_e4m3(v);
    }
}

}  // namespace

bool skinny_fp8_supported(const void *b, int64_t k, int64_t ldb) { return (ldb % 16 == 0) && (k % 16 == 0) && aligned(b, 16) && k > 0; }

void skinny_fp8_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                       int out_dtype, const void *scale_a, const void *scale_b, hipStream_t stream) {
    const uint8_t *ap = static_cast<const uint8_t *>(a), *bp = static_cast<const uint8_t *>(b);
    const float *sa = static_cast<const float *>(scale_a), *sb = static_cast<const float *>(scale_b);
    const bool aligned_a = (lda % 16 == 0) && aligned(a, 16);
    const dim3 grid(uint32_t(cdiv(n, 16)));
    auto go = [&](auto kern, int waves = 4) {
        launch(kern, grid, dim3(64 * waves), 0, stream, ap, lda, bp, ldb, c, int(m), int(n), int(k), sa, sb);
    };
    // few column tiles: eight waves per workgroup keep enough loads in flight on each compute unit
    const bool eight = cdiv(n, 16) < kEightWaveTiles && k >= 8 * 128;
    const bool staged = aligned_a && k % 128 == 0;
#define QMM_FP8_SKINNY(OUT)                                   \
    if (staged && eight) go(skinny_fp8_staged_kernel<OUT, 8>, 8); \
    else if (staged) go(skinny_fp8_staged_kernel<OUT, 4>);    \
    else if (aligned_a) go(skinny_fp8_kernel<OUT, true>);     \
    else go(skinny_fp8_kernel<OUT, false>);
    switch (out_dtype) {
        case HIDET_QMM_F32: QMM_FP8_SKINNY(HIDET_QMM_F32) break;
        case HIDET_QMM_F16: QMM_FP8_SKINNY(HIDET_QMM_F16) break;
        case HIDET_QMM_BF16: QMM_FP8_SKINNY(HIDET_QMM_BF16) break;
        case HIDET_QMM_E4M3: QMM_FP8_SKINNY(HIDET_QMM_E4M3) break;
        default: QMM_FAIL("unsupported output dtype code " << out_dtype);
    }
#undef QMM_FP8_SKINNY
}

// float8_e5m2 operands, up to 16 rows: the plain kernel with the MFMA's bf8 format
void skinny_fp8_e5m2_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                            int out_dtype, const void *scale_a, const void *scale_b, hipStream_t stream) {
    const uint8_t *ap = static_cast<const uint8_t *>(a), *bp = static_cast<const uint8_t *>(b);
    const float *sa = static_cast<const float *>(scale_a), *sb = static_cast<const float *>(scale_b);
    const bool aligned_a = (lda % 16 == 0) && aligned(a, 16);
    const dim3 grid(uint32_t(cdiv(n, 16)));
    auto go = [&](auto kern) { launch(kern, grid, dim3(256), 0, stream, ap, lda, bp, ldb, c, int(m), int(n), int(k), sa, sb); };
#define QMM_BF8_SKINNY(OUT)                                           \
    if (aligned_a) go(skinny_fp8_kernel<OUT, true, kFmtE5M2>);        \
    else go(skinny_fp8_kernel<OUT, false, kFmtE5M2>);
    switch (out_dtype) {
        case HIDET_QMM_F32: QMM_BF8_SKINNY(HIDET_QMM_F32) break;
        case HIDET_QMM_F16: QMM_BF8_SKINNY(HIDET_QMM_F16) break;
        case HIDET_QMM_BF16: QMM_BF8_SKINNY(HIDET_QMM_BF16) break;
        case HIDET_QMM_E5M2: QMM_BF8_SKINNY(HIDET_QMM_E5M2) break;
        default: QMM_FAIL("unsupported output dtype code " << out_dtype << " for float8_e5m2 operands");
    }
#undef QMM_BF8_SKINNY
}

// Block-scaled operands (scale_a f32 [K/128, M], scale_b f32 [N/128, K/128]), up to 16 rows, contiguous a [M, K] and b [N, K],
// K and N multiples of 128, everything 16-byte aligned (the entry point checks that).
void skinny_fp8_block_scaled_launch(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m,
                                    int64_t n, int64_t k, int out_dtype, bool e5m2, hipStream_t stream) {
    const uint8_t *ap = static_cast<const uint8_t *>(a), *bp = static_cast<const uint8_t *>(b);
    const float *sa = static_cast<const float *>(scale_a), *sb = static_cast<const float *>(scale_b);
    const dim3 grid(uint32_t(cdiv(n, 16)));
    const bool eight = cdiv(n, 16) < kEightWaveTiles && k >= 8 * 128;
    auto go = [&](auto kern, int waves) {
        launch(kern, grid, dim3(64 * waves), 0, stream, ap, k, bp, k, c, int(m), int(n), int(k), sa, sb);
    };
#define QMM_FP8_SKINNY_SCALED(OUT, FMT)                                     \
    if (eight) go(skinny_fp8_staged_kernel<OUT, 8, true, FMT>, 8);          \
    else go(skinny_fp8_staged_kernel<OUT, 4, true, FMT>, 4);
    if (e5m2) {  // both operands float8_e5m2; the 8-bit output type is the operands' own
        switch (out_dtype) {
            case HIDET_QMM_F32: QMM_FP8_SKINNY_SCALED(HIDET_QMM_F32, 1) break;
            case HIDET_QMM_F16: QMM_FP8_SKINNY_SCALED(HIDET_QMM_F16, 1) break;
            case HIDET_QMM_BF16: QMM_FP8_SKINNY_SCALED(HIDET_QMM_BF16, 1) break;
            case HIDET_QMM_E5M2: QMM_FP8_SKINNY_SCALED(HIDET_QMM_E5M2, 1) break;
            default: QMM_FAIL("unsupported output dtype code " << out_dtype);
        }
    } else {
        switch (out_dtype) {
            case HIDET_QMM_F32: QMM_FP8_SKINNY_SCALED(HIDET_QMM_F32, 0) break;
            case HIDET_QMM_F16: QMM_FP8_SKINNY_SCALED(HIDET_QMM_F16, 0) break;
            case HIDET_QMM_BF16: QMM_FP8_SKINNY_SCALED(HIDET_QMM_BF16, 0) break;
            case HIDET_QMM_E4M3: QMM_FP8_SKINNY_SCALED(HIDET_QMM_E4M3, 0) break;
            default: QMM_FAIL("unsupported output dtype code " << out_dtype);
        }
    }
#undef QMM_FP8_SKINNY_SCALED
}

}  // namespace qmm
