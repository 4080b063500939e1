// W8A16 decode GEMV / skinny GEMM for weights stored K-contiguous: w is the [K, N] operand of the operator held as
// [N, K] in memory (row n = the K codes of output column n, stride ldw) - the layout of torch's nn.Linear weight, or
// of a [K, N] tensor with strides (1, ldw).  c[m, n] = (sum_k a[m, k] * w[n, k]) * scale[n], fp32 accumulation, M <= 16
// rows per pass.
//
// The reduction runs along the contiguous axis, so nothing has to be exchanged between workgroups: a workgroup owns 16
// output columns, its 4 or 8 waves split K and meet in LDS, N / 16 workgroups stream the weights exactly once.  Lane
// (kg, ls) of a wave reads 32 consecutive bytes of row n0 + ls at k = kbase + 32 kg per 128-deep step (the 16 lanes x 4
// k-groups of a step cover 16 rows x 128 contiguous bytes).  Bytes 8j .. 8j+7 of those 32 are, for j = 0 .. 3, the B
// operand of one v_mfma_f32_16x16x32_f16: the k positions an MFMA sums over may be any 32 as long as both operands
// agree, so MFMA j takes k = kbase + 32 kg + 8 j + (0 .. 7) from lane group kg, and the activation fragment is loaded
// from exactly those positions.  Two bytes become two float16 values with v_perm_b32 (spread) and v_xor_b32 (0x6400 |
// (q ^ 0x80) == 1152 + q): one VALU op per weight; the constant is removed at the end with 1152 * sum_k a[m, k], which
// one more MFMA per fragment (against ones) accumulates on the otherwise idle matrix pipe - exact in fp32 for the
// few thousand terms of a wave's K range.  With K a multiple of 128 (FULL) the loop has no conditions at all: lanes
// of rows >= M and columns >= N read a clamped row and their results are dropped at the end.  Each step of that loop
// sits behind a wave-uniform break, and the compiler moves the step's loads down into its block: a wave has one step in
// flight at a time and the 8 to 11 waves per CU hide the latency (the FP8 kernel of the same shape was measured a third
// slower with all of a trip's loads really issued up front).
#include "common.h"

namespace qmm {
namespace {

template <bool ALIGNED_A, bool FULL, int WAVES, bool STAGE = false>
__global__ __launch_bounds__(64 * WAVES) void skinny_w8a16_nk_kernel(const _Float16 *__restrict__ a, int64_t lda,
                                                              const int8_t *__restrict__ w, int64_t ldw,
                                                              const _Float16 *__restrict__ scale, const _Float16 *__restrict__ bias,
                                                              _Float16 *__restrict__ c, int m, int k, int n) {
    __shared__ float red[WAVES][16][17];
    constexpr int kNkDepth = FULL ? 8 : 4;  // 128-deep steps per trip of the outer loop
    // STAGE (FULL with aligned activations, more than two rows): a wave fetches its 16 x 128 activation block of a step
    // with four fully coalesced loads (4 rows x 256 bytes each) and turns it into MFMA fragments through a private LDS
    // tile of 16 rows x (256 + 16) bytes, two slots.  Fetching the fragments straight from memory touches every cache
    // line of the block four times, and made 16 rows cost 8 us more than one; with one or two rows the direct fetch
    // is a broadcast and a little faster.  No barrier: the LDS operations of one wave execute in order.
    static_assert(!STAGE || (FULL && ALIGNED_A), "staging needs the condition-free loop and 16-byte loads");
    constexpr bool kStage = STAGE;
    __shared__ uint4 stage[kStage ? WAVES : 1][2][16 * 17];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 4, ls = lane & 15;
    const int n0 = blockIdx.x * 16;
    const bool n_ok = n0 + ls < n;
    const bool m_ok = ls < m;

    // K is cut into 128-deep steps dealt to the waves in contiguous runs
    const int steps = (k + 127) >> 7;
    const int steps_per_wave = (steps + WAVES - 1) / WAVES;
    const int s_begin = wave * steps_per_wave, s_end = min(steps, s_begin + steps_per_wave);

    float4_t acc = {0.f, 0.f, 0.f, 0.f}, xsum = {0.f, 0.f, 0.f, 0.f};
    half8_t ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = _Float16(1.0f);
    // FULL: rows past the end are clamped to the last one instead of being masked in the loop
    const int8_t *wp = w + int64_t(FULL ? min(n0 + ls, n - 1) : n0 + ls) * ldw + 32 * kg;
    const _Float16 *ap = a + int64_t(FULL ? min(ls, m - 1) : ls) * lda + 32 * kg;

    for (int s0 = s_begin; s0 < s_end; s0 += kNkDepth) {
        uint4 wv[kNkDepth][2];
        half8_t xa[kNkDepth][4];
        uint4 ax[kStage ? kNkDepth : 1][4];
#pragma unroll
        for (int d = 0; d < kNkDepth; ++d) {
            if (FULL) {
                const int st = min(s0 + d, s_end - 1);  // a step past the wave's range re-reads its last one; not used
                wv[d][0] = *reinterpret_cast<const uint4 *>(wp + int64_t(st) * 128);
                wv[d][1] = *reinterpret_cast<const uint4 *>(wp + int64_t(st) * 128 + 16);
            } else {
                const int kb = (s0 + d) * 128 + 32 * kg;
                wv[d][0] = wv[d][1] = uint4{0u, 0u, 0u, 0u};
                if (n_ok && s0 + d < s_end) {  // K % 16 == 0: a 16-byte piece is inside K or outside as a whole
                    if (kb < k) wv[d][0] = *reinterpret_cast<const uint4 *>(wp + int64_t(s0 + d) * 128);
                    if (kb + 16 < k) wv[d][1] = *reinterpret_cast<const uint4 *>(wp + int64_t(s0 + d) * 128 + 16);
                }
            }
        }
#pragma unroll
        for (int d = 0; d < kNkDepth; ++d) {
            const int kb = (s0 + d) * 128 + 32 * kg;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (FULL) {
                    const int st = min(s0 + d, s_end - 1);
                    if (kStage) {  // load j: rows 4j .. 4j+3, 16 lanes x 16 bytes per row
                        const int r = min(4 * j + kg, m - 1);
                        ax[d][j] = *reinterpret_cast<const uint4 *>(a + int64_t(r) * lda + int64_t(st) * 128 + 8 * ls);
                    } else if (ALIGNED_A) {
                        xa[d][j] = *reinterpret_cast<const half8_t *>(ap + int64_t(st) * 128 + 8 * j);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) xa[d][j][e] = ap[int64_t(st) * 128 + 8 * j + e];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) xa[d][j][e] = _Float16(0.0f);
                    if (m_ok && s0 + d < s_end && kb + 8 * j < k) {  // K % 8 == 0 on this path
                        if (ALIGNED_A) {
                            xa[d][j] = *reinterpret_cast<const half8_t *>(ap + int64_t(s0 + d) * 128 + 8 * j);
                        } else {
#pragma unroll
                            for (int e = 0; e < 8; ++e) xa[d][j][e] = ap[int64_t(s0 + d) * 128 + 8 * j + e];
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int d = 0; d < kNkDepth; ++d) {
            if (FULL && s0 + d >= s_end) break;  // wave-uniform
            if (kStage) {
                uint4 *tile = stage[wave][d & 1];
#pragma unroll
                for (int j = 0; j < 4; ++j) tile[(4 * j + kg) * 17 + ls] = ax[d][j];
#pragma unroll
                for (int j = 0; j < 4; ++j) xa[d][j] = __builtin_bit_cast(half8_t, tile[ls * 17 + 4 * kg + j]);
            }
            const uint32_t raw[8] = {wv[d][0].x, wv[d][0].y, wv[d][0].z, wv[d][0].w, wv[d][1].x, wv[d][1].y, wv[d][1].z, wv[d][1].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // bytes 8j .. 8j+7 = dwords 2j, 2j+1; selectors spread bytes (0, 1) and (2, 3) of a dword into two halves
                constexpr uint32_t kLo = 0x0c010c00u, kHi = 0x0c030c02u;
                union {
                    uint32_t u[4];
                    half8_t h8;
                } b;
                b.u[0] = __builtin_amdgcn_perm(raw[2 * j], raw[2 * j], kLo) ^ 0x64806480u;
                b.u[1] = __builtin_amdgcn_perm(raw[2 * j], raw[2 * j], kHi) ^ 0x64806480u;
                b.u[2] = __builtin_amdgcn_perm(raw[2 * j + 1], raw[2 * j + 1], kLo) ^ 0x64806480u;
                b.u[3] = __builtin_amdgcn_perm(raw[2 * j + 1], raw[2 * j + 1], kHi) ^ 0x64806480u;
                // rows = activation rows, columns = weight rows (output columns); the weights carry + 1152 each
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[d][j], b.h8, acc, 0, 0, 0);
                xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[d][j], ones, xsum, 0, 0, 0);
            }
        }
    }
    // acc[v] = partial c[4 kg + v][n0 + ls]; zero weights of masked lanes also carried + 1152, which xsum removes as well
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][4 * kg + v][ls] = acc[v] - 1152.0f * xsum[v];
    __syncthreads();
    const int row = tid >> 4, cn = tid & 15;
    if (row < m && n0 + cn < n) {  // row < 16 <= the first four waves
        float v = 0.f;
#pragma unroll
        for (int p = 0; p < WAVES; ++p) v += red[p][row][cn];
        c[int64_t(row) * n + n0 + cn] = scaled_biased_f16(v, float(scale[n0 + cn]), bias != nullptr ? float(bias[n0 + cn]) : -0.0f);
    }
}

// More than a few activation rows: the kernel above re-reads the activation rows once per 16 output columns, which at 16
// rows is twice the weight bytes.  Here a wave keeps one activation fragment for CG column groups (16 CG columns per
// workgroup), so that traffic drops by CG; the workgroup's waves split K as before.  K a multiple of 128, aligned
// activations; the loop has no conditions (clamped rows, see above).
template <int CG, int WAVES, int DEPTH>
__global__ __launch_bounds__(64 * WAVES) void skinny_w8a16_nk_wide_kernel(const _Float16 *__restrict__ a, int64_t lda,
                                                                          const int8_t *__restrict__ w, int64_t ldw,
                                                                          const _Float16 *__restrict__ scale,
                                                                          const _Float16 *__restrict__ bias,
                                                                          _Float16 *__restrict__ c, int m, int k, int n) {
    __shared__ float red[WAVES][CG][16][17];
    __shared__ uint4 stage[WAVES][2][16 * 17];  // per wave: activation block of a step, see the kernel above
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 4, ls = lane & 15;
    const int n0 = blockIdx.x * (16 * CG);

    const int steps = k >> 7;
    const int steps_per_wave = (steps + WAVES - 1) / WAVES;
    const int s_begin = wave * steps_per_wave, s_end = min(steps, s_begin + steps_per_wave);

    float4_t acc[CG], xsum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < CG; ++g) acc[g] = float4_t{0.f, 0.f, 0.f, 0.f};
    half8_t ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = _Float16(1.0f);
    const int8_t *wp[CG];
#pragma unroll
    for (int g = 0; g < CG; ++g) wp[g] = w + int64_t(min(n0 + 16 * g + ls, n - 1)) * ldw + 32 * kg;

    for (int s0 = s_begin; s0 < s_end; s0 += DEPTH) {
        uint4 wv[DEPTH][CG][2];
        half8_t xa[DEPTH][4];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int st = min(s0 + d, s_end - 1);  // a step past the wave's range re-reads its last one; not used
#pragma unroll
            for (int g = 0; g < CG; ++g) {
                wv[d][g][0] = *reinterpret_cast<const uint4 *>(wp[g] + int64_t(st) * 128);
                wv[d][g][1] = *reinterpret_cast<const uint4 *>(wp[g] + int64_t(st) * 128 + 16);
            }
        }
        uint4 ax[DEPTH][4];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int st = min(s0 + d, s_end - 1);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int r = min(4 * j + kg, m - 1);
                ax[d][j] = *reinterpret_cast<const uint4 *>(a + int64_t(r) * lda + int64_t(st) * 128 + 8 * ls);
            }
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (s0 + d >= s_end) break;  // wave-uniform
            uint4 *tile = stage[wave][d & 1];
#pragma unroll
            for (int j = 0; j < 4; ++j) tile[(4 * j + kg) * 17 + ls] = ax[d][j];
#pragma unroll
            for (int j = 0; j < 4; ++j) xa[d][j] = __builtin_bit_cast(half8_t, tile[ls * 17 + 4 * kg + j]);
#pragma unroll
            for (int g = 0; g < CG; ++g) {
                const uint32_t raw[8] = {wv[d][g][0].x, wv[d][g][0].y, wv[d][g][0].z, wv[d][g][0].w,
                                         wv[d][g][1].x, wv[d][g][1].y, wv[d][g][1].z, wv[d][g][1].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    constexpr uint32_t kLo = 0x0c010c00u, kHi = 0x0c030c02u;
                    union {
                        uint32_t u[4];
                        half8_t h8;
                    } b;
                    b.u[0] = __builtin_amdgcn_perm(raw[2 * j], raw[2 * j], kLo) ^ 0x64806480u;
                    b.u[1] = __builtin_amdgcn_perm(raw[2 * j], raw[2 * j], kHi) ^ 0x64806480u;
                    b.u[2] = __builtin_amdgcn_perm(raw[2 * j + 1], raw[2 * j + 1], kLo) ^ 0x64806480u;
                    b.u[3] = __builtin_amdgcn_perm(raw[2 * j + 1], raw[2 * j + 1], kHi) ^ 0x64806480u;
                    acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[d][j], b.h8, acc[g], 0, 0, 0);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[d][j], ones, xsum, 0, 0, 0);
        }
    }
#pragma unroll
    for (int g = 0; g < CG; ++g)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave][g][4 * kg + v][ls] = acc[g][v] - 1152.0f * xsum[v];
    __syncthreads();
    for (int o = tid; o < CG * 256; o += 64 * WAVES) {
        const int g = o >> 8, row = (o >> 4) & 15, cn = o & 15;
        const int col = n0 + 16 * g + cn;
        if (row < m && col < n) {
            float v = 0.f;
#pragma unroll
            for (int p = 0; p < WAVES; ++p) v += red[p][g][row][cn];
            c[int64_t(row) * n + col] = scaled_biased_f16(v, float(scale[col]), bias != nullptr ? float(bias[col]) : -0.0f);
        }
    }
}

}  // namespace

bool skinny_w8a16_nk_supported(const void *w, int64_t k, int64_t ldw) {
    return (ldw % 16 == 0) && (k % 16 == 0) && aligned(w, 16) && k > 0;
}

// Any M: 16 rows per pass, every pass streams the weights again (beyond a few passes the [K, N] layout and its MFMA
// GEMM are the better choice).
void skinny_w8a16_nk_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                            int64_t n, int64_t lda, int64_t ldw, hipStream_t stream) {
    const bool aligned_a = (lda % 8 == 0) && aligned(a, 16);
    const dim3 grid(uint32_t(cdiv(n, 16)));
    for (int64_t m0 = 0; m0 < m; m0 += 16) {
        const int mt = int(std::min<int64_t>(16, m - m0));
        const _Float16 *ap = static_cast<const _Float16 *>(a) + m0 * lda;
        _Float16 *cp = static_cast<_Float16 *>(c) + m0 * n;
        auto go = [&](auto kern, int waves) {
            launch(kern, grid, dim3(64 * waves), 0, stream, ap, lda, static_cast<const int8_t *>(w), ldw, static_cast<const _Float16 *>(scale),
                   static_cast<const _Float16 *>(bias), cp, mt, int(k), int(n));
        };
        const bool full = k % 128 == 0;
        // more than 8 rows, a wide matrix and a long K: 32 columns per workgroup, the activation rows are read half as often
        if (full && aligned_a && mt > 8 && cdiv(n, 32) >= 256 && k >= 8192) {
            launch(skinny_w8a16_nk_wide_kernel<2, 8, 4>, dim3(uint32_t(cdiv(n, 32))), dim3(512), 0, stream, ap, lda,
                   static_cast<const int8_t *>(w), ldw, static_cast<const _Float16 *>(scale), static_cast<const _Float16 *>(bias), cp,
                   mt, int(k), int(n));
            continue;
        }
        // few column tiles: eight waves per workgroup keep enough loads in flight on each compute unit
        const bool eight = full && cdiv(n, 16) < 512 && k >= 8 * 128;
        const bool stage = full && aligned_a && mt > 2;
        if (eight && stage) go(skinny_w8a16_nk_kernel<true, true, 8, true>, 8);
        else if (eight) aligned_a ? go(skinny_w8a16_nk_kernel<true, true, 8>, 8) : go(skinny_w8a16_nk_kernel<false, true, 8>, 8);
        else if (stage) go(skinny_w8a16_nk_kernel<true, true, 4, true>, 4);
        else if (aligned_a) full ? go(skinny_w8a16_nk_kernel<true, true, 4>, 4) : go(skinny_w8a16_nk_kernel<true, false, 4>, 4);
        else full ? go(skinny_w8a16_nk_kernel<false, true, 4>, 4) : go(skinny_w8a16_nk_kernel<false, false, 4>, 4);
    }
}

}  // namespace qmm
