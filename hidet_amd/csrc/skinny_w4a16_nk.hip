// Group-wise W4A16 decode GEMV / skinny GEMM (M <= 16 rows per pass) for weights repacked K-contiguous:
//   c[m, n] = sum_g scale[g, n] * sum_{k in group g} a[m, k] * q[k, n],   q = signed 4-bit codes.
//
// w_nk is [N, K / 2] bytes, row n = the K codes of output column n (stride ldw bytes).  Inside every 32-bit word (8
// consecutive k) nibble i holds code k = 2 i for i < 4 and code k = 2 (i - 4) + 1 for i >= 4, so that
// (word >> 4 i) & 0x000F000F is the pair (k = 2 i, k = 2 i + 1) at bits 0-3 and 16-19: one shift and one
// mask-and-xor (a single three-input bit operation) per pair of weights give two 16-bit floats bias + q, in the order
// the MFMA wants them.  Scales stay [K / group, N].
//
// Same structure as the int8 kernel for K-contiguous weights: a workgroup owns 16 output columns, its waves split K
// in 128-deep steps and meet in LDS, nothing is exchanged between workgroups.  Lane (kg, ls) reads 16 consecutive bytes
// (32 codes, k = 128 step + 32 kg ...) of row n0 + ls per step: four MFMA B operands of 8 consecutive k.  A step lies
// inside one group (the group size is 128 times a power of two), so the step's products are accumulated from zero,
// the constant bias * sum_k a[m, k] comes from four more MFMAs against ones, and both are folded into the running
// total with the step's scale of the lane's own output column: two fma per value and step.  The loop has no
// conditions: lanes of rows >= M and columns >= N read a clamped row, their results are dropped.  Activations are
// fetched with coalesced loads and turned into MFMA fragments through a wave-private LDS tile (from 3 rows on; with one
// or two rows the direct fetch is a broadcast).
#include "w4_traits.h"

namespace qmm {
namespace {

constexpr int kDepth = 8;  // 128-deep steps whose loads are issued together

template <int DT, int WAVES, bool STAGE>
__global__ __launch_bounds__(64 * WAVES) void skinny_w4a16_nk_kernel(const uint16_t *__restrict__ a, int64_t lda,
                                                                     const uint8_t *__restrict__ w, int64_t ldw,
                                                                     const uint16_t *__restrict__ scales,
                                                                     uint16_t *__restrict__ c, int m, int k, int n,
                                                                     int group_shift) {
    using T = W4Traits<DT>;
    __shared__ float red[WAVES][16][17];
    __shared__ uint4 stage[STAGE ? WAVES : 1][2][16 * 17];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 4, ls = lane & 15;
    const int n0 = blockIdx.x * 16;
    const int col = min(n0 + ls, n - 1);

    const int steps = k >> 7;
    const int steps_per_wave = (steps + WAVES - 1) / WAVES;
    const int s_begin = wave * steps_per_wave, s_end = min(steps, s_begin + steps_per_wave);

    float4_t total = {0.f, 0.f, 0.f, 0.f};
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    const uint32_t one2 = uint32_t(T::kOne) | (uint32_t(T::kOne) << 16);
    const uint4 ones = uint4{one2, one2, one2, one2};
    const uint8_t *wp = w + int64_t(col) * ldw + 16 * kg;
    const uint16_t *ap = a + int64_t(min(ls, m - 1)) * lda + 32 * kg;

    for (int s0 = s_begin; s0 < s_end; s0 += kDepth) {
        uint4 wv[kDepth], ax[kDepth][4];
        uint16_t sc[kDepth];
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int st = min(s0 + d, s_end - 1);  // a step past the wave's range re-reads its last one; not used
            wv[d] = *reinterpret_cast<const uint4 *>(wp + int64_t(st) * 64);
            sc[d] = scales[int64_t(st >> group_shift) * n + col];
        }
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int st = min(s0 + d, s_end - 1);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (STAGE) {  // load j: rows 4j .. 4j+3, 16 lanes x 16 bytes per row
                    const int r = min(4 * j + kg, m - 1);
                    ax[d][j] = *reinterpret_cast<const uint4 *>(a + int64_t(r) * lda + int64_t(st) * 128 + 8 * ls);
                } else {
                    ax[d][j] = *reinterpret_cast<const uint4 *>(ap + int64_t(st) * 128 + 8 * j);
                }
            }
        }
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            // One block per step (wave-uniform branch): the compiler moves each step's loads down into its block, so a
            // wave has one step in flight at a time and the many waves per CU hide the latency; two steps per block
            // were measured slower (K = 4096, N = 11008: 9.1 -> 9.5 us for one row, 11.2 -> 12.6 us for 16).
            if (s0 + d >= s_end) break;
            uint4 xa[4];
            if (STAGE) {
                uint4 *tile = stage[wave][d & 1];
#pragma unroll
                for (int j = 0; j < 4; ++j) tile[(4 * j + kg) * 17 + ls] = ax[d][j];
#pragma unroll
                for (int j = 0; j < 4; ++j) xa[j] = tile[ls * 17 + 4 * kg + j];
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) xa[j] = ax[d][j];
            }
            const uint32_t raw[4] = {wv[d].x, wv[d].y, wv[d].z, wv[d].w};
            float4_t acc = zero, xs = zero;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint4 b;
                b.x = (raw[j] & 0x000F000Fu) ^ T::kMagic;
                b.y = ((raw[j] >> 4) & 0x000F000Fu) ^ T::kMagic;
                b.z = ((raw[j] >> 8) & 0x000F000Fu) ^ T::kMagic;
                b.w = ((raw[j] >> 12) & 0x000F000Fu) ^ T::kMagic;
                // rows = activation rows, columns = rows of w_nk (output columns); every weight carries + bias
                acc = T::mfma(xa[j], b, acc);
                xs = T::mfma(xa[j], ones, xs);
            }
            const float s = T::to_f32(sc[d]);
            const float sb = -T::kBias * s;  // exact in fp32
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                total[v] = fmaf(acc[v], s, total[v]);
                total[v] = fmaf(xs[v], sb, total[v]);
            }
        }
    }
    // total[v] = partial c[4 kg + v][n0 + ls]
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][4 * kg + v][ls] = total[v];
    __syncthreads();
    const int row = tid >> 4, cn = tid & 15;
    if (row < m && n0 + cn < n) {  // row < 16: threads of the first four waves
        float v = 0.f;
#pragma unroll
        for (int p = 0; p < WAVES; ++p) v += red[p][row][cn];
        c[int64_t(row) * n + n0 + cn] = DT == HIDET_QMM_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
    }
}

}  // namespace

// The group size must be 128 times a power of two (a 128-deep step then lies inside one group and the group of a step
// is a shift away); K a multiple of 128; rows of w_nk and of a 16-byte aligned.
bool skinny_w4a16_nk_supported(const void *a, const void *w, int64_t k, int64_t lda, int64_t ldw, int group) {
    if (group < 128 || (group & (group - 1)) != 0) return false;
    return k > 0 && k % 128 == 0 && ldw % 16 == 0 && aligned(w, 16) && lda % 8 == 0 && aligned(a, 16);
}

// Any M: 16 rows per pass, every pass streams the weights again.
void skinny_w4a16_nk_launch(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n,
                            int64_t lda, int64_t ldw, int group, int dtype, hipStream_t stream) {
    int group_shift = 0;
    while ((128 << group_shift) < group) ++group_shift;
    const dim3 grid(uint32_t(cdiv(n, 16)));
    for (int64_t m0 = 0; m0 < m; m0 += 16) {
        const int mt = int(std::min<int64_t>(16, m - m0));
        const uint16_t *ap = static_cast<const uint16_t *>(a) + m0 * lda;
        uint16_t *cp = static_cast<uint16_t *>(c) + m0 * n;
        auto go = [&](auto kern, int waves) {
            launch(kern, grid, dim3(64 * waves), 0, stream, ap, lda, static_cast<const uint8_t *>(w), ldw,
                   static_cast<const uint16_t *>(scales), cp, mt, int(k), int(n), group_shift);
        };
        const bool stage = mt > 2;
        // eight waves per workgroup: with few column tiles they keep enough loads in flight on each compute unit; with one
        // or two rows they also shorten each wave's chain of dependent steps (K = 4096, N = 11008, one row: 9.6 -> 9.1 us;
        // 4 to 16 rows: 9.8-11.2 -> 10.5-11.5 us, so not there)
        const bool eight = (cdiv(n, 16) < 512 || !stage) && k >= 8 * 128;
        // few column tiles, a long K and one or two rows: sixteen waves halve each wave's chain of steps once more
        // (K = 11008, N = 4096: 10.5 -> 8.7 us; with the LDS tile of the staged form 16 waves would not fit)
        const bool sixteen = cdiv(n, 16) < 512 && !stage && k >= 32 * 128;
#define QMM_W4_NK(DT)                                                                \
    if (sixteen) go(skinny_w4a16_nk_kernel<DT, 16, false>, 16);                      \
    else if (eight && stage) go(skinny_w4a16_nk_kernel<DT, 8, true>, 8);             \
    else if (eight) go(skinny_w4a16_nk_kernel<DT, 8, false>, 8);                     \
    else if (stage) go(skinny_w4a16_nk_kernel<DT, 4, true>, 4);                      \
    else go(skinny_w4a16_nk_kernel<DT, 4, false>, 4);
        if (dtype == HIDET_QMM_F16) {
            QMM_W4_NK(HIDET_QMM_F16)
        } else {
            QMM_W4_NK(HIDET_QMM_BF16)
        }
#undef QMM_W4_NK
    }
}

}  // namespace qmm
