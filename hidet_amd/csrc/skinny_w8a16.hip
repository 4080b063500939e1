// W8A16 decode GEMV / skinny GEMM (M <= 16 rows per pass): c[m, n] = (sum_k a[m, k] * w[k, n]) * scale[n].
//
// HBM-bound: the int8 weight matrix w[K, N] (N contiguous) is streamed exactly once with 16-byte
// loads.  Lane (g, cl) of a wave (g = lane / 16, cl = lane % 16) loads rows 8g .. 8g+7 of a 32-row
// k-step at columns 16cl .. 16cl+15, so one load instruction covers four 256-byte row segments.
// The 8x16 byte block a lane holds is exactly what sixteen 16x16x32 MFMAs need as B operands
// (8 consecutive k for one column each): byte t of two rows is picked with one v_perm_b32 and
// turned into two float16 values with one v_xor_b32 (0x6400 | (q ^ 0x80) == 1152 + q), so no
// weight ever goes through LDS.  The constant 1152 * sum_k a[m, k] is removed per wave with one
// extra MFMA against a vector of ones.  The A operand holds the activation rows (rows >= M are
// zero), so M = 1 and M = 16 cost the same.  K is split over the 4 waves of a workgroup (LDS
// reduction) and over workgroups; the last workgroup to arrive for a column tile adds the partial
// tiles in a fixed order (deterministic), applies the scale and writes float16.
#include "skinny_common.h"

namespace qmm {
namespace {

constexpr int kTileN = kSkinnyTileN;
constexpr int kWaves = kSkinnyWaves;

template <int DEPTH, bool ALIGNED_A, bool FOLD>
__global__ __launch_bounds__(256) void skinny_w8a16_kernel(const _Float16 *__restrict__ a, int64_t lda,
                                                           const int8_t *__restrict__ w,
                                                           const _Float16 *__restrict__ scale, _Float16 *__restrict__ c,
                                                           int m, int k, int n, int rows_per_block, int splits, int tiles,
                                                           float *__restrict__ partials, uint32_t *__restrict__ counters) {
    extern __shared__ float red[];  // [kWaves][m][kRedStride]
    __shared__ int s_last;

    int tile, split;
    if (!skinny_tile_of_block(splits, tiles, &tile, &split)) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, cl = lane & 15;
    const int col0 = tile * kTileN + cl * 16;
    const bool col_ok = col0 < n;

    const int rows_per_wave = rows_per_block / kWaves;
    const int k_begin = split * rows_per_block + wave * rows_per_wave;
    const int k_end = min(k, k_begin + rows_per_wave);

    float4_t acc[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    float4_t xsum = {0.f, 0.f, 0.f, 0.f};
    half8_t ones;
#pragma unroll
    for (int j = 0; j < 8; ++j) ones[j] = _Float16(1.0f);

    const int8_t *wp = w + col0;
    const _Float16 *ap = a + int64_t(cl) * lda;

    for (int kk = k_begin; kk < k_end; kk += 32 * DEPTH) {
        uint4 raw[DEPTH][8];
        half8_t xa[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int row = kk + 32 * d + 8 * g + j;
                raw[d][j] = uint4{0u, 0u, 0u, 0u};
                if (col_ok && row < k_end) raw[d][j] = *reinterpret_cast<const uint4 *>(wp + int64_t(row) * n);
            }
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int kx = kk + 32 * d + 8 * g;
#pragma unroll
            for (int j = 0; j < 8; ++j) xa[d][j] = _Float16(0.0f);
            if (cl < m) {
                if (ALIGNED_A) {
                    if (kx < k_end) xa[d] = *reinterpret_cast<const half8_t *>(ap + kx);
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (kx + j < k_end) xa[d][j] = ap[kx + j];
                }
            }
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                // selector: byte (t % 4) of the even row into bits 0-7, of the odd row into bits 16-23
                constexpr uint32_t kZero = 0x0c;
                const uint32_t sel = (kZero << 24) | (uint32_t(4 + (t & 3)) << 16) | (kZero << 8) | uint32_t(t & 3);
                union {
                    uint32_t u[4];
                    half2_t h2[4];
                    half8_t h8;
                } b;
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const uint32_t lo = reinterpret_cast<const uint32_t *>(&raw[d][2 * p])[t >> 2];
                    const uint32_t hi = reinterpret_cast<const uint32_t *>(&raw[d][2 * p + 1])[t >> 2];
                    b.u[p] = __builtin_amdgcn_perm(hi, lo, sel) ^ 0x64806480u;
                    if (!FOLD) b.h2[p] = b.h2[p] - half2_t{_Float16(1152.0f), _Float16(1152.0f)};
                }
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[d], b.h8, acc[t], 0, 0, 0);
            }
            if (FOLD) xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[d], ones, xsum, 0, 0, 0);
        }
    }

    if (FOLD) {
#pragma unroll
        for (int t = 0; t < 16; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[t][v] -= 1152.0f * xsum[v];
    }
    skinny_reduce_store<_Float16>(acc, m, n, tile, split, splits, scale, c, partials, counters, red, &s_last);
}

// Any shape the fast kernel cannot take (N not a multiple of 16, misaligned weights): one thread per
// output element, serial K, fp32 accumulation.
__global__ __launch_bounds__(256) void naive_w8a16_kernel(const _Float16 *__restrict__ a, int64_t lda,
                                                          const int8_t *__restrict__ w, const _Float16 *__restrict__ scale,
                                                          _Float16 *__restrict__ c, int64_t m, int64_t k, int64_t n) {
    const int64_t o = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (o >= m * n) return;
    const int64_t i = o / n, j = o - i * n;
    float acc = 0.f;
    for (int64_t kk = 0; kk < k; ++kk) acc += float(a[i * lda + kk]) * float(w[kk * n + j]);
    c[o] = _Float16(acc * float(scale[j]));
}

}  // namespace

void skinny_w8a16_launch(const void *a, const void *w, const void *scale, void *c, int64_t m, int64_t k, int64_t n,
                         int64_t lda, int parallel_k_parts, void *workspace, int64_t workspace_bytes, bool strict_workspace,
                         hipStream_t stream) {
    const bool fast = (n % 16 == 0) && aligned(w, 16) && aligned(c, 8) && k > 0;  // 8-byte output stores in the split-K sum
    if (!fast) {
        launch(naive_w8a16_kernel, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, static_cast<const _Float16 *>(a), lda,
               static_cast<const int8_t *>(w), static_cast<const _Float16 *>(scale), static_cast<_Float16 *>(c), m, k, n);
        return;
    }
    int rpb, splits, tiles;
    skinny_plan(k, n, m > 8 ? 768 : 512, parallel_k_parts, 128, &rpb, &splits, &tiles);
    QMM_CHECK(tiles <= kMaxSkinnyTiles, "N too large for the split-K counters");
    skinny_fit_workspace(k, 128, tiles, int(std::min<int64_t>(16, m)), workspace, workspace_bytes, strict_workspace, &rpb, &splits);
    const bool aligned_a = (k % 8 == 0) && (lda % 8 == 0) && aligned(a, 16);
    const int grid = int(cdiv(tiles, 8) * 8 * splits);
    for (int64_t m0 = 0; m0 < m; m0 += 16) {
        const int mt = int(std::min<int64_t>(16, m - m0));
        float *partials = reinterpret_cast<float *>(static_cast<char *>(workspace) + kCounterBytes);
        uint32_t *counters = static_cast<uint32_t *>(workspace);
        const _Float16 *ap = static_cast<const _Float16 *>(a) + m0 * lda;
        _Float16 *cp = static_cast<_Float16 *>(c) + m0 * n;
        const size_t shmem = skinny_lds_bytes(mt);
        auto go = [&](auto kern) {
            if (shmem > 65536) allow_dynamic_lds(reinterpret_cast<const void *>(kern), int(skinny_lds_bytes(16)));  // the most any m needs
            launch(kern, dim3(grid), dim3(256), shmem, stream, ap, lda, static_cast<const int8_t *>(w),
                   static_cast<const _Float16 *>(scale), cp, mt, int(k), int(n), rpb, splits, tiles, partials, counters);
        };
        if (aligned_a) go(skinny_w8a16_kernel<2, true, true>);
        else go(skinny_w8a16_kernel<2, false, true>);
    }
}

}  // namespace qmm
