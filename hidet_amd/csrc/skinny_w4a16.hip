// Group-wise W4A16 decode GEMV / skinny GEMM (M <= 16 rows per pass):
//   c[m, n] = sum_g scale[g, n] * sum_{k in group g} a[m, k] * q[k, n],   q = signed 4-bit codes.
//
// Weights are packed two codes per byte along n, low nibble first (byte [k, j] holds columns 2j and
// 2j+1), scales are [K / group, N] in the activation dtype (bfloat16 or float16).  Same structure as the
// int8 kernel: lane (g, cl) loads rows 8g .. 8g+7 of a 32-row k-step, 8 bytes = 16 columns per row, so a
// load instruction covers four 128-byte row segments and a wave covers 256 columns.  The nibbles are
// byte-gathered pairwise across two rows with v_perm_b32 (one byte = an even and an odd column), and a
// mask-and-xor (one three-input bit operation; plus a shift for the odd column) produces two bfloat16
// (0x4300 | (nibble ^ 8) == 136 + q) or float16 (0x6400 | (nibble ^ 8) == 1032 + q) values: the B operand
// of a 16x16x32 MFMA.  The constant is removed per group with one extra MFMA against ones; at every group
// boundary the fp32 accumulators are scaled into the running totals.
#include "skinny_common.h"
#include "w4_traits.h"

namespace qmm {
namespace {

constexpr int kSkinnyWaves = 4;  // waves per workgroup; they split the workgroup's K slice

template <int DT, int DEPTH, bool ALIGNED_A, bool FULL = false>
__global__ __launch_bounds__(256, 2) void skinny_w4a16_kernel(const uint16_t *__restrict__ a, int64_t lda,
                                                           const uint8_t *__restrict__ w,
                                                           const uint16_t *__restrict__ scales, uint16_t *__restrict__ c,
                                                           int m, int k, int n, int group, int rows_per_block, int splits,
                                                           int tiles, float *__restrict__ mailbox) {
    using T = W4Traits<DT>;
    extern __shared__ float red[];

    int tile, split;
    if (!skinny_tile_of_block(splits, tiles, &tile, &split)) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, cl = lane & 15;
    const int col0 = tile * kSkinnyTileN + cl * 16;
    const bool col_ok = col0 < n;
    const int64_t row_bytes = n >> 1;

    const int rows_per_wave = rows_per_block / kSkinnyWaves;
    const int k_begin = split * rows_per_block + wave * rows_per_wave;
    const int k_end = min(k, k_begin + rows_per_wave);

    float4_t acc[16], total[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
        total[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    float4_t xsum = {0.f, 0.f, 0.f, 0.f};
    const uint32_t one2 = uint32_t(T::kOne) | (uint32_t(T::kOne) << 16);
    const uint4 ones = uint4{one2, one2, one2, one2};

    // FULL: every column exists, every wave's K range is a whole number of iterations and the activations allow 16-byte
    // loads, so the loop has no per-lane conditions; lanes of rows >= M read the last row and their results are dropped
    const uint8_t *wp = w + (col0 >> 1);
    const uint16_t *ap = a + int64_t(FULL ? min(cl, m - 1) : cl) * lda;
    uint4 sc_raw[2] = {uint4{0u, 0u, 0u, 0u}, uint4{0u, 0u, 0u, 0u}};  // 16 scales of the current group

    for (int kk = k_begin; kk < k_end; kk += 32 * DEPTH) {
        uint2 raw[DEPTH][8];
        uint4 xa[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int row = kk + 32 * d + 8 * g + j;
                if (FULL) {
                    raw[d][j] = *reinterpret_cast<const uint2 *>(wp + int64_t(row) * row_bytes);
                    continue;
                }
                raw[d][j] = uint2{0x88888888u, 0x88888888u};  // nibble 8 ^ 8 == code 0
                if (col_ok && row < k_end) raw[d][j] = *reinterpret_cast<const uint2 *>(wp + int64_t(row) * row_bytes);
            }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int kx = kk + 32 * d + 8 * g;
            if (FULL) {
                xa[d] = *reinterpret_cast<const uint4 *>(ap + kx);
                continue;
            }
            xa[d] = uint4{0u, 0u, 0u, 0u};
            if (cl < m) {
                if (ALIGNED_A) {
                    if (kx < k_end) xa[d] = *reinterpret_cast<const uint4 *>(ap + kx);
                } else {
                    uint16_t tmp[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) tmp[j] = (kx + j < k_end) ? ap[kx + j] : uint16_t(0);
                    xa[d] = uint4{uint32_t(tmp[0]) | (uint32_t(tmp[1]) << 16), uint32_t(tmp[2]) | (uint32_t(tmp[3]) << 16),
                                  uint32_t(tmp[4]) | (uint32_t(tmp[5]) << 16), uint32_t(tmp[6]) | (uint32_t(tmp[7]) << 16)};
                }
            }
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int ks = kk + 32 * d;
            if (FULL || ks < k_end) {  // uniform across the wave
                if (ks % group == 0 || ks == k_begin) {
                    if (FULL || col_ok) {
                        const uint16_t *sp = scales + int64_t(ks / group) * n + col0;
                        sc_raw[0] = *reinterpret_cast<const uint4 *>(sp);
                        sc_raw[1] = *reinterpret_cast<const uint4 *>(sp + 8);
                    }
                }
                // byte b of dword h of rows 2p and 2p+1 goes to bits 0-7 and 16-23 of one register (v_perm_b32); its low
                // nibbles are column 8h + 2b of both rows, its high nibbles column 8h + 2b + 1: mask-and-xor (one
                // three-input bit operation) gives the two 16-bit floats bias + q, for the odd column after a shift
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int byte = 0; byte < 4; ++byte) {
                        constexpr uint32_t kZero = 0x0c;
                        const uint32_t sel = (kZero << 24) | (uint32_t(4 + byte) << 16) | (kZero << 8) | uint32_t(byte);
                        uint4 be, bo;
                        uint32_t *bep = reinterpret_cast<uint32_t *>(&be), *bop = reinterpret_cast<uint32_t *>(&bo);
#pragma unroll
                        for (int p = 0; p < 4; ++p) {
                            const uint32_t lo = h ? raw[d][2 * p].y : raw[d][2 * p].x;
                            const uint32_t hi = h ? raw[d][2 * p + 1].y : raw[d][2 * p + 1].x;
                            const uint32_t x = __builtin_amdgcn_perm(hi, lo, sel);
                            bep[p] = (x & 0x000F000Fu) ^ T::kMagic;
                            bop[p] = ((x >> 4) & 0x000F000Fu) ^ T::kMagic;
                        }
                        const int t = 8 * h + 2 * byte;
                        acc[t] = T::mfma(xa[d], be, acc[t]);
                        acc[t + 1] = T::mfma(xa[d], bo, acc[t + 1]);
                    }
                }
                xsum = T::mfma(xa[d], ones, xsum);
                if ((ks + 32) % group == 0 || ks + 32 >= k_end) {  // group complete (or slice ends): fold it in
                    const uint16_t *sv = reinterpret_cast<const uint16_t *>(sc_raw);
#pragma unroll
                    for (int t = 0; t < 16; ++t) {
                        const float s = T::to_f32(sv[t]);
                        const float sb = -T::kBias * s;  // exact: a power of two plus a small multiple times a 16-bit float
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            total[t][v] = fmaf(acc[t][v], s, total[t][v]);
                            total[t][v] = fmaf(xsum[v], sb, total[t][v]);
                            acc[t][v] = 0.f;
                        }
                    }
                    xsum = float4_t{0.f, 0.f, 0.f, 0.f};
                }
            }
        }
    }
    const SkinnyScale no_scale;  // all ones: the group scales are already in the totals
    if (DT == HIDET_QMM_F16)
        skinny_finish<_Float16, kSkinnyWaves>(total, m, n, tile, split, splits, no_scale, reinterpret_cast<_Float16 *>(c), mailbox, red);
    else
        skinny_finish<uint16_t, kSkinnyWaves>(total, m, n, tile, split, splits, no_scale, c, mailbox, red);
}

// Any shape the fast kernel cannot take: one thread per output element, serial K, fp32 accumulation.
template <int DT>
__global__ __launch_bounds__(256) void naive_w4a16_kernel(const uint16_t *__restrict__ a, int64_t lda,
                                                          const uint8_t *__restrict__ w, const uint16_t *__restrict__ scales,
                                                          uint16_t *__restrict__ c, int64_t m, int64_t k, int64_t n, int group) {
    using T = W4Traits<DT>;
    const int64_t o = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (o >= m * n) return;
    const int64_t i = o / n, j = o - i * n;
    float total = 0.f;
    for (int64_t g0 = 0; g0 < k; g0 += group) {
        float acc = 0.f;
        for (int64_t kk = g0; kk < g0 + group; ++kk) {
            const uint8_t byte = w[(kk * n + j) >> 1];
            const int q = (int(int8_t((j & 1) ? byte : uint8_t(byte << 4)))) >> 4;  // sign-extend the nibble
            acc += T::to_f32(a[i * lda + kk]) * float(q);
        }
        total += acc * T::to_f32(scales[(g0 / group) * n + j]);
    }
    if (DT == HIDET_QMM_F16) c[o] = f32_to_f16_bits(total);
    else c[o] = f32_to_bf16_bits(total);
}

}  // namespace

bool skinny_w4a16_fast(const void *w, const void *scales, int64_t k, int64_t n, int group) {
    return (n % 16 == 0) && (group % 32 == 0) && aligned(w, 8) && aligned(scales, 16) && k > 0;
}

void skinny_w4a16_launch(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n,
                         int64_t lda, int group, int dtype, int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                         hipStream_t stream) {
    const uint16_t *ap0 = static_cast<const uint16_t *>(a);
    const uint8_t *wp = static_cast<const uint8_t *>(w);
    const uint16_t *sp = static_cast<const uint16_t *>(scales);
    uint16_t *cp0 = static_cast<uint16_t *>(c);
    if (!skinny_w4a16_fast(w, scales, k, n, group)) {
        if (dtype == HIDET_QMM_F16)
            launch(naive_w4a16_kernel<HIDET_QMM_F16>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap0, lda, wp, sp, cp0, m, k, n, group);
        else
            launch(naive_w4a16_kernel<HIDET_QMM_BF16>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap0, lda, wp, sp, cp0, m, k, n, group);
        return;
    }
    int rpb, splits, tiles;
    skinny_plan(k, n, 512, parallel_k_parts, 128, &rpb, &splits, &tiles);
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    skinny_fit_mailbox(k, 128, tiles, int(std::min<int64_t>(16, m)), ws.mailbox_bytes, false, &rpb, &splits);
    const bool aligned_a = (k % 8 == 0) && (lda % 8 == 0) && aligned(a, 16);
    const int grid = int(cdiv(tiles, 8) * 8 * splits);
    for (int64_t m0 = 0; m0 < m; m0 += 16) {
        const int mt = int(std::min<int64_t>(16, m - m0));
        const size_t shmem = skinny_lds_bytes(mt, kSkinnyWaves);
        auto go = [&](auto kern) {
            if (shmem > 65536) allow_dynamic_lds(reinterpret_cast<const void *>(kern), int(skinny_lds_bytes(16, kSkinnyWaves)));  // the most any m needs
            launch(kern, dim3(grid), dim3(256), shmem, stream, ap0 + m0 * lda, lda, wp, sp, cp0 + m0 * n, mt, int(k), int(n),
                   group, rpb, splits, tiles, ws.mailbox);
        };
        const bool full = aligned_a && n % kSkinnyTileN == 0 && k % rpb == 0 && rpb % (kSkinnyWaves * 64) == 0;
        if (full) {
            if (dtype == HIDET_QMM_F16) go(skinny_w4a16_kernel<HIDET_QMM_F16, 2, true, true>);
            else go(skinny_w4a16_kernel<HIDET_QMM_BF16, 2, true, true>);
        } else if (dtype == HIDET_QMM_F16) {
            if (aligned_a) go(skinny_w4a16_kernel<HIDET_QMM_F16, 2, true>);
            else go(skinny_w4a16_kernel<HIDET_QMM_F16, 2, false>);
        } else {
            if (aligned_a) go(skinny_w4a16_kernel<HIDET_QMM_BF16, 2, true>);
            else go(skinny_w4a16_kernel<HIDET_QMM_BF16, 2, false>);
        }
    }
}

}  // namespace qmm
