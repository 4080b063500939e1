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

constexpr int kSkinnyWaves = 8;   // waves per workgroup; they split the workgroup's K slice
constexpr int kNonTemporal = 2;   // cache policy bits of a buffer load: sc0 = 1, nt = 2, sc1 = 16
constexpr int kDepth = 2;          // 32-row steps fetched together

// Same launch plan and load discipline as the int8 kernel: the (tile, 32-row step) units dealt evenly to 8-wave
// workgroups, non-temporal loads with no condition around them - rows past the wave's range lie outside the buffer and
// read as zero bytes, which are code 0 - and the exchange of skinny_tails. A step is 32 rows and the group size a
// multiple of 32, so a step never straddles two groups.
template <int DT, bool ALIGNED_A, bool BIAS>
__global__ __launch_bounds__(64 * kSkinnyWaves) void skinny_w4a16_kernel(int ksteps, uint32_t ksteps_magic, int per_group, int longer, int splits, uint32_t splits_magic,
                                                                        const uint8_t *__restrict__ w, const uint16_t *__restrict__ a,
                                                                        int64_t lda, int m, int k, int n, int group,
                                                                        SkinnyPlanRest plan_rest, const uint16_t *__restrict__ scales,
                                                                        const uint16_t *__restrict__ bias, uint16_t *__restrict__ c,
                                                                        float *__restrict__ mailbox, uint32_t *__restrict__ lost_flag) {
    using T = W4Traits<DT>;
    extern __shared__ float red[];

    const SkinnyPlanHead plan_head = {ksteps, ksteps_magic, per_group, longer, splits, splits_magic};
    const SkinnyPlan plan(plan_head, plan_rest);
    int grp;
    if (!skinny_group_of_block(plan_head, plan_rest.tiles, int(blockIdx.x), &grp)) return;
    const SkinnyWork wk = skinny_work_of(plan_head, grp);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, cl = lane & 15;
    const int row_bytes = n >> 1;
    int run_lo, run_hi, part;
    skinny_wave_run(wk, wave, kSkinnyWaves, &run_lo, &run_hi, &part);

    const uint32_t one2 = uint32_t(T::kOne) | (uint32_t(T::kOne) << 16);
    const uint4 ones = uint4{one2, one2, one2, one2};
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(a), 0, ALIGNED_A ? int((int64_t(m - 1) * lda + k) * 2) : 0, 0x00020000);
    const uint16_t *ap = a + int64_t(cl) * lda;
    const int a_row_off = int(int64_t(cl) * lda * 2);
    // scales of a lane's 16 columns: 32 bytes per group
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(scales), 0, int(int64_t(k / group) * n * 2), 0x00020000);

    // the wave's run lies in one tile (skinny_wave_run)
    {
        const int tile = wk.tile + part;
        const int tile_col = tile * kSkinnyTileN;
        const bool col_ok = tile_col + cl * 16 < n;
        const int k_begin = (run_lo - tile * plan.ksteps) * 32;
        const int k_end = min(k, (run_hi - tile * plan.ksteps) * 32);
        const int nsteps = run_hi - run_lo;

        float4_t acc[16], total[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
            total[t] = float4_t{0.f, 0.f, 0.f, 0.f};
        }
        float4_t xsum = {0.f, 0.f, 0.f, 0.f};

        // weights: the wave's rows at the tile's first byte column; a lane whose 16 columns lie past N reads the tile's
        // first columns and its results are never stored
        const int64_t w_bytes = int64_t(k_end - k_begin) * row_bytes - (tile_col >> 1);
        const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t *>(w + int64_t(k_begin) * row_bytes + (tile_col >> 1)), 0, int(w_bytes < 0 ? 0 : w_bytes), 0x00020000);
        uint32_t w_off = uint32_t(8 * g) * uint32_t(row_bytes) + (col_ok ? cl * 8 : 0);
        const int s_col_off = (tile_col + (col_ok ? cl * 16 : 0)) * 2;
        uint4v_t sc_raw[2] = {uint4v_t{0u, 0u, 0u, 0u}, uint4v_t{0u, 0u, 0u, 0u}};

        // kDepth 32-row steps are fetched together: a step is only 4 KiB per wave here (8 bytes per lane and row).
        for (int step0 = 0; step0 < nsteps; step0 += kDepth) {
            uint2 raw[kDepth][8];
            uint4 xa[kDepth];
#pragma unroll
            for (int d = 0; d < kDepth; ++d) {
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, w_off + uint32_t(r) * uint32_t(row_bytes), 0, kNonTemporal);
                    raw[d][r] = uint2{v[0], v[1]};
                }
                w_off += 32u * uint32_t(row_bytes);
                asm volatile("" : "+v"(w_off));
                const int kx = k_begin + 32 * (step0 + d) + 8 * g;
                if (ALIGNED_A) {
                    const int off = (cl < m && kx < k_end) ? a_row_off + kx * 2 : 0x7FFFFFF0;
                    xa[d] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, off, 0, 0));
                } else {
                    uint16_t tmp[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) tmp[j] = (cl < m && kx + j < k_end) ? ap[kx + j] : uint16_t(0);
                    xa[d] = uint4{uint32_t(tmp[0]) | (uint32_t(tmp[1]) << 16), uint32_t(tmp[2]) | (uint32_t(tmp[3]) << 16),
                                  uint32_t(tmp[4]) | (uint32_t(tmp[5]) << 16), uint32_t(tmp[6]) | (uint32_t(tmp[7]) << 16)};
                }
            }
#pragma unroll
            for (int d = 0; d < kDepth; ++d) {
                const int step = step0 + d;
                if (step >= nsteps) break;  // uniform across the wave
                const int ks = k_begin + 32 * step;
                if (ks % group == 0 || step == 0) {  // a new group starts
                    const int soff = (ks / group) * n * 2 + s_col_off;
                    sc_raw[0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, soff, 0, 0);
                    sc_raw[1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, soff + 16, 0, 0);
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
                            const uint32_t lo32 = h ? raw[d][2 * p].y : raw[d][2 * p].x;
                            const uint32_t hi32 = h ? raw[d][2 * p + 1].y : raw[d][2 * p + 1].x;
                            const uint32_t x = __builtin_amdgcn_perm(hi32, lo32, sel);
                            bep[p] = (x & 0x000F000Fu) ^ T::kMagic;
                            bop[p] = ((x >> 4) & 0x000F000Fu) ^ T::kMagic;
                        }
                        const int t = 8 * h + 2 * byte;
                        acc[t] = T::mfma(xa[d], be, acc[t]);
                        acc[t + 1] = T::mfma(xa[d], bo, acc[t + 1]);
                    }
                }
                xsum = T::mfma(xa[d], ones, xsum);
                if ((ks + 32) % group == 0 || step == nsteps - 1) {  // group complete (or the wave's range ends): fold it in
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
        skinny_stash(total, m, wave, red);
    }
    // no column factor: the group scales are already in the totals; BIAS: the bias (of the output's type) is added to the
    // rounded result, as a matmul followed by an add would. Without one the kernels are the ones that never knew of it.
    const SkinnyScale no_scale = {nullptr, BIAS ? reinterpret_cast<const _Float16 *>(bias) : nullptr};
    // (worked out here, not inside the loop: there it was measured to cost the loop more than it saves the tail)
    const SkinnyRoles roles = skinny_roles_of(plan, wk, grp, kSkinnyWaves);
    if constexpr (DT == HIDET_QMM_F16)
        skinny_tails<_Float16, kSkinnyWaves>(plan, wk, roles, m, n, no_scale, reinterpret_cast<_Float16 *>(c), mailbox, lost_flag, red);
    else if constexpr (BIAS)
        skinny_tails<bf16_biased_t, kSkinnyWaves>(plan, wk, roles, m, n, no_scale, reinterpret_cast<bf16_biased_t *>(c), mailbox, lost_flag, red);
    else
        skinny_tails<uint16_t, kSkinnyWaves>(plan, wk, roles, m, n, no_scale, c, mailbox, lost_flag, red);
}

// Any shape the fast kernel cannot take: one thread per output element, serial K, fp32 accumulation.
template <int DT>
__global__ __launch_bounds__(256) void naive_w4a16_kernel(const uint16_t *__restrict__ a, int64_t lda,
                                                          const uint8_t *__restrict__ w, const uint16_t *__restrict__ scales,
                                                          const uint16_t *__restrict__ bias, uint16_t *__restrict__ c, int64_t m,
                                                          int64_t k, int64_t n, int group) {
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
    const float b = bias != nullptr ? T::to_f32(bias[j]) : -0.0f;  // -0.0 changes nothing, not even the sign of a zero
    if (DT == HIDET_QMM_F16) c[o] = __builtin_bit_cast(uint16_t, scaled_biased_f16(total, 1.0f, b));
    else c[o] = biased_bf16_bits(total, b);
}

}  // namespace

bool skinny_w4a16_fast(const void *w, const void *scales, int64_t k, int64_t n, int group) {
    return (n % 16 == 0) && n < (int64_t(1) << 30) && (group % 32 == 0) && aligned(w, 8) && aligned(scales, 16) && k > 0;
}

void skinny_w4a16_launch(const void *a, const void *w, const void *scales, const void *bias, void *c, int64_t m, int64_t k, int64_t n,
                         int64_t lda, int group, int dtype, int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                         hipStream_t stream) {
    const uint16_t *ap0 = static_cast<const uint16_t *>(a);
    const uint16_t *bp = static_cast<const uint16_t *>(bias);
    const uint8_t *wp = static_cast<const uint8_t *>(w);
    const uint16_t *sp = static_cast<const uint16_t *>(scales);
    uint16_t *cp0 = static_cast<uint16_t *>(c);
    if (!skinny_w4a16_fast(w, scales, k, n, group) || !aligned(bias, 8)) {  // 8-byte bias loads
        if (dtype == HIDET_QMM_F16)
            launch(naive_w4a16_kernel<HIDET_QMM_F16>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap0, lda, wp, sp, bp, cp0, m, k, n, group);
        else
            launch(naive_w4a16_kernel<HIDET_QMM_BF16>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap0, lda, wp, sp, bp, cp0, m, k, n, group);
        return;
    }
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    const SkinnyPlan plan = skinny_make_plan(k, n, parallel_k_parts, int(std::min<int64_t>(16, m)), ws.mailbox_bytes, false, /*flat_ok=*/false, device_cus());
    // a wave's run of rows and the scale table are addressed with 31-bit offsets
    if ((cdiv(cdiv(skinny_units(plan), plan.groups), kSkinnyWaves) * 32 + 64) * (n / 2) >= (int64_t(1) << 31) - (1 << 20) ||
        (k / group) * n * 2 >= (int64_t(1) << 31) - (1 << 20)) {
        if (dtype == HIDET_QMM_F16)
            launch(naive_w4a16_kernel<HIDET_QMM_F16>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap0, lda, wp, sp, bp, cp0, m, k, n, group);
        else
            launch(naive_w4a16_kernel<HIDET_QMM_BF16>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap0, lda, wp, sp, bp, cp0, m, k, n, group);
        return;
    }
    // 16-byte activation loads through a buffer descriptor: aligned rows, offsets below 2^31
    const bool aligned_a = (k % 8 == 0) && (lda % 8 == 0) && aligned(a, 16) && (15 * lda + k) * 2 < (int64_t(1) << 31) - (1 << 20);
    uint32_t *lost_flag = ws.counters != nullptr ? ws.counters + kExchangeLostWord : nullptr;
    for (int64_t m0 = 0; m0 < m; m0 += 16) {
        const int mt = int(std::min<int64_t>(16, m - m0));
        const size_t shmem = skinny_lds_bytes(mt, kSkinnyWaves);
        auto go = [&](auto kern) {
            if (shmem > 65536) allow_dynamic_lds(reinterpret_cast<const void *>(kern), int(skinny_lds_bytes(16, kSkinnyWaves)));  // the most any m needs
            launch(kern, dim3(skinny_grid(plan)), dim3(64 * kSkinnyWaves), shmem, stream, plan.ksteps, plan.ksteps_magic, plan.per_group, plan.longer, plan.splits, plan.splits_magic,
                   wp, ap0 + m0 * lda, lda, mt, int(k), int(n), group, static_cast<SkinnyPlanRest>(plan), sp, bp, cp0 + m0 * n, ws.mailbox,
                   lost_flag);
        };
        if (dtype == HIDET_QMM_F16) {
            if (bias != nullptr) {
                if (aligned_a) go(skinny_w4a16_kernel<HIDET_QMM_F16, true, true>);
                else go(skinny_w4a16_kernel<HIDET_QMM_F16, false, true>);
            } else {
                if (aligned_a) go(skinny_w4a16_kernel<HIDET_QMM_F16, true, false>);
                else go(skinny_w4a16_kernel<HIDET_QMM_F16, false, false>);
            }
        } else {
            if (bias != nullptr) {
                if (aligned_a) go(skinny_w4a16_kernel<HIDET_QMM_BF16, true, true>);
                else go(skinny_w4a16_kernel<HIDET_QMM_BF16, false, true>);
            } else {
                if (aligned_a) go(skinny_w4a16_kernel<HIDET_QMM_BF16, true, false>);
                else go(skinny_w4a16_kernel<HIDET_QMM_BF16, false, false>);
            }
        }
    }
}

}  // namespace qmm
