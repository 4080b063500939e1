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
// zero), so M = 1 and M = 16 cost the same.  The (tile, 32-row step) units of the matrix are dealt
// evenly to the workgroups of the launch and, inside a workgroup, to its waves (SkinnyPlan): the waves'
// sums meet in LDS, the workgroups' partial tiles in the mailbox (skinny_tails: the workgroup that holds
// a column tile's last step adds the partial tiles in a fixed order, applies the scale and writes float16).
//
// The weight loads carry the non-temporal hint: the matrix is read once, and keeping it out of the
// way of the caches was measured 0.5 us faster at 4096 x 11008.  A wave has RING steps (8 loads, 8 KiB each)
// in flight at a time; the waves of a CU overlap each other's waits.
#include "skinny_common.h"

namespace qmm {
namespace {

constexpr int kTileN = kSkinnyTileN;
constexpr int kNonTemporal = 2;  // cache policy bits of a buffer load: sc0 = 1, nt = 2, sc1 = 16
// 32-row steps a wave keeps in flight, waves of a workgroup. Measured at 4096 x 11008, one row, against 10.2 us: two
// steps in flight 11.1 us; 12 waves 11.7 us, 16 waves 13.7 us (more loads under way per CU made every variant slower).
constexpr int kRing = 1, kWaves = 8;

// One 32-row step of a wave: the eight 16-byte row segments a lane holds and its activation fragment.
struct SkinnyStep {
    uint4v_t raw[8];
    half8_t xa;
};

template <bool ALIGNED_A, int WAVES, int RING, bool BIAS>
__global__ __launch_bounds__(64 * WAVES) void skinny_w8a16_kernel(int ksteps, uint32_t ksteps_magic, int per_group, int longer, int splits, uint32_t splits_magic,
                                                                  const int8_t *__restrict__ w, const _Float16 *__restrict__ a,
                                                                  int64_t lda, int m, int k, int n, SkinnyPlanRest plan_rest,
                                                                  const _Float16 *__restrict__ scale,
                                                                  const _Float16 *__restrict__ bias, _Float16 *__restrict__ c,
                                                                  float *__restrict__ mailbox, uint32_t *__restrict__ lost_flag) {
    extern __shared__ float red[];  // [WAVES][m][kSkinnyRedStride]

    const SkinnyPlanHead plan_head = {ksteps, ksteps_magic, per_group, longer, splits, splits_magic};
    const SkinnyPlan plan(plan_head, plan_rest);
    int grp;
    if (!skinny_group_of_block(plan_head, plan_rest.tiles, int(blockIdx.x), &grp)) return;
    const SkinnyWork wk = skinny_work_of(plan_head, grp);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, cl = lane & 15;
    static_assert(WAVES == 8 || WAVES == 4, "skinny_wave_run deals a run to at most 8 waves");
    int run_lo, run_hi, part;
    skinny_wave_run(wk, wave, WAVES, &run_lo, &run_hi, &part);

    // this workgroup's part in the exchange: worked out behind the wave's first loads (below), not looked at before the tail
    SkinnyRoles roles;
    auto learn_roles = [&]() {
        // an opaque zero in every input keeps this arithmetic - and the wait for the kernel arguments that arrive by a fetch -
        // where it is called: behind the wave's first loads, not before them
        int zero = 0;
        asm volatile("" : "+s"(zero));
        SkinnyPlan plan_now = plan;
        plan_now.per_group_magic += zero;
        plan_now.per_group1_magic += zero;
        const int grp_now = grp + zero;
        roles = skinny_roles_of(plan_now, skinny_work_of(plan_head, grp_now), grp_now, WAVES);
    };

    // Activations: 8 consecutive k of row cl per step; rows >= m and k >= K get an offset outside the buffer (zero).
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(a), 0, ALIGNED_A ? int((int64_t(m - 1) * lda + k) * 2) : 0, 0x00020000);
    const _Float16 *ap = a + int64_t(cl) * lda;
    const int a_row_off = int(int64_t(cl) * lda * 2);

    // The wave's run lies in one tile (skinny_wave_run). Weights: a buffer that starts at the run's first row and the tile's
    // first column and ends with row k_end - 1, so rows past the wave's range read as zero without a condition in the loop
    // (the whole offset sits in the per-lane register: the scalar offset of a buffer load is not range-checked). Such a
    // row then counts as code 0 whatever the activation is. A lane whose 16 columns lie past N reads the tile's first
    // columns; its results are never stored. Steps past the wave's range read zeros.
    const int tile = wk.tile + part;
    const int tile_col = tile * kTileN;
    const int k_begin = (run_lo - tile * plan.ksteps) * 32;
    const int k_end = min(k, (run_hi - tile * plan.ksteps) * 32);
    const int ngroups = (run_hi - run_lo + RING - 1) / RING;
    const int64_t w_bytes = int64_t(k_end - k_begin) * n - tile_col;
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(w + int64_t(k_begin) * n + tile_col), 0, int(w_bytes < 0 || ngroups == 0 ? 0 : w_bytes), 0x00020000);
    // offset of row 8g of the next step to be issued; kept opaque so that it stays one register instead of one per load
    uint32_t w_off = uint32_t(8 * g) * uint32_t(n) + (tile_col + cl * 16 < n ? cl * 16 : 0);
    SkinnyStep ring[RING];
    auto issue = [&](SkinnyStep &st, int step) {
#pragma unroll
        for (int r = 0; r < 8; ++r)
            st.raw[r] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, w_off + uint32_t(r) * uint32_t(n), 0, kNonTemporal);
        w_off += 32u * uint32_t(n);
        asm volatile("" : "+v"(w_off));
        const int kx = k_begin + 32 * step + 8 * g;
        if (ALIGNED_A) {
            const int off = (cl < m && kx < k_end) ? a_row_off + kx * 2 : 0x7FFFFFF0;
            st.xa = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, off, 0, 0));
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) st.xa[e] = (cl < m && kx + e < k_end) ? ap[kx + e] : _Float16(0.0f);
        }
    };
    // the wave's first loads leave before anything else is set up (of an empty run: nothing but zeros)
#pragma unroll
    for (int j = 0; j < RING; ++j) issue(ring[j], j);
    learn_roles();
    half8_t ones;
#pragma unroll
    for (int j = 0; j < 8; ++j) ones[j] = _Float16(1.0f);
    float4_t acc[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    float4_t xsum = {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const SkinnyStep &st) {
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            // selector: byte (t % 4) of the even row into bits 0-7, of the odd row into bits 16-23
            constexpr uint32_t kZero = 0x0c;
            const uint32_t sel = (kZero << 24) | (uint32_t(4 + (t & 3)) << 16) | (kZero << 8) | uint32_t(t & 3);
            union {
                uint32_t u[4];
                half8_t h8;
            } b;
#pragma unroll
            for (int p = 0; p < 4; ++p) b.u[p] = __builtin_amdgcn_perm(st.raw[2 * p + 1][t >> 2], st.raw[2 * p][t >> 2], sel) ^ 0x64806480u;
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(st.xa, b.h8, acc[t], 0, 0, 0);
        }
        xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(st.xa, ones, xsum, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);  // nothing of a later step may move up here: it would wait for that step's loads
    };
    // Straight-line groups of RING steps (no condition around a load or a step): the waits the compiler places then count
    // exactly the loads issued behind the step that is about to be computed.
    for (int sg = 1; sg < ngroups; ++sg) {
#pragma unroll
        for (int j = 0; j < RING; ++j) {
            compute(ring[j]);
            issue(ring[j], sg * RING + j);
        }
    }
#pragma unroll
    for (int j = 0; j < RING; ++j) compute(ring[j]);
#pragma unroll
    for (int t = 0; t < 16; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[t][v] -= 1152.0f * xsum[v];
    skinny_stash(acc, m, wave, red);
    // calls without a bias run the epilogue that never knew of one: every instruction behind the last weight counts
    const SkinnyScale col_scale = {scale, BIAS ? bias : nullptr};
    if constexpr (BIAS) skinny_tails<_Float16, WAVES>(plan, wk, roles, m, n, col_scale, c, mailbox, lost_flag, red);
    else skinny_tails<f16_unbiased_t, WAVES>(plan, wk, roles, m, n, col_scale, reinterpret_cast<f16_unbiased_t *>(c), mailbox, lost_flag, red);
}

// Any shape the fast kernel cannot take (N not a multiple of 16, misaligned weights): one thread per
// output element, serial K, fp32 accumulation.
__global__ __launch_bounds__(256) void naive_w8a16_kernel(const _Float16 *__restrict__ a, int64_t lda,
                                                          const int8_t *__restrict__ w, const _Float16 *__restrict__ scale,
                                                          const _Float16 *__restrict__ bias, _Float16 *__restrict__ c, int64_t m,
                                                          int64_t k, int64_t n) {
    const int64_t o = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (o >= m * n) return;
    const int64_t i = o / n, j = o - i * n;
    float acc = 0.f;
    for (int64_t kk = 0; kk < k; ++kk) acc += float(a[i * lda + kk]) * float(w[kk * n + j]);
    c[o] = scaled_biased_f16(acc, float(scale[j]), bias != nullptr ? float(bias[j]) : -0.0f);
}

}  // namespace

void skinny_w8a16_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                         int64_t n, int64_t lda, int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                         bool strict_workspace, hipStream_t stream) {
    // 8-byte scale and bias loads, column offsets in bytes below 2^31
    const bool fast = (n % 16 == 0) && n < (int64_t(1) << 30) && aligned(w, 16) && aligned(scale, 8) && aligned(bias, 8) && k > 0;
    constexpr int waves = kWaves;
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    SkinnyPlan plan;
    if (fast) plan = skinny_make_plan(k, n, parallel_k_parts, int(std::min<int64_t>(16, m)), ws.mailbox_bytes, strict_workspace, /*flat_ok=*/true, device_cus());
    // a wave's run of rows is addressed with 31-bit offsets
    if (!fast || (cdiv(cdiv(skinny_units(plan), plan.groups), waves) * 32 + 160) * n >= (int64_t(1) << 31) - (1 << 20)) {
        launch(naive_w8a16_kernel, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, static_cast<const _Float16 *>(a), lda,
               static_cast<const int8_t *>(w), static_cast<const _Float16 *>(scale), static_cast<const _Float16 *>(bias),
               static_cast<_Float16 *>(c), m, k, n);
        return;
    }
    // 16-byte activation loads through a buffer descriptor: aligned rows, offsets below 2^31
    const bool aligned_a = (k % 8 == 0) && (lda % 8 == 0) && aligned(a, 16) && (15 * lda + k) * 2 < (int64_t(1) << 31) - (1 << 20);
    uint32_t *lost_flag = ws.counters != nullptr ? ws.counters + kExchangeLostWord : nullptr;
    for (int64_t m0 = 0; m0 < m; m0 += 16) {
        const int mt = int(std::min<int64_t>(16, m - m0));
        const _Float16 *ap = static_cast<const _Float16 *>(a) + m0 * lda;
        _Float16 *cp = static_cast<_Float16 *>(c) + m0 * n;
        const size_t shmem = skinny_lds_bytes(mt, waves);
        auto go = [&](auto kern) {
            if (shmem > 65536) allow_dynamic_lds(reinterpret_cast<const void *>(kern), int(skinny_lds_bytes(16, waves)));  // the most any m needs
            launch(kern, dim3(skinny_grid(plan)), dim3(64 * waves), shmem, stream, plan.ksteps, plan.ksteps_magic, plan.per_group, plan.longer, plan.splits, plan.splits_magic,
                   static_cast<const int8_t *>(w), ap, lda, mt, int(k), int(n), static_cast<SkinnyPlanRest>(plan),
                   static_cast<const _Float16 *>(scale), static_cast<const _Float16 *>(bias), cp, ws.mailbox, lost_flag);
        };
        if (bias != nullptr) {
            if (aligned_a) go(skinny_w8a16_kernel<true, waves, kRing, true>);
            else go(skinny_w8a16_kernel<false, waves, kRing, true>);
        } else {
            if (aligned_a) go(skinny_w8a16_kernel<true, waves, kRing, false>);
            else go(skinny_w8a16_kernel<false, waves, kRing, false>);
        }
    }
}

}  // namespace qmm
