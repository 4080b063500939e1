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
// zero), so M = 1 and M = 16 cost the same.  K is split over the waves of a workgroup (LDS
// reduction) and over workgroups (skinny_finish: the workgroup of a column tile's last K slice adds
// the partial tiles in a fixed order, applies the scale and writes float16).
//
// The weight loads carry the non-temporal hint: the matrix is read once, and keeping it out of the
// way of the caches was measured 0.5 us faster at 4096 x 11008.  A wave has one step (8 loads, 8 KiB)
// in flight at a time; deeper queues per wave were measured slower on this memory system (two steps:
// +0.3 us, four: +2 us), the waves of a CU overlap each other's waits instead.
#include "skinny_common.h"

namespace qmm {
namespace {

constexpr int kTileN = kSkinnyTileN;
constexpr int kNonTemporal = 2;  // cache policy bits of a buffer load: sc0 = 1, nt = 2, sc1 = 16

// One 32-row step of a wave: the eight 16-byte row segments a lane holds and its activation fragment.
struct SkinnyStep {
    uint4v_t raw[8];
    half8_t xa;
};

template <bool ALIGNED_A, int WAVES, int RING>
__global__ __launch_bounds__(64 * WAVES) void skinny_w8a16_kernel(const _Float16 *__restrict__ a, int64_t lda,
                                                                  const int8_t *__restrict__ w,
                                                                  const _Float16 *__restrict__ scale,
                                                                  const _Float16 *__restrict__ bias, _Float16 *__restrict__ c,
                                                                  int m, int k, int n, int rows_per_block, int splits, int tiles,
                                                                  float *__restrict__ mailbox) {
    extern __shared__ float red[];  // [WAVES][m][kSkinnyRedStride]

    int tile, split;
    if (!skinny_tile_of_block(splits, tiles, &tile, &split)) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, cl = lane & 15;
    const int tile_col = tile * kTileN;
    const bool col_ok = tile_col + cl * 16 < n;

    const int rows_per_wave = rows_per_block / WAVES;
    const int k_begin = split * rows_per_block + wave * rows_per_wave;
    const int k_end = min(k, k_begin + rows_per_wave);
    const int nsteps = k_end > k_begin ? (k_end - k_begin + 31) >> 5 : 0;
    const int ngroups = (nsteps + RING - 1) / RING;

    // the column factors this thread applies at the very end: fetched now, not looked at before then (a use here would
    // wait for the load before the first weight load is issued)
    const SkinnyScale col_scale = skinny_fetch_scale(scale, bias, tile_col, n, m, splits, WAVES);

    float4_t acc[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    float4_t xsum = {0.f, 0.f, 0.f, 0.f};
    half8_t ones;
#pragma unroll
    for (int j = 0; j < 8; ++j) ones[j] = _Float16(1.0f);

    // Weights: a buffer that starts at the wave's first row and the tile's first column and ends with row k_end - 1, so
    // rows past the wave's range read as zero without a condition in the loop (the whole offset sits in the per-lane
    // register: the scalar offset of a buffer load is not range-checked). Such a row then counts as code 0 whatever the
    // activation is. A lane whose 16 columns lie past N reads the tile's first columns; its results are never stored.
    const int64_t w_bytes = int64_t(k_end - k_begin) * n - tile_col;
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(w + int64_t(k_begin) * n + tile_col), 0, int(w_bytes < 0 ? 0 : w_bytes), 0x00020000);
    // offset of row 8g of the next step to be issued; kept opaque so that it stays one register instead of one per load
    uint32_t w_off = uint32_t(8 * g) * uint32_t(n) + (col_ok ? cl * 16 : 0);
    // Activations: 8 consecutive k of row cl per step; rows >= m and k >= K get an offset outside the buffer (zero).
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(a), 0, ALIGNED_A ? int((int64_t(m - 1) * lda + k) * 2) : 0, 0x00020000);
    const _Float16 *ap = a + int64_t(cl) * lda;
    const int a_row_off = int(int64_t(cl) * lda * 2);

    auto issue = [&](SkinnyStep &st, int step) {
#pragma unroll
        for (int r = 0; r < 8; ++r)
            st.raw[r] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, w_off + uint32_t(r) * uint32_t(n), 0, kNonTemporal);
        w_off += 32u * uint32_t(n);
        asm volatile("" : "+v"(w_off));
        const int kx = k_begin + 32 * step + 8 * g;
        if (ALIGNED_A) {
            const int off = (cl < m && kx < k) ? a_row_off + kx * 2 : 0x7FFFFFF0;
            st.xa = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, off, 0, 0));
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) st.xa[e] = (cl < m && kx + e < k) ? ap[kx + e] : _Float16(0.0f);
        }
    };
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
    // exactly the loads issued behind the step that is about to be computed. Steps past the wave's range read zeros.
    if (ngroups > 0) {
        SkinnyStep ring[RING];
#pragma unroll
        for (int j = 0; j < RING; ++j) issue(ring[j], j);
        for (int grp = 1; grp < ngroups; ++grp) {
#pragma unroll
            for (int j = 0; j < RING; ++j) {
                compute(ring[j]);
                issue(ring[j], grp * RING + j);
            }
        }
#pragma unroll
        for (int j = 0; j < RING; ++j) compute(ring[j]);
    }

#pragma unroll
    for (int t = 0; t < 16; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[t][v] -= 1152.0f * xsum[v];
    skinny_finish<_Float16, WAVES>(acc, m, n, tile, split, splits, col_scale, c, mailbox, red);
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
    c[o] = _Float16(fmaf(acc, float(scale[j]), bias != nullptr ? float(bias[j]) : 0.0f));
}

}  // namespace

void skinny_w8a16_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                         int64_t n, int64_t lda, int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                         bool strict_workspace, hipStream_t stream) {
    const bool fast = (n % 16 == 0) && aligned(w, 16) && aligned(scale, 8) && aligned(bias, 8) && k > 0;  // 8-byte scale and bias loads
    const int waves = 8;
    int rpb = 0, splits = 0, tiles = 0;
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    if (fast) {
        skinny_plan_one_round(k, n, waves, parallel_k_parts, &rpb, &splits, &tiles);
        skinny_fit_mailbox(k, 32 * waves, tiles, int(std::min<int64_t>(16, m)), ws.mailbox_bytes, strict_workspace, &rpb, &splits);
    }
    // a wave's K range is addressed with 31-bit offsets
    if (!fast || (int64_t(rpb) / waves + 160) * n >= (int64_t(1) << 31) - (1 << 20)) {
        launch(naive_w8a16_kernel, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, static_cast<const _Float16 *>(a), lda,
               static_cast<const int8_t *>(w), static_cast<const _Float16 *>(scale), static_cast<const _Float16 *>(bias),
               static_cast<_Float16 *>(c), m, k, n);
        return;
    }
    // 16-byte activation loads through a buffer descriptor: aligned rows, offsets below 2^31
    const bool aligned_a = (k % 8 == 0) && (lda % 8 == 0) && aligned(a, 16) && (15 * lda + k) * 2 < (int64_t(1) << 31) - (1 << 20);
    const int grid = int(cdiv(tiles, 8) * 8 * splits);
    for (int64_t m0 = 0; m0 < m; m0 += 16) {
        const int mt = int(std::min<int64_t>(16, m - m0));
        const _Float16 *ap = static_cast<const _Float16 *>(a) + m0 * lda;
        _Float16 *cp = static_cast<_Float16 *>(c) + m0 * n;
        const size_t shmem = skinny_lds_bytes(mt, waves);
        auto go = [&](auto kern) {
            if (shmem > 65536) allow_dynamic_lds(reinterpret_cast<const void *>(kern), int(skinny_lds_bytes(16, waves)));  // the most any m needs
            launch(kern, dim3(grid), dim3(64 * waves), shmem, stream, ap, lda, static_cast<const int8_t *>(w),
                   static_cast<const _Float16 *>(scale), static_cast<const _Float16 *>(bias), cp, mt, int(k), int(n), rpb, splits,
                   tiles, ws.mailbox);
        };
        if (aligned_a) go(skinny_w8a16_kernel<true, 8, 1>);
        else go(skinny_w8a16_kernel<false, 8, 1>);
    }
}

}  // namespace qmm
