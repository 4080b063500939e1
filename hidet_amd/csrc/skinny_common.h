// Shared tail of the bandwidth-bound skinny kernels (M <= 16 rows per pass, 256-column tiles, 4 waves
// per workgroup that split K): LDS reduction over the waves, then either a direct store or the
// cross-workgroup split-K exchange.
#pragma once
#include "common.h"

namespace qmm {

constexpr int kSkinnyTileN = 256;
constexpr int kSkinnyWaves = 4;
constexpr int kSkinnyRedStride = 272;  // 16 lanes x 17 floats: conflict-free LDS writes
constexpr int kMaxSkinnyTiles = int(kCounterBytes / 4);

inline size_t skinny_lds_bytes(int m) { return size_t(kSkinnyWaves) * m * kSkinnyRedStride * sizeof(float); }

template <typename OutT>
__device__ __forceinline__ OutT skinny_to_out(float v);
template <>
__device__ __forceinline__ _Float16 skinny_to_out<_Float16>(float v) { return _Float16(v); }
template <>
__device__ __forceinline__ uint16_t skinny_to_out<uint16_t>(float v) { return f32_to_bf16_bits(v); }  // bfloat16 bits

// Workgroup -> (column tile, K split).  Workgroups are dealt round-robin to the 8 XCDs: every K split
// of a column tile gets the same residue mod 8, so the partial tiles of a column tile meet in one L2.
__device__ __forceinline__ bool skinny_tile_of_block(int splits, int tiles, int *tile, int *split) {
    const int bid = blockIdx.x;
    const int rest = bid >> 3;
    *split = rest % splits;
    *tile = (rest / splits) * 8 + (bid & 7);
    return *tile < tiles;
}

// res[t][v] is this lane's partial sum for output row 4 * (lane / 16) + v and column
// tile * 256 + (lane % 16) * 16 + t.  `red` is dynamic LDS of skinny_lds_bytes(m).
// col_scale (may be null) is a per-column float16 factor applied to the final sum.
//
// Cross-workgroup exchange without cache-wide fences: a partial tile is written with agent-scope
// (write-through) stores, their completion is awaited, and only then is the arrival counted; the
// last workgroup to arrive reads all partial tiles back with agent-scope loads and adds them in
// split order, so the result does not depend on arrival order.  A release/acquire fence pair here
// would write back and invalidate the whole L2 once per workgroup, which costs more than the GEMV.
template <typename OutT>
__device__ __forceinline__ void skinny_reduce_store(const float4_t (&res)[16], int m, int n, int tile, int split,
                                                    int splits, const _Float16 *__restrict__ col_scale,
                                                    OutT *__restrict__ c, float *__restrict__ partials,
                                                    uint32_t *__restrict__ counters, float *red, int *s_last) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, cl = lane & 15;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int row = 4 * g + v;
        if (row < m) {
            float *dst = red + (wave * m + row) * kSkinnyRedStride + cl * 17;
#pragma unroll
            for (int t = 0; t < 16; ++t) dst[t] = res[t][v];
        }
    }
    __syncthreads();

    const int col = tile * kSkinnyTileN + tid;
    const int ridx = tid + (tid >> 4);
    const float s = (col_scale != nullptr && col < n) ? float(col_scale[col]) : 1.0f;
    if (splits == 1) {
        if (col < n) {
            for (int row = 0; row < m; ++row) {
                float v = 0.f;
#pragma unroll
                for (int wv = 0; wv < kSkinnyWaves; ++wv) v += red[(wv * m + row) * kSkinnyRedStride + ridx];
                c[int64_t(row) * n + col] = skinny_to_out<OutT>(v * s);
            }
        }
        return;
    }

    float *mine = partials + (int64_t(tile) * splits + split) * m * kSkinnyTileN;
    for (int row = 0; row < m; ++row) {
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < kSkinnyWaves; ++wv) v += red[(wv * m + row) * kSkinnyRedStride + ridx];
        __hip_atomic_store(mine + row * kSkinnyTileN + tid, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): every store of this lane has been acknowledged
    __syncthreads();
    if (tid == 0) {
        const uint32_t old = __hip_atomic_fetch_add(&counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_last = (old == uint32_t(splits - 1));
    }
    __syncthreads();
    if (!*s_last) return;
    if (col < n) {
        const float *base = partials + int64_t(tile) * splits * m * kSkinnyTileN;
        if (m == 1) {
            float v = 0.f;
            for (int sp0 = 0; sp0 < splits; sp0 += 16) {  // 16 loads in flight, added in split order
                float part[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    part[u] = 0.f;
                    if (sp0 + u < splits)
                        part[u] = __hip_atomic_load(base + int64_t(sp0 + u) * kSkinnyTileN + tid, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) v += part[u];
            }
            c[col] = skinny_to_out<OutT>(v * s);
        } else {
            // rows in groups of 4, splits in groups of 4: 16 loads in flight, each row added in split order
            for (int row0 = 0; row0 < m; row0 += 4) {
                float v[4] = {0.f, 0.f, 0.f, 0.f};
                for (int sp0 = 0; sp0 < splits; sp0 += 4) {
                    float part[4][4];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            part[u][r] = 0.f;
                            if (sp0 + u < splits && row0 + r < m)
                                part[u][r] = __hip_atomic_load(base + (int64_t(sp0 + u) * m + row0 + r) * kSkinnyTileN + tid,
                                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
#pragma unroll
                    for (int u = 0; u < 4; ++u)
#pragma unroll
                        for (int r = 0; r < 4; ++r) v[r] += part[u][r];
                }
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (row0 + r < m) c[int64_t(row0 + r) * n + col] = skinny_to_out<OutT>(v[r] * s);
            }
        }
    }
    if (tid == 0) __hip_atomic_store(&counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // zero for the next call
}

// K split of a skinny launch. Each workgroup streams a slice of `rows_per_block` weight rows (a whole multiple of
// `granule` = 4 waves x one 32-row step) of its 256-column tile. Measured on K = 4096 .. 11008, N = 4096 .. 12288,
// M = 1 .. 16, int8 and int4 weights: slices of about `slice_rows` = 512 rows are fastest (768 for int8 weights with more
// than 8 activation rows, whose partial tiles cost more to exchange) - shorter ones pay for the partial-tile exchange,
// longer ones leave too few workgroups to keep HBM busy - and narrow outputs get more splits so that at least ~128
// workgroups run. `hint_parts` > 0 forces the split count.
inline void skinny_plan(int64_t k, int64_t n, int slice_rows, int hint_parts, int granule, int *rows_per_block, int *splits,
                        int *tiles) {
    const int64_t t = cdiv(n, kSkinnyTileN);
    int64_t want = hint_parts;
    if (want <= 0) want = std::max<int64_t>((k + slice_rows / 2) / slice_rows, cdiv(128, t));
    want = std::max<int64_t>(1, std::min<int64_t>(want, cdiv(k, granule)));
    const int64_t rpb = cdiv(cdiv(k, want), granule) * granule;
    *rows_per_block = int(rpb);
    *splits = int(cdiv(k, rpb));
    *tiles = int(t);
}

}  // namespace qmm
