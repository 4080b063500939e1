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
// (skinny_tile_of: workgroup `bid` of a launch of cdiv(tiles, 8) * 8 * splits workgroups; a pure function so that the
// host can enumerate a launch, as the tests do.)
__host__ __device__ __forceinline__ bool skinny_tile_of(int bid, int splits, int tiles, int *tile, int *split) {
    const int rest = bid >> 3;
    *split = rest % splits;
    *tile = (rest / splits) * 8 + (bid & 7);
    return *tile < tiles;
}
__device__ __forceinline__ bool skinny_tile_of_block(int splits, int tiles, int *tile, int *split) {
    return skinny_tile_of(int(blockIdx.x), splits, tiles, tile, split);
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
        }
    }
    if (m > 1) {
        // 256 threads = 4 row lanes x 64 column quads: thread (rl, cq) sums rows rl, rl + 4, ... of columns 4cq .. 4cq+3
        // with 16-byte agent-scope loads, two rows x eight splits = 16 loads in flight, each row added in split order.
        const int cq = tid & 63, rl = tid >> 6;
        const int col4 = tile * kSkinnyTileN + cq * 4;
        if (col4 < n) {  // n is a multiple of 16 on this path: the quad is in or out as a whole
            constexpr int kAgentScope = 1 << 4;  // sc1
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
                partials + int64_t(tile) * splits * m * kSkinnyTileN, 0, splits * m * kSkinnyTileN * 4, 0x00020000);
            float s4[4] = {1.f, 1.f, 1.f, 1.f};
            if (col_scale != nullptr) {
#pragma unroll
                for (int e = 0; e < 4; ++e) s4[e] = float(col_scale[col4 + e]);
            }
            for (int row0 = rl; row0 < m; row0 += 8) {
                float4_t v[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
                for (int sp0 = 0; sp0 < splits; sp0 += 8) {
                    uint4v_t part[2][8];
#pragma unroll
                    for (int r = 0; r < 2; ++r)
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            const int row = row0 + 4 * r, sp = sp0 + u;
                            // past the last row or split: an offset outside the buffer, which reads as zero
                            const int off = (row < m && sp < splits) ? ((sp * m + row) * kSkinnyTileN + cq * 4) * 4 : 0x7FFFFFF0;
                            part[r][u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, kAgentScope);
                        }
#pragma unroll
                    for (int r = 0; r < 2; ++r)
#pragma unroll
                        for (int u = 0; u < 8; ++u) v[r] += __builtin_bit_cast(float4_t, part[r][u]);
                }
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const int row = row0 + 4 * r;
                    if (row < m) {
                        uint16_t h[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) h[e] = __builtin_bit_cast(uint16_t, skinny_to_out<OutT>(v[r][e] * s4[e]));
                        *reinterpret_cast<uint2 *>(c + int64_t(row) * n + col4) =
                            uint2{uint32_t(h[0]) | (uint32_t(h[1]) << 16), uint32_t(h[2]) | (uint32_t(h[3]) << 16)};
                    }
                }
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

// Bytes of workspace a skinny launch with `splits` K slices touches: the counters and one fp32 partial tile per
// (column tile, K slice) of `rows` (at most 16) activation rows. One slice exchanges nothing.
inline int64_t skinny_workspace_need(int tiles, int splits, int rows) {
    return splits > 1 ? kCounterBytes + int64_t(tiles) * splits * rows * kSkinnyTileN * 4 : 0;
}

// Makes the plan fit the caller's workspace: fewer, longer K slices (down to one, which needs no workspace) when the
// partial tiles would not fit. `strict` callers get an error instead, naming the bytes the plan needs.
inline void skinny_fit_workspace(int64_t k, int granule, int tiles, int rows, const void *workspace, int64_t workspace_bytes,
                                 bool strict, int *rows_per_block, int *splits) {
    const int64_t avail = workspace != nullptr ? workspace_bytes : 0;
    const int64_t need = skinny_workspace_need(tiles, *splits, rows);
    if (need <= avail) return;
    if (strict) QMM_FAIL("scratch too small for this shape: the K split needs " << need << " bytes, " << avail << " are there");
    const int64_t per_split = int64_t(tiles) * rows * kSkinnyTileN * 4;
    int64_t fit = avail > kCounterBytes ? (avail - kCounterBytes) / per_split : 1;
    fit = std::max<int64_t>(1, std::min<int64_t>(fit, *splits));
    const int64_t rpb = cdiv(cdiv(k, fit), granule) * granule;
    *rows_per_block = int(rpb);
    *splits = int(cdiv(k, rpb));
}

}  // namespace qmm
