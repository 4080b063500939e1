// Shared parts of the bandwidth-bound skinny kernels (M <= 16 rows per pass, 256-column tiles, the waves of a
// workgroup split its K slice): the launch plan, the LDS reduction over the waves and the split-K exchange
// between workgroups.
#pragma once
#include "common.h"

namespace qmm {

constexpr int kSkinnyTileN = 256;
// LDS reduction tile: one row of 256 floats per (wave, activation row), 1040 bytes apart, as 64 chunks of 16 bytes. The
// chunk of columns 4c .. 4c+3 sits at position skinny_red_chunk(c). A lane (g, cl) of the main loop writes the four
// chunks 4cl .. 4cl+3 of rows 4g .. 4g+3 with 16-byte stores: the row pitch puts the four g of an instruction into
// different quarters of the 64 banks (4 rows = 16 x 256 + 64 bytes) and the permutation spreads the four lanes that
// share a quarter over its four 16-byte slots, so an instruction takes the four passes its 1 KiB needs and no more.
// Readers fetch whole chunks (or single floats of them) of consecutive columns: every bank once per 256 bytes.
constexpr int kSkinnyRedStride = 260;  // floats
__device__ __forceinline__ int skinny_red_chunk(int c) { return (c & ~3) | ((c ^ (c >> 4)) & 3); }

inline size_t skinny_lds_bytes(int m, int waves) { return size_t(waves) * m * kSkinnyRedStride * sizeof(float); }

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

// The tail of a bandwidth-bound kernel: LDS reduction over the WAVES waves of a workgroup, then either the final store or
// the split-K exchange through the mailbox.
//
// res[t][v] is this lane's partial sum for output row 4 * (lane / 16) + v and column tile * 256 + (lane % 16) * 16 + t.
// `red` is dynamic LDS of skinny_lds_bytes(m, WAVES). col_scale holds the column factors and biases this thread applies
// to its outputs (SkinnyScale: the caller fetches them with skinny_fetch_scale before its main loop, so that no load
// sits between the last weight and the output).
//
// Who does what in the tail: in the column layout thread tid owns column tid % 256 of rows tid / 256, tid / 256 + WAVES / 4,
// ... (one dword per access, four waves per row); in the quad layout it owns columns 4 (tid % 64) .. + 3 of rows tid / 64,
// tid / 64 + WAVES, ... (16 bytes per access, one wave per row). Either way every wave has work: the same bytes moved
// by a single wave were measured 1 us slower per launch, and every batch of reads from the mailbox costs a round trip
// to the memory side (1.5 to 2 us), so a thread wants all its reads in one batch of 16. The column layout is the faster
// one per byte (8 rows at 4096 x 11008: 12.9 against 13.3 us) and is used whenever its reads fit that one batch
// (skinny_column_layout).
//
// Exchange: the mailbox holds one fp32 tile [m][256] per (column tile, K slice) and is all zero between launches. Every
// slice but the last stores its tile (agent scope, +0.0 sent as -0.0, so a stored word is never zero) and is done: no
// acknowledgement, no counter. The workgroup of the LAST slice - the highest workgroup index of the column tile, so all
// the others were dispatched before it - reads the tiles back until no word is zero, adds them in slice order (its own
// last: the result does not depend on timing), writes the output and puts the zeros back with plain stores, which the
// end of the kernel makes visible to the next launch. The wait is bounded: after kSkinnySpinLimit re-reads the output
// is NaN instead of a hang.
constexpr int kSkinnySpinLimit = 1 << 20;

// Column factors of a thread for both thread layouts of the tail, fetched by the caller before its main loop and not
// looked at there (a use would make the first weight load wait for them).
struct SkinnyScale {
    _Float16 one = _Float16(1.0f);                                                    // column tid % 256
    half4_t quad = {_Float16(1.0f), _Float16(1.0f), _Float16(1.0f), _Float16(1.0f)};  // columns 4 (tid % 64) .. + 3
    _Float16 bias_one = _Float16(0.0f);                                               // added after the scale
    half4_t bias_quad = {_Float16(0.0f), _Float16(0.0f), _Float16(0.0f), _Float16(0.0f)};
};
// Which of the tail's two thread layouts a launch uses: one column per thread (dwords, `waves / 4` rows at a time) while a
// thread's reads of the exchange fit one batch of 16 - rows per thread x other slices, in the shapes collect<LG> has:
// 4 x 4, 2 x 8 or 1 x 16 - and whenever nothing is exchanged and there are few rows; else four columns per thread.
__device__ __forceinline__ bool skinny_column_layout(int m, int splits, int waves) {
    const int row_groups = waves / 4, rows = (m + row_groups - 1) / row_groups, others = splits - 1;
    if (others == 0) return m <= 4;
    return (rows <= 4 && others <= 4) || (rows <= 2 && others <= 8) || (rows <= 1 && others <= 16);
}

// `bias` may be null (no bias). 8-byte loads in the quad layout: scale and bias 8-byte aligned, n a multiple of 4.
__device__ __forceinline__ SkinnyScale skinny_fetch_scale(const _Float16 *scale, const _Float16 *bias, int tile_col, int n, int m,
                                                          int splits, int waves) {
    SkinnyScale s;
    const int tid = threadIdx.x;
    if (skinny_column_layout(m, splits, waves)) {
        const int col = tile_col + (tid & 255);
        if (col < n) {
            s.one = scale[col];
            if (bias != nullptr) s.bias_one = bias[col];
        }
    } else {
        const int col = tile_col + (tid & 63) * 4;
        if (col < n) {
            s.quad = *reinterpret_cast<const half4_t *>(scale + col);
            if (bias != nullptr) s.bias_quad = *reinterpret_cast<const half4_t *>(bias + col);
        }
    }
    return s;
}

// CW columns per thread: the word a thread moves is one dword or four. Agent scope (sc1): loads bypass the L1, stores
// write through.
template <int CW>
struct SkinnyWord;
template <>
struct SkinnyWord<1> {
    typedef uint32_t type;
    static __device__ __forceinline__ type absent() { return 0x80000000u; }  // -0.0: adds nothing, counts as arrived
    static __device__ __forceinline__ bool has_zero(type v) { return v == 0u; }
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 1 << 4); }
    static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, int off, type v) { __builtin_amdgcn_raw_buffer_store_b32(v, r, off, 0, 1 << 4); }
    static __device__ __forceinline__ void clear(__amdgpu_buffer_rsrc_t r, int off) { __builtin_amdgcn_raw_buffer_store_b32(0u, r, off, 0, 0); }
    static __device__ __forceinline__ type never_zero(type v) { return v == 0u ? 0x80000000u : v; }
    static __device__ __forceinline__ float get(type v, int) { return __uint_as_float(v); }
};
template <>
struct SkinnyWord<4> {
    typedef uint4v_t type;
    static __device__ __forceinline__ type absent() { return type{0x80000000u, 0x80000000u, 0x80000000u, 0x80000000u}; }
    static __device__ __forceinline__ bool has_zero(type v) { return v[0] == 0u || v[1] == 0u || v[2] == 0u || v[3] == 0u; }
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int off) { return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 1 << 4); }
    static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, int off, type v) { __builtin_amdgcn_raw_buffer_store_b128(v, r, off, 0, 1 << 4); }
    static __device__ __forceinline__ void clear(__amdgpu_buffer_rsrc_t r, int off) { __builtin_amdgcn_raw_buffer_store_b128(type{0u, 0u, 0u, 0u}, r, off, 0, 0); }
    static __device__ __forceinline__ type never_zero(type v) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (v[e] == 0u) v[e] = 0x80000000u;
        return v;
    }
    static __device__ __forceinline__ float get(type v, int e) { return __uint_as_float(v[e]); }
};

template <typename OutT, int WAVES, int CW>
struct SkinnyTail {
    typedef SkinnyWord<CW> W;
    typedef typename W::type Word;
    static constexpr int kThreadsPerRow = kSkinnyTileN / CW;                // 256 or 64
    static constexpr int kRowGroups = WAVES * 64 / kThreadsPerRow;         // rows the workgroup handles at a time
    static_assert(WAVES % 4 == 0, "whole rows of threads");
    int m, n, row_first, col_in_tile;
    int64_t out_col;
    const float *red;
    float scale[CW], bias[CW];
    OutT *c;

    struct Vals {
        float v[CW];
    };
    __device__ __forceinline__ Vals own(int row) const {
        const float *src = red + row * kSkinnyRedStride + skinny_red_chunk(col_in_tile >> 2) * 4 + (col_in_tile & 3);  // CW columns never straddle a chunk
        Vals r;
#pragma unroll
        for (int e = 0; e < CW; ++e) r.v[e] = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) {
            if constexpr (CW == 4) {
                const float4_t q = *reinterpret_cast<const float4_t *>(src + wv * m * kSkinnyRedStride);
#pragma unroll
                for (int e = 0; e < 4; ++e) r.v[e] += q[e];
            } else {
                r.v[0] += src[wv * m * kSkinnyRedStride];
            }
        }
        return r;
    }
    __device__ __forceinline__ void store(int row, const Vals &x) const {
        OutT *dst = c + int64_t(row) * n + out_col;
        if constexpr (CW == 1) {
            dst[0] = skinny_to_out<OutT>(fmaf(x.v[0], scale[0], bias[0]));
        } else {
            uint16_t h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = __builtin_bit_cast(uint16_t, skinny_to_out<OutT>(fmaf(x.v[e], scale[e], bias[e])));
            // 8 bytes at once when the row starts allow it (n a multiple of 4 is given, the base pointer may not be aligned)
            if ((reinterpret_cast<uintptr_t>(dst) & 7) == 0) {
                *reinterpret_cast<uint2 *>(dst) = uint2{uint32_t(h[0]) | (uint32_t(h[1]) << 16), uint32_t(h[2]) | (uint32_t(h[3]) << 16)};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) reinterpret_cast<uint16_t *>(dst)[e] = h[e];
            }
        }
    }
    static __device__ __forceinline__ Word pack(const Vals &x) {
        if constexpr (CW == 1) {
            return W::never_zero(__float_as_uint(x.v[0]));
        } else {
            return W::never_zero(Word{__float_as_uint(x.v[0]), __float_as_uint(x.v[1]), __float_as_uint(x.v[2]), __float_as_uint(x.v[3])});
        }
    }

    // A slice that is not the last: send the partial tile.
    __device__ __forceinline__ void send(__amdgpu_buffer_rsrc_t box, int split) const {
#pragma unroll 1
        for (int row = row_first; row < m; row += kRowGroups)
            W::store(box, ((split * m + row) * kSkinnyTileN + col_in_tile) * 4, pack(own(row)));
    }

    // The last slice: 16 reads in flight, (16 >> LG) rows x (1 << LG) slices per trip.
    template <int LG>
    __device__ __forceinline__ void collect(__amdgpu_buffer_rsrc_t box, int others) const {
        constexpr int kRows = 16 >> LG, kSlices = 1 << LG;
#pragma unroll 1
        for (int row0 = row_first; row0 < m; row0 += kRows * kRowGroups) {
            Vals total[kRows];
#pragma unroll
            for (int r = 0; r < kRows; ++r) {
                if (row0 + r * kRowGroups < m) total[r] = own(row0 + r * kRowGroups);
                else
#pragma unroll
                    for (int e = 0; e < CW; ++e) total[r].v[e] = 0.f;
            }
            bool lost = false;
            // the sum runs over the slices in order and ends with this workgroup's own part: keep `total` for last
            Vals others_sum[kRows];
#pragma unroll
            for (int r = 0; r < kRows; ++r)
#pragma unroll
                for (int e = 0; e < CW; ++e) others_sum[r].v[e] = 0.f;
#pragma unroll 1
            for (int sp0 = 0; sp0 < others; sp0 += kSlices) {
                Word bits[16];
                int off[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const int row = row0 + (u >> LG) * kRowGroups, sp = sp0 + (u & (kSlices - 1));
                    off[u] = (row < m && sp < others) ? ((sp * m + row) * kSkinnyTileN + col_in_tile) * 4 : -1;
                    bits[u] = W::absent();
                    if (off[u] >= 0) bits[u] = W::load(box, off[u]);
                }
#pragma unroll 1
                for (int spin = 0;; ++spin) {
                    bool missing = false;
#pragma unroll
                    for (int u = 0; u < 16; ++u) missing |= W::has_zero(bits[u]);
                    if (!missing) break;
                    if (spin == kSkinnySpinLimit) {
                        lost = true;
                        break;
                    }
                    asm volatile("" ::: "memory");  // the mailbox changes under the loop: the reads below are issued again
#pragma unroll
                    for (int u = 0; u < 16; ++u)
                        if (W::has_zero(bits[u])) bits[u] = W::load(box, off[u]);
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) {
#pragma unroll
                    for (int e = 0; e < CW; ++e) others_sum[u >> LG].v[e] += W::get(bits[u], e);
                    if (off[u] >= 0) W::clear(box, off[u]);
                }
            }
#pragma unroll
            for (int r = 0; r < kRows; ++r) {
                const int row = row0 + r * kRowGroups;
                if (row < m) {
                    Vals out;
#pragma unroll
                    for (int e = 0; e < CW; ++e) out.v[e] = lost ? __builtin_nanf("") : others_sum[r].v[e] + total[r].v[e];
                    store(row, out);
                }
            }
        }
    }

    __device__ __forceinline__ void run(int tile, int split, int splits, float *mailbox) const {
        if (splits == 1) {
#pragma unroll 1
            for (int row = row_first; row < m; row += kRowGroups) store(row, own(row));
            return;
        }
        const int others = splits - 1;
        const __amdgpu_buffer_rsrc_t box = __builtin_amdgcn_make_buffer_rsrc(mailbox + int64_t(tile) * splits * m * kSkinnyTileN, 0,
                                                                             others * m * kSkinnyTileN * 4, 0x00020000);
        if (split != others) {
            send(box, split);
            return;
        }
        const int my_rows = (m - row_first + kRowGroups - 1) / kRowGroups;
        if (others <= 4 && my_rows > 2) collect<2>(box, others);
        else if (others <= 8 && my_rows > 1) collect<3>(box, others);
        else collect<4>(box, others);
    }
};

template <typename OutT, int WAVES>
__device__ __forceinline__ void skinny_finish(const float4_t (&res)[16], int m, int n, int tile, int split, int splits,
                                              const SkinnyScale &col_scale, OutT *__restrict__ c, float *__restrict__ mailbox,
                                              float *red) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, cl = lane & 15;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int row = 4 * g + v;
        if (row < m) {
            float *dst = red + (wave * m + row) * kSkinnyRedStride;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<float4_t *>(dst + skinny_red_chunk(4 * cl + j) * 4) =
                    float4_t{res[4 * j][v], res[4 * j + 1][v], res[4 * j + 2][v], res[4 * j + 3][v]};
        }
    }
    __syncthreads();

    if (skinny_column_layout(m, splits, WAVES)) {
        SkinnyTail<OutT, WAVES, 1> tail;
        tail.m = m;
        tail.n = n;
        tail.row_first = __builtin_amdgcn_readfirstlane(tid >> 8);  // the same for a whole wave: row and slice tests are scalar
        tail.col_in_tile = tid & 255;
        tail.out_col = int64_t(tile) * kSkinnyTileN + tail.col_in_tile;
        tail.red = red;
        tail.scale[0] = float(col_scale.one);
        tail.bias[0] = float(col_scale.bias_one);
        tail.c = c;
        if (tail.out_col < n && tail.row_first < m) tail.run(tile, split, splits, mailbox);
    } else {
        SkinnyTail<OutT, WAVES, 4> tail;
        tail.m = m;
        tail.n = n;
        tail.row_first = __builtin_amdgcn_readfirstlane(tid >> 6);
        tail.col_in_tile = (tid & 63) * 4;
        tail.out_col = int64_t(tile) * kSkinnyTileN + tail.col_in_tile;
        tail.red = red;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            tail.scale[e] = float(col_scale.quad[e]);
            tail.bias[e] = float(col_scale.bias_quad[e]);
        }
        tail.c = c;
        if (tail.out_col < n && tail.row_first < m) tail.run(tile, split, splits, mailbox);  // n is a multiple of 16: a quad is in or out as a whole
    }
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

// K split of the int8 kernel, whose workgroups have `waves` waves: one round of one workgroup per CU. Measured on
// K = 4096 .. 14336, N = 1024 .. 32000: the fastest split is the largest whose workgroups still fit the 256 CUs at once
// (43 column tiles: 4 or 5 slices 11.3 us, 6 slices = 258 workgroups 13.9 us; 112 tiles: 2 slices 39 us, 4 slices
// 41 us), with at least two 32-row steps per wave (512 rows per 8-wave workgroup). `hint_parts` > 0 forces the count.
inline void skinny_plan_one_round(int64_t k, int64_t n, int waves, int hint_parts, int *rows_per_block, int *splits, int *tiles) {
    const int granule = 32 * waves;
    const int64_t t = cdiv(n, kSkinnyTileN);
    int64_t want = hint_parts;
    if (want <= 0) want = std::min<int64_t>(std::max<int64_t>(1, 256 / t), std::max<int64_t>(1, k / (2 * granule)));
    want = std::max<int64_t>(1, std::min<int64_t>(want, cdiv(k, granule)));
    const int64_t rpb = cdiv(cdiv(k, want), granule) * granule;
    *rows_per_block = int(rpb);
    *splits = int(cdiv(k, rpb));
    *tiles = int(t);
}

// Bytes of mailbox a skinny launch with `splits` K slices touches: one fp32 partial tile per (column tile, K slice but
// the last) of `rows` (at most 16) activation rows; the slot of the last slice is never written. One slice exchanges nothing.
inline int64_t skinny_mailbox_need(int tiles, int splits, int rows) {
    return splits > 1 ? int64_t(tiles) * splits * rows * kSkinnyTileN * 4 : 0;
}

// Makes the plan fit the mailbox: fewer, longer K slices (down to one, which needs none) when the partial tiles would
// not fit. `strict` callers get an error instead, naming the bytes the plan needs.
inline void skinny_fit_mailbox(int64_t k, int granule, int tiles, int rows, int64_t mailbox_bytes, bool strict,
                               int *rows_per_block, int *splits) {
    const int64_t need = skinny_mailbox_need(tiles, *splits, rows);
    if (need <= mailbox_bytes) return;
    if (strict) QMM_FAIL("scratch too small for this shape: the K split needs " << need << " bytes, " << mailbox_bytes << " are there");
    const int64_t per_split = int64_t(tiles) * rows * kSkinnyTileN * 4;
    int64_t fit = std::max<int64_t>(1, std::min<int64_t>(mailbox_bytes / per_split, *splits));
    const int64_t rpb = cdiv(cdiv(k, fit), granule) * granule;
    *rows_per_block = int(rpb);
    *splits = int(cdiv(k, rpb));
}

}  // namespace qmm
