// Shared parts of the bandwidth-bound skinny kernels (M <= 16 rows per pass, 256-column tiles, the waves of a
// workgroup split its run of 32-row steps): the launch plan, the LDS reduction over the waves and the exchange of
// partial tiles between workgroups.
#pragma once
#include <type_traits>

#include "common.h"

namespace qmm {

constexpr int kSkinnyTileN = 256;
// LDS reduction tile: one row of 256 floats per (slot, activation row), 1040 bytes apart, as 64 chunks of 16 bytes. The
// chunk of columns 4c .. 4c+3 sits at position skinny_red_chunk(c). A lane (g, cl) of the main loop writes the four
// chunks 4cl .. 4cl+3 of rows 4g .. 4g+3 with 16-byte stores: the row pitch puts the four g of an instruction into
// different quarters of the 64 banks (4 rows = 16 x 256 + 64 bytes) and the permutation spreads the four lanes that
// share a quarter over its four 16-byte slots, so an instruction takes the four passes its 1 KiB needs and no more.
// Readers fetch whole chunks (or single floats of them) of consecutive columns: every bank once per 256 bytes.
constexpr int kSkinnyRedStride = 260;  // floats
__device__ __forceinline__ int skinny_red_chunk(int c) { return (c & ~3) | ((c ^ (c >> 4)) & 3); }

inline size_t skinny_lds_bytes(int m, int waves) { return size_t(waves) * m * kSkinnyRedStride * sizeof(float); }

// Output type of a bfloat16 kernel that adds a bias vector (bfloat16 bits) in its epilogue; plain bfloat16 bits are uint16_t.
struct bf16_biased_t {
    uint16_t bits;
};
// Output type of a float16 kernel whose caller gave no bias: the column factor only, one rounding (_Float16 itself stands for
// the epilogue with both).
struct f16_unbiased_t {
    _Float16 v;
};

template <typename OutT>
__device__ __forceinline__ OutT skinny_to_out(float v);
template <>
__device__ __forceinline__ _Float16 skinny_to_out<_Float16>(float v) { return _Float16(v); }
template <>
__device__ __forceinline__ uint16_t skinny_to_out<uint16_t>(float v) { return f32_to_bf16_bits(v); }  // bfloat16 bits

// Division by a number the host knows: magic = floor(2^32 / d) (2^32 - 1 for d = 1) gives the quotient or one less for
// every n below 2^31; one comparison decides. A handful of scalar instructions where a division takes thirty: these
// sit between a workgroup's start and its first load, and between its last load and its output.
__host__ __device__ __forceinline__ uint32_t skinny_magic(uint32_t d) { return d <= 1 ? 0xFFFFFFFFu : uint32_t((uint64_t(1) << 32) / d); }
__host__ __device__ __forceinline__ int skinny_div(int n, int d, uint32_t magic) {
    uint32_t q = uint32_t((uint64_t(uint32_t(n)) * magic) >> 32);
    if ((q + 1) * uint32_t(d) <= uint32_t(n)) ++q;
    return int(q);
}

// The launch plan. The work of a launch is a flat sequence of units, unit tile * ksteps + step being the 32-row step
// `step` of the 256-column tile `tile`; the workgroups take consecutive runs of units/groups units (the first
// units % groups of them one more) and deal them to their waves the same way. Every workgroup therefore streams the
// same number of bytes (to within one step) whatever the shape, and a launch of 256 workgroups puts one on every CU
// (4096 x 11008: 43 tiles x 128 steps = 5504 units, 21 or 22 per workgroup; column tiles x whole K slices would leave
// 84 of the 256 CUs without work, and the kernel's time follows the number of CUs that read, not the bytes: loads alone
// take 9.8 us from 172 CUs, 7.9 from 256). groups >= tiles, so a run touches at most two tiles: a workgroup contributes
// a partial tile to its first tile and, when its run crosses into the next one, a second partial tile there.
struct SkinnyPlanHead {  // what a workgroup needs before its first load: passed as the kernels' leading arguments, which
                         // reach a wave in registers instead of through a fetch
    int ksteps = 0;      // 32-row steps per tile: cdiv(K, 32)
    uint32_t ksteps_magic = 0;
    int per_group = 0;   // units / groups: the first `longer` workgroups run one unit more than that
    int longer = 0;      // units % groups
    int splits = 0;      // > 0: groups = tiles * splits, and the launch deals the tiles to the XCDs (skinny_group_of_block)
    uint32_t splits_magic = 0;
};
struct SkinnyPlanRest {
    int tiles = 0;       // 256-column tiles: cdiv(N, 256)
    int groups = 0;      // workgroups of the launch, tiles <= groups <= tiles * ksteps
    int max_others = 0;  // the most partial tiles any tile's last workgroup has to fetch (0: nothing is exchanged)
    uint32_t per_group_magic = 0, per_group1_magic = 0;  // for divisions by per_group and per_group + 1
    int spin_limit = 0;  // re-reads of the mailbox after which a collector gives up
};
struct SkinnyPlan : SkinnyPlanHead, SkinnyPlanRest {
    __host__ __device__ SkinnyPlan() {}
    __host__ __device__ SkinnyPlan(const SkinnyPlanHead &h, const SkinnyPlanRest &r) : SkinnyPlanHead(h), SkinnyPlanRest(r) {}
};

__host__ __device__ __forceinline__ int skinny_units(const SkinnyPlan &p) { return p.tiles * p.ksteps; }

// Which run a workgroup of the launch takes. Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.
// With few activation rows the order does not matter (one row at 4096 x 11008: 10.5 us either way) and workgroup b takes
// run b. With many rows the partial tiles are large (16 KiB each at 16 rows) and it pays to have a tile's contributors
// on one XCD, where the collector's reads find the senders' stores in that XCD's L2 (16 rows at 4096 x 4096: 10.7 against
// 12.0 us): the plan then has `splits` runs per tile, tile t belongs to XCD t % 8, and the launch is padded to a multiple
// of 8 tiles (false: a workgroup of the padding, nothing to do).
__host__ __device__ __forceinline__ bool skinny_group_of_block(const SkinnyPlanHead &p, int tiles, int block, int *g) {
    *g = block;
    if (p.splits == 0) return true;
    const int rest = block >> 3, octet = skinny_div(rest, p.splits, p.splits_magic), tile = octet * 8 + (block & 7);
    *g = tile * p.splits + (rest - octet * p.splits);
    return tile < tiles;
}
__host__ __device__ __forceinline__ int skinny_grid(const SkinnyPlan &p) {
    return p.splits == 0 ? p.groups : (p.tiles + 7) / 8 * 8 * p.splits;
}
// first unit of run g (g == groups: one past the last unit). With whole runs per tile (splits > 0) the tile's steps are
// dealt to its `splits` runs - per_group and longer then count within a tile - and no run crosses a tile boundary.
__host__ __device__ __forceinline__ int skinny_first_unit(const SkinnyPlanHead &p, int g) {
    if (p.splits == 0) return g * p.per_group + (g < p.longer ? g : p.longer);
    const int tile = skinny_div(g, p.splits, p.splits_magic), slice = g - tile * p.splits;
    return tile * p.ksteps + slice * p.per_group + (slice < p.longer ? slice : p.longer);
}
// the run that holds unit u
__host__ __device__ __forceinline__ int skinny_group_of_unit(const SkinnyPlan &p, int u) {
    int base = 0;
    if (p.splits > 0) {
        const int tile = skinny_div(u, p.ksteps, p.ksteps_magic);
        u -= tile * p.ksteps;
        base = tile * p.splits;
    }
    const int split = p.longer * (p.per_group + 1);  // the units of the longer runs come first
    return base + (u < split ? skinny_div(u, p.per_group + 1, p.per_group1_magic) : p.longer + skinny_div(u - split, p.per_group, p.per_group_magic));
}

// The run of one workgroup.
struct SkinnyWork {
    int tile;    // the tile of the run's first unit
    int u0, u1;  // the run
    int bound;   // first unit of tile + 1: units from here on belong to the second tile
    // The workgroup holding a tile's last unit collects that tile: it is the highest-numbered contributor, so every
    // workgroup it waits for was dispatched before it. It fetches the partial tiles of the tile's other contributors,
    // workgroups first .. g - 1, from mailbox slots first .. g - 1 (slot = sender's index: a workgroup sends at most
    // once - its part of `tile` when the run ends inside that tile, its part of tile + 1 when the run crosses the
    // boundary, and then it collects `tile`).
    __host__ __device__ bool collects(void) const { return u1 >= bound; }
    __host__ __device__ bool crosses(void) const { return u1 > bound; }
};
__host__ __device__ __forceinline__ SkinnyWork skinny_work_of(const SkinnyPlanHead &p, int g) {
    SkinnyWork w;
    w.u0 = skinny_first_unit(p, g);
    w.u1 = skinny_first_unit(p, g + 1);
    w.tile = skinny_div(w.u0, p.ksteps, p.ksteps_magic);
    w.bound = (w.tile + 1) * p.ksteps;
    return w;
}
// How a workgroup deals its run to its `waves` (at most 8) waves: evenly, and when the run crosses from one tile into the
// next, so that no wave does: the first `c` waves share the units before the boundary, the others those behind it, c
// in proportion to the two lengths (each side gets at least one wave): of the two whole numbers around
// waves * len0 / len the one that leaves the busiest wave fewer units. A wave then sums for one tile only, one pass over
// its accumulators, and leaves one partial result in LDS slot `wave`.
__host__ __device__ __forceinline__ int skinny_waves_before_bound(const SkinnyWork &w, int waves) {
    // (straight-line on purpose: every workgroup evaluates this before its first load)
    const int len = w.u1 - w.u0, len0 = (w.u1 < w.bound ? w.u1 : w.bound) - w.u0, len1 = len - len0;
    int c = 0;  // floor(waves * len0 / len) without a division
#pragma unroll
    for (int wv = 1; wv < waves; ++wv) c += (wv * len <= waves * len0) ? 1 : 0;
    // c waves: those before the boundary are the busier ones (len0 / c units each); c + 1 waves: those behind it are
    // (len1 / (waves - c - 1) each)
    const bool one_more = (c < 1) | ((c + 1 < waves) & (len1 * c < len0 * (waves - c - 1)));
    c += one_more ? 1 : 0;
    return len1 > 0 ? c : waves;
}
// floor(2^32 / p) for p = 2 .. 8, 2^32 - 1 for p = 1: skinny_div by a small count that only the workgroup knows
__host__ __device__ __forceinline__ uint32_t skinny_small_magic(int p) {
    // a tree of selects on the bits of p - 1 (a chain of comparisons would be compiled into a jump table's worth of branches)
    const uint32_t i = uint32_t(p - 1);
    const bool b0 = i & 1u, b1 = i & 2u, b2 = i & 4u;
    const uint32_t m12 = b0 ? 0x80000000u : 0xFFFFFFFFu, m34 = b0 ? 0x40000000u : 0x55555555u;
    const uint32_t m56 = b0 ? 0x2AAAAAAAu : 0x33333333u, m78 = b0 ? 0x20000000u : 0x24924924u;
    const uint32_t m1234 = b1 ? m34 : m12, m5678 = b1 ? m78 : m56;
    return b2 ? m5678 : m1234;
}
// the run of wave `wave` (lo == hi: nothing to do) and which of the workgroup's two tiles it lies in (0 or 1)
__host__ __device__ __forceinline__ void skinny_wave_run(const SkinnyWork &w, int wave, int waves, int *lo, int *hi, int *part) {
    const int c = skinny_waves_before_bound(w, waves);
    const bool behind = wave >= c;
    const int base = behind ? w.bound : w.u0, end = behind ? w.u1 : (w.u1 < w.bound ? w.u1 : w.bound);
    const int sharers = behind ? waves - c : c, idx = behind ? wave - c : wave;
    const int span = end - base;  // at most ksteps, below 2^26
    const uint32_t magic = skinny_small_magic(sharers);
    *lo = base + skinny_div(idx * span, sharers, magic);
    *hi = base + skinny_div((idx + 1) * span, sharers, magic);
    *part = behind ? 1 : 0;
}

// What a workgroup does behind its main loop: which LDS slots hold which tile's parts and its part in the exchange.
struct SkinnyRoles {
    int c0 = 0;            // the first tile's parts are LDS slots [0, c0), the second tile's [c0, waves)
    int finish = 0;        // this workgroup holds the first tile's last unit and writes its output
    int fetch_first = 0;   // ... after adding the partial tiles of mailbox slots fetch_first .. fetch_first + fetch_others - 1
    int fetch_others = 0;
    int send_slot = -1;    // >= 0: the partial tile of LDS slots [send_lo, send_hi) goes to this mailbox slot
    int send_lo = 0, send_hi = 0;
    int send_tile = 0;     // the tile that partial tile belongs to
};
__host__ __device__ __forceinline__ SkinnyRoles skinny_roles_of(const SkinnyPlan &p, const SkinnyWork &wk, int g, int waves) {
    SkinnyRoles r;
    r.c0 = skinny_waves_before_bound(wk, waves);
    r.finish = wk.collects();
    r.send_tile = wk.tile;
    if (wk.crosses()) {  // first of the next tile
        r.send_slot = g;
        r.send_lo = r.c0;
        r.send_hi = waves;
        r.send_tile = wk.tile + 1;
    } else if (!wk.collects()) {
        r.send_slot = g;
        r.send_lo = 0;
        r.send_hi = waves;
    }
    if (r.finish) {
        r.fetch_first = skinny_group_of_unit(p, wk.tile * p.ksteps);
        r.fetch_others = g - r.fetch_first;
    }
    return r;
}

// The tail of a bandwidth-bound kernel: LDS reduction over the waves of a workgroup, then either the final store or
// the exchange through the mailbox.
//
// res[t][v] is a lane's partial sum for output row 4 * (lane / 16) + v and column tile * 256 + (lane % 16) * 16 + t;
// skinny_stash puts it into LDS slot `slot` = the wave's index of `red` (dynamic LDS of skinny_lds_bytes(m, WAVES)). col_scale names
// the column factors and biases of the output (SkinnyScale).
//
// Who does what in the tail: in the column layout thread tid owns column tid % 256 of rows tid / 256, tid / 256 + WAVES / 4,
// ... (one dword per access, four waves per row); in the quad layout it owns columns 4 (tid % 64) .. + 3 of rows tid / 64,
// tid / 64 + WAVES, ... (16 bytes per access, one wave per row). Either way every wave has work: the same bytes moved
// by a single wave were measured 1 us slower per launch. The column layout is the faster one per byte (8 rows at
// 4096 x 11008: 12.9 against 13.3 us) and is used while a thread has few rows (skinny_column_layout).
//
// Exchange: the mailbox holds one fp32 tile [m][256] per workgroup and is all zero between launches. A workgroup that
// is not the last of a tile stores its partial tile into its own slot (agent scope, +0.0 sent as -0.0, so a stored word
// is never zero) and is done: no acknowledgement, no counter. The workgroup that holds a tile's LAST unit - the highest
// workgroup index among the tile's contributors, so all the others were dispatched before it - reads their slots until
// no word is zero, adds them in workgroup order (its own last: the result does not depend on timing), writes the output
// and puts the zeros back with plain stores, which the end of the kernel makes visible to the next launch. The wait is
// bounded: after SkinnyPlan::spin_limit re-reads the output is NaN instead of a hang, the slots are cleared all the
// same and a word of the workspace's counter block records the loss (kExchangeLostWord) for the host to find.

// Which of the tail's two thread layouts a launch uses: one column per thread (dwords, `waves / 4` rows at a time) while a
// thread's reads of the exchange are few - rows per thread x partial tiles to fetch within 4 x 4, 2 x 8 or 1 x 16 - and
// whenever nothing is exchanged and there are few rows; else four columns per thread. `others` is the launch's
// largest count of partial tiles a collector fetches (SkinnyPlan::max_others).
__host__ __device__ __forceinline__ bool skinny_column_layout(int m, int others, int waves) {
    const int row_groups = waves / 4, rows = (m + row_groups - 1) / row_groups;
    if (others == 0) return m <= 4;
    return (rows <= 4 && others <= 4) || (rows <= 2 && others <= 8) || (rows <= 1 && others <= 16);
}

// Column factors of the output, c = sum * scale[n] + bias[n]: vectors of n elements of the output's 16-bit type (declared
// float16 here; the bfloat16 kernels pass bfloat16 bits through the same pointers), either may be null (scale 1, bias 0). The tail fetches them while its reads of the mailbox are under way, not earlier: a load issued between the
// weight loads would have to come back before the weights issued after it.
struct SkinnyScale {
    const _Float16 *scale = nullptr, *bias = nullptr;
};

// CW columns per thread: the word a thread moves is one dword or four. Agent scope (sc1): loads bypass the L1, stores
// write through. The scalar part of an address (slot and row) rides in the instruction's scalar offset.
constexpr int kSkinnyAgentScope = 1 << 4;  // cache policy bits of a buffer access: sc1
template <int CW>
struct SkinnyWord;
template <>
struct SkinnyWord<1> {
    typedef uint32_t type;
    static __device__ __forceinline__ uint32_t least(type v) { return v; }
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int voff, int soff) { return __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, kSkinnyAgentScope); }
    static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, int voff, int soff, type v) { __builtin_amdgcn_raw_buffer_store_b32(v, r, voff, soff, kSkinnyAgentScope); }
    static __device__ __forceinline__ void clear(__amdgpu_buffer_rsrc_t r, int voff, int soff) { __builtin_amdgcn_raw_buffer_store_b32(0u, r, voff, soff, 0); }
    static __device__ __forceinline__ type never_zero(type v) { return v == 0u ? 0x80000000u : v; }
    static __device__ __forceinline__ float get(type v, int) { return __uint_as_float(v); }
};
template <>
struct SkinnyWord<4> {
    typedef uint4v_t type;
    static __device__ __forceinline__ uint32_t least(type v) { return min(min(v[0], v[1]), min(v[2], v[3])); }
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int voff, int soff) { return __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, kSkinnyAgentScope); }
    static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, int voff, int soff, type v) { __builtin_amdgcn_raw_buffer_store_b128(v, r, voff, soff, kSkinnyAgentScope); }
    static __device__ __forceinline__ void clear(__amdgpu_buffer_rsrc_t r, int voff, int soff) { __builtin_amdgcn_raw_buffer_store_b128(type{0u, 0u, 0u, 0u}, r, voff, soff, 0); }
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
    SkinnyScale factors;
    float scale[CW], bias[CW];  // this thread's, once fetch_factors and use_factors have run
    uint32_t scale_bits[2], bias_bits[2];
    OutT *c;
    uint32_t *lost_flag;  // may be null
    int spin_limit;
    int voff;   // byte offset of this thread's columns in a mailbox row

    struct Vals {
        float v[CW];
    };
    // the sum of LDS slots [lo, hi) for this thread's columns of `row`
    __device__ __forceinline__ Vals own(int row, int lo, int hi) const {
        const float *src = red + row * kSkinnyRedStride + skinny_red_chunk(col_in_tile >> 2) * 4 + (col_in_tile & 3);  // CW columns never straddle a chunk
        Vals r;
#pragma unroll
        for (int e = 0; e < CW; ++e) r.v[e] = 0.f;
        // every slot is read, whatever it holds, and the ones of the other tile are dropped afterwards: conditions around
        // the reads would make each one wait for the one before
        if constexpr (CW == 4) {
            float4_t q[WAVES];
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) q[wv] = *reinterpret_cast<const float4_t *>(src + wv * m * kSkinnyRedStride);
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv)
#pragma unroll
                for (int e = 0; e < 4; ++e) r.v[e] += (wv >= lo && wv < hi) ? q[wv][e] : 0.f;
        } else {
            float q[WAVES];
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) q[wv] = src[wv * m * kSkinnyRedStride];
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) r.v[0] += (wv >= lo && wv < hi) ? q[wv] : 0.f;
        }
        return r;
    }
    // one output element: float16 outputs take the column factor and the bias (two roundings, see scaled_biased_f16);
    // bfloat16 outputs have neither (the int4 kernel folds its group scales in before) unless the kernel asks for the bias
    // with the output type bf16_biased_t: the same two roundings then. (A type of its own, so that the calls without a
    // bias keep the shorter epilogue: every instruction behind the last weight delays the kernel's end.)
    __device__ __forceinline__ OutT finish(float sum, int e) const {
        if constexpr (std::is_same<OutT, _Float16>::value) return scaled_biased_f16(sum, scale[e], bias[e]);
        else if constexpr (std::is_same<OutT, f16_unbiased_t>::value) return f16_unbiased_t{_Float16(sum * scale[e])};
        else if constexpr (std::is_same<OutT, bf16_biased_t>::value) return bf16_biased_t{biased_bf16_bits(sum, bias[e])};
        else return skinny_to_out<OutT>(sum);
    }
    __device__ __forceinline__ void store(int row, const Vals &x) const {
        OutT *dst = c + int64_t(row) * n + out_col;
        if constexpr (CW == 1) {
            dst[0] = finish(x.v[0], 0);
        } else {
            uint16_t h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = __builtin_bit_cast(uint16_t, finish(x.v[e], e));
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

    // Column factors of this thread's output columns: the loads (no branch depends on a pointer or on the column: columns
    // past n and a missing vector read as zero bits through the descriptors) and, later, their use.
    __device__ __forceinline__ void fetch_factors() {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(factors.scale), 0,
                                                                            factors.scale != nullptr ? n * 2 : 0, 0x00020000);
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(factors.bias), 0,
                                                                            factors.bias != nullptr ? n * 2 : 0, 0x00020000);
        const int off = int(out_col) * 2;
        constexpr bool kBias = !std::is_same<OutT, f16_unbiased_t>::value;
        if constexpr (CW == 1) {
            scale_bits[0] = __builtin_amdgcn_raw_buffer_load_b16(rs, off, 0, 0);
            if constexpr (kBias) bias_bits[0] = __builtin_amdgcn_raw_buffer_load_b16(rb, off, 0, 0);
        } else {  // 8-byte loads: vectors 8-byte aligned, n a multiple of 4
            const auto q = __builtin_amdgcn_raw_buffer_load_b64(rs, off, 0, 0);
            scale_bits[0] = q[0];
            scale_bits[1] = q[1];
            if constexpr (kBias) {
                const auto b = __builtin_amdgcn_raw_buffer_load_b64(rb, off, 0, 0);
                bias_bits[0] = b[0];
                bias_bits[1] = b[1];
            }
        }
    }
    __device__ __forceinline__ void use_factors() {
#pragma unroll
        for (int e = 0; e < CW; ++e) {
            // the vectors have the output's type: float16, or bfloat16 bits
            const uint16_t sb = uint16_t(scale_bits[e >> 1] >> (16 * (e & 1))), bb = uint16_t(bias_bits[e >> 1] >> (16 * (e & 1)));
            constexpr bool kHalf16 = std::is_same<OutT, _Float16>::value || std::is_same<OutT, f16_unbiased_t>::value;
            scale[e] = factors.scale != nullptr ? (kHalf16 ? f16_bits_to_f32(sb) : bf16_bits_to_f32(sb)) : 1.0f;
            bias[e] = factors.bias != nullptr ? (kHalf16 ? f16_bits_to_f32(bb) : bf16_bits_to_f32(bb)) : -0.0f;
        }
    }

    // One partial tile (LDS slots [lo, hi)) into mailbox slot `slot`: this thread's columns of rows row_begin,
    // row_begin + kRowGroups, ...
    __device__ __forceinline__ void send(float *mailbox, int slot, int lo, int hi, int row_begin) const {
        const __amdgpu_buffer_rsrc_t box = __builtin_amdgcn_make_buffer_rsrc(mailbox + int64_t(slot) * m * kSkinnyTileN, 0,
                                                                             m * kSkinnyTileN * 4, 0x00020000);
#pragma unroll 1
        for (int row = row_begin; row < m; row += kRowGroups) W::store(box, voff, row * (kSkinnyTileN * 4), pack(own(row, lo, hi)));
    }

    // Everything a workgroup does behind its LDS reduction, in the order that keeps the kernel's end short:
    //   1. a workgroup that holds a tile's last unit (`fetch_others` > 0 partial tiles of other workgroups to add, in
    //      mailbox slots fetch_first ..) issues its first reads of the mailbox;
    //   2. a workgroup with a partial tile to hand over (send_slot >= 0: LDS slots [send_lo, send_hi)) stores it;
    //   3. the collector adds up and writes the tile's output rows (`finish`: it writes them whether or not there is
    //      anything to fetch). Its own part is LDS slots [0, c0).
    // A trip of the collector is one output row of this thread and up to 8 or 16 mailbox slots, all reads issued
    // before the first is looked at; when a word is still zero the trip is simply made again. The code is kept small and
    // free of branches on purpose (a trip always issues all its reads, those past the last slot at an offset outside
    // the buffer): a workgroup runs it once, from cold instruction memory, one instruction after the other, and every
    // instruction between the last weight and the output delays the kernel's end.
    __device__ __forceinline__ void run(float *mailbox, const SkinnyRoles &roles, int send_slot) {
        if (!roles.finish || roles.fetch_others == 0) {
            if (roles.finish) fetch_factors();
            if (send_slot >= 0) send(mailbox, send_slot, roles.send_lo, roles.send_hi, row_first);
            if (roles.finish) {
                use_factors();
#pragma unroll 1
                for (int row = row_first; row < m; row += kRowGroups) store(row, own(row, 0, roles.c0));
            }
            return;
        }
        // a trip: one output row of this thread and up to 8 or 16 slots (two rows of 8 slots per trip were measured
        // slower than two trips: 16 rows at 4096 x 11008 16.3 against 14.2 us); with at most 4 slots to fetch - whole
        // slices per tile - a trip takes two or four of the thread's rows, which costs no more than one
        if (roles.fetch_others > 8) collect<1, 16>(mailbox, roles, send_slot);
        else if (roles.fetch_others <= 4 && m > 2 * kRowGroups) collect<4, 4>(mailbox, roles, send_slot);
        else if (roles.fetch_others <= 4 && m > kRowGroups) collect<2, 4>(mailbox, roles, send_slot);
        else collect<1, 8>(mailbox, roles, send_slot);
    }

    template <int ROWS, int SLOTS>
    __device__ __forceinline__ void collect(float *mailbox, const SkinnyRoles &roles, int send_slot) {
        const __amdgpu_buffer_rsrc_t box = __builtin_amdgcn_make_buffer_rsrc(mailbox + int64_t(roles.fetch_first) * m * kSkinnyTileN, 0,
                                                                             roles.fetch_others * m * kSkinnyTileN * 4, 0x00020000);
        const int slot_bytes = m * kSkinnyTileN * 4;
        int row = row_first, sp0 = 0, spin = 0;
        bool lost = false, factors_fetched = false, factors_known = false;
        // the sum runs over the senders in order and ends with this workgroup's own part: keep `total` for last
        Vals others_sum[ROWS], total[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
#pragma unroll
            for (int e = 0; e < CW; ++e) others_sum[r].v[e] = total[r].v[e] = 0.f;
#pragma unroll 1
        for (;;) {
            const int last = min(SLOTS - 1, roles.fetch_others - sp0 - 1);
            Word bits[ROWS][SLOTS];
            int soff[ROWS][SLOTS], vo[ROWS][SLOTS];
            bool valid[ROWS][SLOTS];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
#pragma unroll
                for (int u = 0; u < SLOTS; ++u) {
                    // past the last slot or the last row: an offset outside the buffer, which reads zeros without a trip to
                    // memory (the reads that do go there bypass the caches: each costs as much as a useful one)
                    valid[r][u] = u <= last && row + r * kRowGroups < m;
                    vo[r][u] = valid[r][u] ? voff : 0x7FFFFFF0;
                    soff[r][u] = (sp0 + min(u, last)) * slot_bytes + min(row + r * kRowGroups, m - 1) * (kSkinnyTileN * 4);
                    bits[r][u] = W::load(box, vo[r][u], soff[r][u]);
                }
            }
            if (!factors_fetched) {
                fetch_factors();
                factors_fetched = true;
            }
            if (send_slot >= 0) {  // goes out while the first reads are under way
                send(mailbox, send_slot, roles.send_lo, roles.send_hi, row_first);
                send_slot = -1;
            }
            if (sp0 == 0 && spin == 0) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) total[r] = own(min(row + r * kRowGroups, m - 1), 0, roles.c0);
            }
            uint32_t least = 0xFFFFFFFFu;
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
#pragma unroll
                for (int u = 0; u < SLOTS; ++u) least = min(least, valid[r][u] ? W::least(bits[r][u]) : 0xFFFFFFFFu);
            if (__builtin_amdgcn_ballot_w64(least == 0u) != 0) {  // something has not arrived
                if (spin >= spin_limit) {
                    lost = true;
                } else if (m <= 4) {
                    ++spin;
                    asm volatile("" ::: "memory");  // the mailbox changes under the loop
                    continue;  // few rows, few bytes: the whole wave simply makes the trip again
                } else {
                    // many rows: the partial tiles are large, their senders take a microsecond and more to store them, and
                    // a collector that read everything again on every round would load the memory side with as many bytes
                    // again each time (16 rows, 15 senders: 22 against 16 us). Only what is missing is read again.
#pragma unroll 1
                    for (;;) {
                        ++spin;
                        asm volatile("" ::: "memory");
                        bool missing = false;
#pragma unroll
                        for (int r = 0; r < ROWS; ++r)
#pragma unroll
                            for (int u = 0; u < SLOTS; ++u)
                                if (valid[r][u] && W::least(bits[r][u]) == 0u) {
                                    bits[r][u] = W::load(box, vo[r][u], soff[r][u]);
                                    missing = true;
                                }
                        if (__builtin_amdgcn_ballot_w64(missing) == 0) break;
                        if (spin >= spin_limit) {
                            lost = true;
                            break;
                        }
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
#pragma unroll
                for (int u = 0; u < SLOTS; ++u) {
#pragma unroll
                    for (int e = 0; e < CW; ++e) others_sum[r].v[e] += W::get(bits[r][u], e);  // zeros where nothing was read
                    W::clear(box, vo[r][u], soff[r][u]);
                }
            }
            spin = 0;
            sp0 += SLOTS;
            if (sp0 < roles.fetch_others) continue;
            if (lost && lost_flag != nullptr) *lost_flag = 1u;
            if (!factors_known) {
                use_factors();
                factors_known = true;
            }
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                Vals out;
#pragma unroll
                for (int e = 0; e < CW; ++e) {
                    out.v[e] = lost ? __builtin_nanf("") : others_sum[r].v[e] + total[r].v[e];
                    others_sum[r].v[e] = 0.f;
                }
                if (row + r * kRowGroups < m) store(row + r * kRowGroups, out);
            }
            lost = false;
            sp0 = 0;
            row += ROWS * kRowGroups;
            if (row >= m) break;
        }
    }
};

// A wave's partial sums for one tile into LDS slot `slot` (the layout the tail's readers expect, see kSkinnyRedStride).
__device__ __forceinline__ void skinny_stash(const float4_t (&res)[16], int m, int slot, float *red) {
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4, cl = lane & 15;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int row = 4 * g + v;
        if (row < m) {
            float *dst = red + (slot * m + row) * kSkinnyRedStride;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<float4_t *>(dst + skinny_red_chunk(4 * cl + j) * 4) =
                    float4_t{res[4 * j][v], res[4 * j + 1][v], res[4 * j + 2][v], res[4 * j + 3][v]};
        }
    }
}

template <typename OutT, int WAVES, int CW>
__device__ __forceinline__ void skinny_tails_as(const SkinnyPlan &plan, const SkinnyWork &wk, const SkinnyRoles &roles, int m, int n,
                                                const SkinnyScale &col_scale, OutT *__restrict__ c, float *__restrict__ mailbox,
                                                uint32_t *lost_flag, const float *red) {
    constexpr int kHalf = SkinnyTail<OutT, WAVES, CW>::kRowGroups / 2;
    const int tid = threadIdx.x;
    SkinnyTail<OutT, WAVES, CW> tail;
    tail.m = m;
    tail.n = n;
    tail.red = red;
    tail.c = c;
    tail.lost_flag = lost_flag;
    tail.spin_limit = plan.spin_limit;
    tail.factors = col_scale;
    tail.scale_bits[0] = tail.scale_bits[1] = tail.bias_bits[0] = tail.bias_bits[1] = 0u;
    if constexpr (CW == 1) {
        tail.row_first = __builtin_amdgcn_readfirstlane(tid >> 8);  // the same for a whole wave: row tests are scalar
        tail.col_in_tile = tid & 255;
    } else {
        tail.row_first = __builtin_amdgcn_readfirstlane(tid >> 6);
        tail.col_in_tile = (tid & 63) * 4;
    }
    // n is a multiple of 16 where CW is 4: a quad of columns is in or out as a whole
    tail.out_col = int64_t(wk.tile) * kSkinnyTileN + tail.col_in_tile;
    if (tail.out_col >= n) return;  // then the columns of the next tile lie past n as well
    bool send_ok = int64_t(roles.send_tile) * kSkinnyTileN + tail.col_in_tile < n;
    // With few rows half of the waves own no output row. They hand over the workgroup's partial tile (row r is sent by the
    // threads that would own row r + half), so that a collector's waves that read the mailbox have no store of their own
    // in flight: a wave's memory operations complete in the order issued, and a read behind a store waits for the
    // store's acknowledgement from the memory side.
    tail.voff = tail.col_in_tile * 4;
    if (m <= kHalf) {
        if (tail.row_first >= kHalf) {
            if (send_ok && roles.send_slot >= 0 && tail.row_first - kHalf < m) tail.send(mailbox, roles.send_slot, roles.send_lo, roles.send_hi, tail.row_first - kHalf);
            return;
        }
        send_ok = false;
    }
    if (tail.row_first >= m) return;
    tail.run(mailbox, roles, send_ok ? roles.send_slot : -1);
}

// Everything behind the main loops: call after every wave has stashed its parts (this function holds the barrier).
// `roles` is skinny_roles_of of this workgroup.
template <typename OutT, int WAVES>
__device__ __forceinline__ void skinny_tails(const SkinnyPlan &plan, const SkinnyWork &wk, const SkinnyRoles &roles, int m, int n,
                                             const SkinnyScale &col_scale, OutT *__restrict__ c, float *__restrict__ mailbox,
                                             uint32_t *lost_flag, const float *red) {
    __syncthreads();
    if (skinny_column_layout(m, plan.max_others, WAVES)) skinny_tails_as<OutT, WAVES, 1>(plan, wk, roles, m, n, col_scale, c, mailbox, lost_flag, red);
    else skinny_tails_as<OutT, WAVES, 4>(plan, wk, roles, m, n, col_scale, c, mailbox, lost_flag, red);
}

// ---- host side: the plan of a launch ------------------------------------------------------------------------------

constexpr int kSkinnyGroups = 256;           // most workgroups of a plan: one per CU of a full MI355X
constexpr int kSkinnyPlanWaves = 8;          // waves of a workgroup of the kernels that use the plan
constexpr int kSkinnyMinUnitsPerGroup = 2 * kSkinnyPlanWaves;  // two 32-row steps per wave
// The runs ignore the tile boundaries up to this many activation rows and while a tile has no more than this many
// contributors; beyond, whole runs per tile with a tile's runs on one XCD are faster (one row at 11008 x 4096, 16 tiles:
// 12.4 against 10.4 us; 16 rows at 4096 x 4096: 12.0 against 10.4 us; 4 and 8 rows at 4096 x 11008: 12.7 and 13.5 against
// 12.4 and 13.2 us). The int4 kernel always takes whole runs per tile: its matrix is half the bytes, and the exchange
// with five or six senders per tile cost it more than the idle CUs of four slices (one row: 10.0 against 9.6 us).
constexpr int kSkinnyFlatRows = 2, kSkinnyFlatSharers = 8;

// Bytes of mailbox a plan touches: one fp32 partial tile of `rows` (at most 16) activation rows per workgroup, slot =
// workgroup index. A plan of one workgroup per tile exchanges nothing.
inline int64_t skinny_mailbox_need(const SkinnyPlan &p, int rows) {
    return p.groups > p.tiles ? int64_t(p.groups) * rows * kSkinnyTileN * 4 : 0;
}

// The largest number of partial tiles any collector of the plan fetches.
inline int skinny_max_others(const SkinnyPlan &p) {
    int most = 0;
    if (p.groups == p.tiles) return 0;
    for (int t = 0; t < p.tiles; ++t)
        most = std::max(most, skinny_group_of_unit(p, (t + 1) * p.ksteps - 1) - skinny_group_of_unit(p, t * p.ksteps));
    return most;
}

// The plan of a launch over w[K, N] with `rows` (<= 16) activation rows per pass: 256 workgroups when every one of them
// still gets 16 units (two steps per wave), fewer on small matrices, one per tile on outputs wider than 256 tiles.
// `hint_parts` > 0 asks for that many workgroups per tile instead. The partial tiles must fit the mailbox: a plan that
// does not is cut down to fewer workgroups (one per tile needs no mailbox at all); `strict` callers get an error
// instead, naming the bytes the plan needs.
inline SkinnyPlan skinny_make_plan(int64_t k, int64_t n, int hint_parts, int rows, int64_t mailbox_bytes, bool strict, bool flat_ok = true,
                                   int cus = kSkinnyGroups) {
    SkinnyPlan p;
    const int64_t tiles = cdiv(n, kSkinnyTileN), ksteps = cdiv(k, 32), units = tiles * ksteps;
    QMM_CHECK(units < (int64_t(1) << 30), "K x N too large for one launch of the bandwidth-bound kernel: " << k << " x " << n);
    p.tiles = int(tiles);
    p.ksteps = int(ksteps);
    // one workgroup per CU of the device the launch goes to (fewer CUs than a full MI355X: a partition, a CU mask known to
    // the runtime), never more than 256: the mailbox bound of the callers is stated for that many
    const int64_t most = std::max(1, std::min(cus, kSkinnyGroups));
    // few rows: as many workgroups as there are CUs, whatever the number of tiles; many rows (or a number of parts asked
    // for): whole runs per tile, a tile's runs on one XCD
    int64_t splits = hint_parts > 0 ? std::min<int64_t>(hint_parts, ksteps) : 0;
    if (splits == 0 && (!flat_ok || rows > kSkinnyFlatRows || tiles * kSkinnyFlatSharers < most))
    {
        splits = std::max<int64_t>(1, std::min<int64_t>(most / tiles, units / kSkinnyMinUnitsPerGroup / tiles));
        // a launch takes as long as its busiest wave: no more slices than that wave's number of steps needs (4096 rows: 4
        // slices of 4 steps per wave, not 5 of 3 or 4)
        const auto wave_steps = [&](int64_t sl) { return cdiv(cdiv(ksteps, sl), kSkinnyPlanWaves); };
        while (splits > 1 && wave_steps(splits - 1) == wave_steps(splits)) --splits;
    }
    int64_t groups = splits > 0 ? tiles * splits : std::max<int64_t>(tiles, std::min<int64_t>(most, units / kSkinnyMinUnitsPerGroup));
    p.groups = int(groups);
    const int64_t slot_bytes = int64_t(rows) * kSkinnyTileN * 4;
    if (skinny_mailbox_need(p, rows) > mailbox_bytes) {
        if (strict)
            QMM_FAIL("scratch too small for this shape: the exchange of partial tiles needs " << skinny_mailbox_need(p, rows) << " bytes, "
                                                                                          << mailbox_bytes << " are there");
        p.groups = int(std::max<int64_t>(tiles, std::min<int64_t>(groups, mailbox_bytes / slot_bytes)));
        if (splits > 0) {
            splits = p.groups / tiles;
            p.groups = int(tiles * splits);
        }
    }
    p.splits = int(splits);
    p.splits_magic = skinny_magic(uint32_t(splits));
    p.per_group = int(splits > 0 ? ksteps / splits : units / p.groups);
    p.longer = int(splits > 0 ? ksteps % splits : units % p.groups);
    p.ksteps_magic = skinny_magic(uint32_t(p.ksteps));
    p.per_group_magic = skinny_magic(uint32_t(p.per_group));
    p.per_group1_magic = skinny_magic(uint32_t(p.per_group + 1));
    p.spin_limit = exchange_spin_limit().load(std::memory_order_relaxed);
    p.max_others = skinny_max_others(p);
    return p;
}

}  // namespace qmm
