// Group-wise W4A16 GEMM (M > 32): c[m, n] = sum_g scale[g, n] * sum_{k in g} a[m, k] * q[k, n] on
// bf16 / fp16 MFMA with fp32 accumulation.
//
// In the register kernels the packed weights go straight from global memory into registers: lane (kg, ns)
// loads one dword (8 columns) of rows 8kg .. 8kg+7 per 32-row k-step, a wave covers 128 columns.  Each
// nibble is dequantised exactly as the definition says: u = nibble ^ 8 = q + 8 is widened with
// v_cvt_f32_ubyte, one fma gives q * scale = u * scale - 8 * scale in fp32 and v_cvt_pk rounds two
// of them to the 16-bit type, which is bit for bit the dequantised weight `dtype(q) * scale`.  The eight
// values of one column over eight rows are the B operand of a 16x16x32 MFMA.  A wave owns RB*16 rows
// x 128 columns.
//
// Three kernels.  gemm_w4a16_lds_kernel (K and group size multiples of 64, N a multiple of 32, tensors addressable
// with 31-bit offsets) widens each weight once per workgroup into an LDS tile and is described where it is defined.
// gemm_w4a16_kernel16 (same conditions without the one on N; used where 256-row tiles fit the matrix badly) is built
// like the int8 GEMM and widens in registers as described above: buffer loads without address arithmetic, the
// activation tile straight into a three-slot LDS ring (buffer_load ... lds) two stages ahead, the A fragments of a
// k-step read one k-step ahead by hand-placed ds_read_b128, the raw weight rows of a k-step refilled one stage ahead
// as soon as they are consumed, the group's scales fetched one stage before the group starts.  Both use 2D XCD
// regions and the deterministic K split for grids that leave CUs idle.  gemm_w4a16_kernel (register-staged,
// double-buffered LDS, every load predicated) takes the rest.
#include "common.h"
#include "gemm_tiling.h"

namespace qmm {
namespace {

constexpr int kBK = 64;

template <int DT>
struct W4G;
template <>
struct W4G<HIDET_QMM_BF16> {
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        const bf16x2_t v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};  // v_cvt_pk_bf16_f32: nearest even
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float4_t mfma(const uint4 &a, const uint4 &b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t b) { return bf16_bits_to_f32(b); }
    static __device__ __forceinline__ uint16_t from_f32(float f) { return f32_to_bf16_bits(f); }
};
template <>
struct W4G<HIDET_QMM_F16> {
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        const half2_t v = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float4_t mfma(const uint4 &a, const uint4 &b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t b) { return f16_bits_to_f32(b); }
    static __device__ __forceinline__ uint16_t from_f32(float f) { return f32_to_f16_bits(f); }
};

template <int RB, int WM, int WN>
struct GemmW4Cfg {
    static constexpr int kBM = WM * RB * 16;
    static constexpr int kBN = WN * 128;
    static constexpr int kThreads = WM * WN * 64;
    static constexpr int kAChunks = kBM * 8 / kThreads;
    static constexpr int kLdsBytes = 2 * kBM * 128;
};

template <int DT, int RB, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm_w4a16_kernel(const uint16_t *__restrict__ a, int64_t lda,
                                                                      const uint8_t *__restrict__ w,
                                                                      const uint16_t *__restrict__ scales,
                                                                      uint16_t *__restrict__ c, int m, int k, int n,
                                                                      int group, int tiles_m, int tiles_n) {
    using Cfg = GemmW4Cfg<RB, WM, WN>;
    using T = W4G<DT>;
    extern __shared__ uint4 lds[];

    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int cb_begin = (tiles_n * xcd) / 8, cb_end = (tiles_n * (xcd + 1)) / 8;
    if (local >= (cb_end - cb_begin) * tiles_m) return;
    const int cb = cb_begin + local / tiles_m;
    const int rbk = local % tiles_m;
    const int m0 = rbk * Cfg::kBM;
    const int n0 = cb * Cfg::kBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int kg = lane >> 4, ns = lane & 15;
    const int col = n0 + wn * 128 + ns * 8;  // first of this lane's 8 columns
    const bool col_ok = col < n;              // n % 8 == 0
    const int64_t row_bytes = n >> 1;

    float4_t acc[RB][8];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[rb][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int a_row = tid >> 3, a_chunk = tid & 7;
    const uint16_t *a_base = a + int64_t(m0 + a_row) * lda + a_chunk * 8;
    const uint8_t *w_base = w + (col >> 1);

    uint4 a_regs[Cfg::kAChunks];
    uint32_t w_raw[2][8];
    float sc[8], sc8[8];  // scale and -8 * scale of this lane's 8 columns for the current group
#pragma unroll
    for (int t = 0; t < 8; ++t) sc[t] = sc8[t] = 0.f;

    auto load_a = [&](int kbase) {
#pragma unroll
        for (int j = 0; j < Cfg::kAChunks; ++j) {
            const int row = m0 + a_row + j * (Cfg::kThreads / 8);
            a_regs[j] = uint4{0u, 0u, 0u, 0u};
            if (row < m && kbase + a_chunk * 8 < k)
                a_regs[j] = *reinterpret_cast<const uint4 *>(a_base + int64_t(j * (Cfg::kThreads / 8)) * lda + kbase);
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int j = 0; j < Cfg::kAChunks; ++j) {
            const int r = a_row + j * (Cfg::kThreads / 8);
            lds[buf * Cfg::kBM * 8 + r * 8 + (a_chunk ^ (r & 7))] = a_regs[j];
        }
    };
    auto load_w = [&](int kbase, int ks) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int row = kbase + ks * 32 + kg * 8 + j;
            w_raw[ks][j] = 0u;
            if (col_ok && row < k) w_raw[ks][j] = *reinterpret_cast<const uint32_t *>(w_base + int64_t(row) * row_bytes);
        }
    };

    load_a(0);
    load_w(0, 0);
    load_w(0, 1);
    store_a(0);
    __syncthreads();

    const int stages = (k + kBK - 1) / kBK;
    for (int s = 0; s < stages; ++s) {
        const int buf = s & 1;
        const bool more = s + 1 < stages;
        if (more) load_a((s + 1) * kBK);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int kpos = s * kBK + ks * 32;
            if (kpos < k) {
                if (kpos % group == 0 && col_ok) {
                    const uint4 sraw = *reinterpret_cast<const uint4 *>(scales + int64_t(kpos / group) * n + col);
                    const uint16_t *sv = reinterpret_cast<const uint16_t *>(&sraw);
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        sc[t] = T::to_f32(sv[t]);
                        sc8[t] = -8.0f * sc[t];
                    }
                }
                // nibble ^ 8 = q + 8; ev[j] keeps columns 0,2,4,6 of row j in its 4 bytes, od[j] columns 1,3,5,7
                uint32_t ev[8], od[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t r = w_raw[ks][j] ^ 0x88888888u;
                    ev[j] = r & 0x0F0F0F0Fu;
                    od[j] = (r >> 4) & 0x0F0F0F0Fu;
                }
                if (more) load_w((s + 1) * kBK, ks);
                uint4 afrag[RB];
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    const int r = (wm * RB + rb) * 16 + ns;
                    afrag[rb] = lds[buf * Cfg::kBM * 8 + r * 8 + ((ks * 4 + kg) ^ (r & 7))];
                }
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    uint4 b;
                    uint32_t *bp = reinterpret_cast<uint32_t *>(&b);
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const uint32_t lo = ((t & 1) ? od[2 * p] : ev[2 * p]) >> (8 * (t >> 1));
                        const uint32_t hi = ((t & 1) ? od[2 * p + 1] : ev[2 * p + 1]) >> (8 * (t >> 1));
                        const float flo = __builtin_fmaf(float(lo & 0xFFu), sc[t], sc8[t]);
                        const float fhi = __builtin_fmaf(float(hi & 0xFFu), sc[t], sc8[t]);
                        bp[p] = T::pack2(flo, fhi);
                    }
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) acc[rb][t] = T::mfma(afrag[rb], b, acc[rb][t]);
                }
            }
        }
        if (more) store_a(buf ^ 1);
        __syncthreads();
    }

    if (!col_ok) return;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = m0 + (wm * RB + rb) * 16 + kg * 4 + v;
            if (row < m) {
                uint4 o;
                uint32_t *op = reinterpret_cast<uint32_t *>(&o);
#pragma unroll
                for (int t = 0; t < 8; t += 2)
                    op[t >> 1] = uint32_t(T::from_f32(acc[rb][t][v])) | (uint32_t(T::from_f32(acc[rb][t + 1][v])) << 16);
                *reinterpret_cast<uint4 *>(c + int64_t(row) * n + col) = o;
            }
        }
}

template <int DT, int RB, int WM, int WN>
void launch_cfg(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n, int64_t lda,
                int group, hipStream_t stream) {
    using Cfg = GemmW4Cfg<RB, WM, WN>;
    const int tiles_m = int(cdiv(m, Cfg::kBM)), tiles_n = int(cdiv(n, Cfg::kBN));
    const int64_t grid = int64_t(8) * cdiv(tiles_n, 8) * tiles_m;
    QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
    launch(gemm_w4a16_kernel<DT, RB, WM, WN>, dim3(uint32_t(grid)), dim3(Cfg::kThreads), size_t(Cfg::kLdsBytes), stream,
           static_cast<const uint16_t *>(a), lda, static_cast<const uint8_t *>(w), static_cast<const uint16_t *>(scales),
           static_cast<uint16_t *>(c), int(m), int(k), int(n), group, tiles_m, tiles_n);
}


// ---- fast path -------------------------------------------------------------------------------------------------------

template <int RB, int WM, int WN>
struct GemmW4Cfg16 {
    static constexpr int kBM = WM * RB * 16;
    static constexpr int kBN = WN * 128;
    static constexpr int kThreads = WM * WN * 64;
    static constexpr int kAChunks = kBM * 8 / kThreads;
    static constexpr int kRingBytes = 3 * kBM * 128;
    static constexpr int kLdsBytes = kRingBytes + 16;  // + the fix-up's flag; the ring must start at LDS address 0
};

template <int DT, int RB, int WM, int WN, int MIN_BLOCKS>
__global__ __launch_bounds__(WM * WN * 64, MIN_BLOCKS) void gemm_w4a16_kernel16(
    const uint16_t *__restrict__ a, int64_t lda, const uint8_t *__restrict__ w, const uint16_t *__restrict__ scales,
    uint16_t *__restrict__ c, int m, int k, int n, int group, int tiles_m, int tiles_n, int xm, int xn, int concurrent,
    int tail_parts, int tail_stride, float *__restrict__ partials, uint32_t *__restrict__ counters) {
    using Cfg = GemmW4Cfg16<RB, WM, WN>;
    using T = W4G<DT>;
    extern __shared__ uint4 lds[];  // no static LDS in this kernel: fragment reads address the ring from 0
    int &s_last = *reinterpret_cast<int *>(lds + Cfg::kRingBytes / 16);

    GemmWorkItem item;
    if (!gemm_work_item(tiles_m, tiles_n, xm, xn, concurrent, tail_parts, tail_stride, &item)) return;
    const int m0 = item.tile_m * Cfg::kBM;
    const int n0 = item.tile_n * Cfg::kBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int kg = lane >> 4, ns = lane & 15;
    const int col = n0 + wn * 128 + ns * 8;  // first of this lane's 8 columns
    const bool col_ok = col < n;              // n % 8 == 0

    float4_t acc[RB][8];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[rb][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int row_bytes = n >> 1;
    const __amdgpu_buffer_rsrc_t rsrc_w =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(w), 0, int(int64_t(k) * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(scales), 0, int(int64_t(k / group) * n * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(a), 0, int((int64_t(m - 1) * lda + k) * 2), 0x00020000);

    // activation staging: instruction j of a wave fills the 64 consecutive 16-byte LDS slots
    // (j * kThreads + wave * 64 .. + 63); slot id holds chunk ((id % 8) ^ key(row)) of tile row id / 8
    constexpr int kOutside = 0x7FFFFFF0;  // rows / columns past the tensor read as zero
    int a_off[Cfg::kAChunks];
#pragma unroll
    for (int j = 0; j < Cfg::kAChunks; ++j) {
        const int id = j * Cfg::kThreads + tid;
        const int r = id >> 3;
        const int row = m0 + r;
        a_off[j] = row < m ? int((int64_t(row) * lda + ((id & 7) ^ lds_swizzle_key_step1(r)) * 8) * 2) : kOutside;
    }
    int w_off[8];  // row 8kg + j of a k-step, this lane's dword (8 columns)
#pragma unroll
    for (int j = 0; j < 8; ++j) w_off[j] = col_ok ? (kg * 8 + j) * row_bytes + (col >> 1) : kOutside;
    const int s_off = col_ok ? col * 2 : kOutside;

    const int stages = k / kBK;
    const int s_begin = (stages * item.part) / item.parts, s_end = (stages * (item.part + 1)) / item.parts;

    uint32_t w_raw[2][8];    // raw rows of the two k-steps of a stage; refilled one stage ahead once consumed
    float sc[8], sc8[8];     // scale (/ 16 for odd columns) and -8 * scale of this lane's 8 columns, current group
    uint4v_t sc_next;        // raw scales of the group that starts with the next stage

    auto load_a = [&](int st, int slot) {
#pragma unroll
        for (int j = 0; j < Cfg::kAChunks; ++j)
            buffer_load_to_lds_b128(rsrc_a, lds + slot * Cfg::kBM * 8 + j * Cfg::kThreads + wave * 64, a_off[j],
                                    (st < stages ? st : stages - 1) * (kBK * 2));  // the scalar offset is not range-checked
    };
    auto load_w = [&](int st, int q) {
        // the scalar offset is not part of the buffer's range check: never let it point past the tensor (a prefetch
        // for a stage past the end re-reads the last stage; its values are not used)
        const int soff = ((st < stages ? st : stages - 1) * kBK + q * 32) * row_bytes;
#pragma unroll
        for (int j = 0; j < 8; ++j) w_raw[q][j] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_w, w_off[j], soff, 0);
    };
    auto load_scales = [&](int st) {  // scales of the group stage st lies in (zero past the end)
        sc_next = __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, s_off, ((st * kBK) / group) * n * 2, 0);
    };
    auto take_scales = [&]() {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float sv = T::to_f32(uint16_t(sc_next[t >> 1] >> (16 * (t & 1))));
            sc8[t] = -8.0f * sv;
            sc[t] = (t & 1) ? sv * 0.0625f : sv;  // odd columns are widened as 16 * u
        }
    };

    // LDS byte address of this lane's A fragment for row block 0 of its wave, k-step 0 / 1, ring slot 0
    uint32_t af_addr[2];
    {
        const int r = wm * RB * 16 + ns;
#pragma unroll
        for (int q = 0; q < 2; ++q) af_addr[q] = uint32_t((r * 8 + ((q * 4 + kg) ^ lds_swizzle_key_step1(r))) * 16);
    }

    int4v_t af[2][RB];  // A fragments of the current and of the next k-step
    auto read_frags = [&](int4v_t (&dst)[RB], uint32_t addr) {
        static_assert(RB == 4 || RB == 8, "row blocks per wave");
        dst[0] = lds_read_b128_early<0 * 2048>(addr);
        dst[1] = lds_read_b128_early<1 * 2048>(addr);
        dst[2] = lds_read_b128_early<2 * 2048>(addr);
        dst[3] = lds_read_b128_early<3 * 2048>(addr);
        if constexpr (RB == 8) {
            dst[4] = lds_read_b128_early<4 * 2048>(addr);
            dst[5] = lds_read_b128_early<5 * 2048>(addr);
            dst[6] = lds_read_b128_early<6 * 2048>(addr);
            dst[7] = lds_read_b128_early<7 * 2048>(addr);
        }
    };
    auto wait_frags = [&](int4v_t (&f)[RB]) {  // the RB newest reads (the next k-step's) may stay in flight
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) lds_wait_keep_newer<RB>(f[rb]);
    };

    // One k-step: the A fragments in `cur` are in flight or landed; the reads of the next k-step's fragments go out
    // first, then for each of the 8 columns of this lane: dequantise its 8 weights, RB MFMAs. Rows 2p, 2p+1 of the raw
    // block are dead after column 7, so the refill for the next stage is issued then.
    auto kstep = [&](auto q_tag, int s, uint32_t next_addr) {
        constexpr int Q = decltype(q_tag)::value;
        int4v_t(&cur)[RB] = af[Q];
        int4v_t(&nxt)[RB] = af[Q ^ 1];
        // nibble ^ 8 = q + 8 = u. ev[j] keeps u of columns 0,2,4,6 of row j in its 4 bytes, od[j] keeps 16 * u of columns
        // 1,3,5,7 (their nibbles stay in the high half of each byte; sc[] of odd columns holds scale / 16, exact). One
        // v_cvt_f32_ubyteN then widens a weight without any shift. The empty asm keeps the compiler from re-deriving
        // each byte from the raw dword with a shift and a mask of its own.
        uint32_t ev[8], od[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t r = w_raw[Q][j] ^ 0x88888888u;
            ev[j] = r & 0x0F0F0F0Fu;
            od[j] = r & 0xF0F0F0F0u;
            asm volatile("" : "+v"(ev[j]), "+v"(od[j]));
        }
        load_w(s + 1, Q);
        read_frags(nxt, next_addr);  // after the last k-step this reads a slot nobody uses any more; dropped below
        __builtin_amdgcn_sched_barrier(0);
        wait_frags(cur);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            uint4 b;
            uint32_t *bp = reinterpret_cast<uint32_t *>(&b);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const uint32_t lo = ((t & 1) ? od[2 * p] : ev[2 * p]) >> (8 * (t >> 1));
                const uint32_t hi = ((t & 1) ? od[2 * p + 1] : ev[2 * p + 1]) >> (8 * (t >> 1));
                const float flo = __builtin_fmaf(float(lo & 0xFFu), sc[t], sc8[t]);
                const float fhi = __builtin_fmaf(float(hi & 0xFFu), sc[t], sc8[t]);
                bp[p] = T::pack2(flo, fhi);
            }
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
                acc[rb][t] = T::mfma(__builtin_bit_cast(uint4, cur[rb]), b, acc[rb][t]);
        }
    };

    load_a(s_begin, 0);
    load_a(s_begin + 1, 1);
    load_w(s_begin, 0);
    load_w(s_begin, 1);
    load_scales(s_begin);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    take_scales();
    __syncthreads();
    read_frags(af[0], af_addr[0]);

    // The loop body has no branches: the scales of the next stage's group are fetched and converted every stage
    // (one 16-byte load and 16 VALU ops per lane and stage) rather than at group boundaries only.
    for (int s = s_begin, slot = 0; s < s_end; ++s) {
        load_a(s + 2, slot >= 1 ? slot - 1 : 2);  // slot (s + 2) % 3: last read in stage s - 1
        load_scales(s + 1 < stages ? s + 1 : s);
        const uint32_t slot_off = uint32_t(slot * Cfg::kBM * 128);
        const int next_slot = slot == 2 ? 0 : slot + 1;
        kstep(std::integral_constant<int, 0>(), s, af_addr[1] + slot_off);
        // Every wave must hold the second k-step's fragments before the barrier (two barriers later their slot is
        // overwritten), and the activation loads of stage s + 1 (issued one stage ago) must have landed in LDS
        // before anyone reads them; what this stage issued so far (A chunks, scales, 8 weight rows) may stay in flight.
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) lds_wait_keep_newer<0>(af[1][rb]);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(Cfg::kAChunks + 1 + 8));
        __syncthreads();
        kstep(std::integral_constant<int, 1>(), s, af_addr[0] + uint32_t(next_slot * Cfg::kBM * 128));
        take_scales();
        slot = next_slot;
    }
    // drain: the fragment reads issued for the k-step past the end are not used, but their registers must not be reused
    // before they have landed, and LDS must not be released with activation loads in flight
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) lds_wait_keep_newer<0>(af[0][rb]);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __builtin_amdgcn_sched_barrier(0);

    if (item.parts > 1) {
        uint32_t rows_valid = 0;  // row blocks of this wave that reach into the matrix
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) rows_valid |= uint32_t(m0 + (wm * RB + rb) * 16 < m) << rb;
        if (!gemm_k_split_fixup<Cfg::kThreads>(acc, item, partials, counters, &s_last, rows_valid)) return;
    }

    if (!col_ok) return;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = m0 + (wm * RB + rb) * 16 + kg * 4 + v;
            if (row < m) {
                uint4 o;
                uint32_t *op = reinterpret_cast<uint32_t *>(&o);
#pragma unroll
                for (int t = 0; t < 8; t += 2)
                    op[t >> 1] = uint32_t(T::from_f32(acc[rb][t][v])) | (uint32_t(T::from_f32(acc[rb][t + 1][v])) << 16);
                *reinterpret_cast<uint4 *>(c + int64_t(row) * n + col) = o;
            }
        }
}

template <int DT, int RB, int WM, int WN, int MIN_BLOCKS>
void launch_cfg16(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n, int64_t lda,
                  int group, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    using Cfg = GemmW4Cfg16<RB, WM, WN>;
    const int tiles_m = int(cdiv(m, Cfg::kBM)), tiles_n = int(cdiv(n, Cfg::kBN));
    constexpr int kConcurrent = 32 * MIN_BLOCKS;
    const GemmTiling tiling = make_gemm_tiling(tiles_m, tiles_n, kConcurrent);
    GemmTail tail = make_gemm_tail(tiling, kConcurrent, kConcurrent, 4);
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    while (tail.parts > 1 &&
           (k / kBK < 8 * tail.parts || ws.scratch_bytes < int64_t(8) * tail.max_tiles * tail.parts * Cfg::kBM * Cfg::kBN * 4))
        --tail.parts;
    const int64_t grid = gemm_grid_with_tail(tiling, kConcurrent, tail);
    QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
    allow_dynamic_lds(reinterpret_cast<const void *>(gemm_w4a16_kernel16<DT, RB, WM, WN, MIN_BLOCKS>), Cfg::kLdsBytes);
    launch(gemm_w4a16_kernel16<DT, RB, WM, WN, MIN_BLOCKS>, dim3(uint32_t(grid)), dim3(Cfg::kThreads), size_t(Cfg::kLdsBytes),
           stream, static_cast<const uint16_t *>(a), lda, static_cast<const uint8_t *>(w), static_cast<const uint16_t *>(scales),
           static_cast<uint16_t *>(c), int(m), int(k), int(n), group, tiles_m, tiles_n, tiling.xm, tiling.xn, kConcurrent,
           tail.parts, tail.max_tiles, reinterpret_cast<float *>(ws.scratch), ws.counters);
}


// ---- dequantise once per workgroup --------------------------------------------------------------------------------------
//
// gemm_w4a16_kernel16 widens every weight once per wave and M tile; with M in the hundreds or thousands that is
// several times per weight and the VALU, not the MFMA, sets the pace. Here a workgroup of 8 waves owns 256 rows x 128
// columns and widens each weight of a 64-row stage ONCE: the packed rows (4 KiB) and the group's scales (256 B) come
// into an LDS ring by buffer_load ... lds three stages ahead; thread (byte b, 8-row chunk c) reads its 8 bytes (two
// columns x 8 rows), widens the 16 weights (v_bfe_i32, v_cvt_f32_i32, v_mul, v_cvt_pk) and writes two 16-byte chunks
// into a double-buffered tile laid out like the activation tile (one 128-byte row of 64 k per output column, chunks
// swizzled by row), from which every wave reads its B fragments. LDS row r of that tile holds output column
// (r / 64) * 64 + (r % 16) * 4 + (r / 16) % 4: the 16 lanes of a fragment read 16 consecutive LDS rows (no bank
// conflicts) and a lane's four MFMA column blocks are four consecutive output columns (8-byte stores).
//
// Every LDS access of the kernel is hand-placed asm: the compiler orders any LDS access of its own behind ALL
// outstanding buffer_load ... lds (it cannot tell which bytes they write), which would serialise the ring.

struct GemmW4LdsCfg {
    static constexpr int kBM = 256;
    static constexpr int kBN = 128;
    static constexpr int kThreads = 512;
    static constexpr int kAChunks = kBM * 8 / kThreads;
    static constexpr int kASlotBytes = kBM * 128;
    static constexpr int kBBufBytes = kBN * 128;
    static constexpr int kBBase = 3 * kASlotBytes;
    static constexpr int kRawBase = kBBase + 2 * kBBufBytes;
    static constexpr int kRawSlotBytes = 64 * 64 + 256;  // 64 rows x 64 bytes, then 128 scales
    static constexpr int kRingBytes = kRawBase + 3 * kRawSlotBytes;
    static constexpr int kLdsBytes = kRingBytes + 16;  // + the fix-up's flag; the ring must start at LDS address 0
    };

template <int OFFSET>
__device__ __forceinline__ uint32_t lds_read_u8_early(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_u8 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
__device__ __forceinline__ uint32_t lds_read_b32_early(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
__device__ __forceinline__ void lds_write_b128(uint32_t addr, const uint4v_t &v) {
    asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
// waits until at most NEWER LDS operations issued after the reads into these registers are outstanding
template <int NEWER>
__device__ __forceinline__ void lds_wait_keep_newer(uint32_t (&b)[8], uint32_t &s) {
    asm volatile("s_waitcnt lgkmcnt(%9)"
                 : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7]), "+v"(s)
                 : "n"(NEWER));
}
template <int NEWER>
__device__ __forceinline__ void lds_wait_keep_newer(int4v_t (&f)[4], int4v_t (&g)[4]) {
    asm volatile("s_waitcnt lgkmcnt(%8)"
                 : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(g[0]), "+v"(g[1]), "+v"(g[2]), "+v"(g[3])
                 : "n"(NEWER));
}

// Stages [s_begin, s_end) of output tile (tile_m, tile_n), by the whole workgroup. `split`: the tile is computed in
// pieces and fix(acc, rows_valid) exchanges them; it returns true in the workgroup that finishes the tile.
template <int DT, typename Fix>
__device__ __forceinline__ void gemm_w4a16_lds_tile(const uint16_t *__restrict__ a, int64_t lda, const uint8_t *__restrict__ w,
                                                    const uint16_t *__restrict__ scales, uint16_t *__restrict__ c, int m, int k, int n,
                                                    int group, int tile_m, int tile_n, int s_begin, int s_end, bool split, Fix fix) {
    using Cfg = GemmW4LdsCfg;
    using T = W4G<DT>;
    extern __shared__ uint4 lds[];  // no static LDS in this kernel: every access addresses the ring from 0

    const int m0 = tile_m * Cfg::kBM;
    const int n0 = tile_n * Cfg::kBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;  // 4 x 2 waves of 64 rows x 64 columns
    const int kg = lane >> 4, ns = lane & 15;

    float4_t acc[4][4];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[rb][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int row_bytes = n >> 1;
    const __amdgpu_buffer_rsrc_t rsrc_w =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(w), 0, int(int64_t(k) * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(scales), 0, int(int64_t(k / group) * n * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(a), 0, int((int64_t(m - 1) * lda + k) * 2), 0x00020000);

    constexpr int kOutside = 0x7FFFFFF0;  // rows / columns past the tensor read as zero
    int a_off[Cfg::kAChunks];
#pragma unroll
    for (int j = 0; j < Cfg::kAChunks; ++j) {
        const int id = j * Cfg::kThreads + tid;
        const int r = id >> 3;
        const int row = m0 + r;
        a_off[j] = row < m ? int((int64_t(row) * lda + ((id & 7) ^ lds_swizzle_key_step1(r)) * 8) * 2) : kOutside;
    }
    // packed rows: lanes 0..31 of wave v bring 16 bytes each: row 8v + lane / 4 of the stage, quarter lane % 4 of the
    // tile's 64 bytes. scales: lanes 0..7 bring one dword (two columns) each. (n % 32 == 0: whole quarters.)
    const int wq_col = (n0 >> 1) + (lane & 3) * 16;
    const int wq_off = wq_col < row_bytes ? (lane >> 2) * row_bytes + wq_col : kOutside;
    const int sq_col = n0 + 2 * (wave * 8 + lane);
    const int sq_off = sq_col < n ? sq_col * 2 : kOutside;

    const int stages = k / kBK;

    // A short matrix leaves most of a 256-row tile empty: a wave skips the activation loads whose 8 rows all lie past
    // the end (instruction j of wave v brings rows 64 j + 8 v .. + 7) and, if its 64 output rows do, its fragment reads
    // and MFMAs, so that the stage costs what the widening costs.
    int a_cnt = 0;
#pragma unroll
    for (int j = 0; j < Cfg::kAChunks; ++j) a_cnt += int(m0 + j * 64 + wave * 8 < m);
    const bool wave_active = m0 + wm * 64 < m;

    auto load_a = [&](int st, int slot, auto all_tag) {
        // the scalar offset is not part of the buffer's range check: never let it point past the tensor (a prefetch
        // for a stage past the end re-reads the last stage; its values are not used)
        const int stc = st < stages ? st : stages - 1;
#pragma unroll
        for (int j = 0; j < Cfg::kAChunks; ++j)
            if (decltype(all_tag)::value || j < a_cnt)
                buffer_load_to_lds_b128(rsrc_a, lds + slot * Cfg::kBM * 8 + j * Cfg::kThreads + wave * 64, a_off[j], stc * (kBK * 2));
    };
    auto wait_older_loads = [&](auto all_tag) {  // all but the loads of the last load_a + load_raw have landed
        if (decltype(all_tag)::value) {
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(Cfg::kAChunks + 2));
            return;
        }
        switch (a_cnt) {
            case 0: __builtin_amdgcn_s_waitcnt(waitcnt_vm(2)); break;
            case 1: __builtin_amdgcn_s_waitcnt(waitcnt_vm(3)); break;
            case 2: __builtin_amdgcn_s_waitcnt(waitcnt_vm(4)); break;
            case 3: __builtin_amdgcn_s_waitcnt(waitcnt_vm(5)); break;
            default: __builtin_amdgcn_s_waitcnt(waitcnt_vm(6)); break;
        }
    };
    auto load_raw = [&](int st, int slot) {
        const int stc = st < stages ? st : stages - 1;
        char *dst = reinterpret_cast<char *>(lds) + Cfg::kRawBase + slot * Cfg::kRawSlotBytes;
        if (lane < 32)
            buffer_load_to_lds_b128(rsrc_w, reinterpret_cast<uint4 *>(dst + wave * 512), wq_off, (stc * kBK + wave * 8) * row_bytes);
        if (lane < 8)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_s, (__attribute__((address_space(3))) void *)(dst + 4096 + wave * 32),
                                                     4, sq_off, ((stc * kBK) / group) * n * 2, 0, 0);
    };

    // Dequantisation: thread (lane, wave) widens bytes `lane` (columns 2 lane, 2 lane + 1) of rows 8 wave .. 8 wave + 7.
    // (the upper half of a wave takes the neighbouring k-group, wave ^ 1: a wave's two 16-byte writes of a stage then land on
    // all sixteen 16-byte bank groups, four lanes each, instead of eight lanes on eight of them)
    const int kgrp = wave ^ (lane >> 5);
    const uint32_t raw_rd = uint32_t(Cfg::kRawBase + kgrp * 512 + lane);
    const uint32_t sc_rd = uint32_t(Cfg::kRawBase + 4096 + lane * 4);
    uint32_t bw_addr[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const int sig = (lane >> 5) * 64 + (2 * (lane & 1) + e) * 16 + ((lane & 31) >> 1);
        bw_addr[e] = uint32_t(Cfg::kBBase + (sig * 8 + (kgrp ^ lds_swizzle_key_step1(sig))) * 16);
    }
    uint32_t bytes[8], sc2;
    auto read_raw = [&](int slot) {
        const uint32_t base = raw_rd + slot * Cfg::kRawSlotBytes;
        bytes[0] = lds_read_u8_early<0 * 64>(base);
        bytes[1] = lds_read_u8_early<1 * 64>(base);
        bytes[2] = lds_read_u8_early<2 * 64>(base);
        bytes[3] = lds_read_u8_early<3 * 64>(base);
        bytes[4] = lds_read_u8_early<4 * 64>(base);
        bytes[5] = lds_read_u8_early<5 * 64>(base);
        bytes[6] = lds_read_u8_early<6 * 64>(base);
        bytes[7] = lds_read_u8_early<7 * 64>(base);
        sc2 = lds_read_b32_early(sc_rd + slot * Cfg::kRawSlotBytes);
    };
    uint4v_t chunk[2];
    auto dequant = [&]() {  // q * scale is exact in fp32: one rounding, to the 16-bit type
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float sv = T::to_f32(uint16_t(sc2 >> (16 * e)));
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int q0 = int(bytes[2 * p] << (28 - 4 * e)) >> 28, q1 = int(bytes[2 * p + 1] << (28 - 4 * e)) >> 28;
                chunk[e][p] = T::pack2(float(q0) * sv, float(q1) * sv);
            }
        }
    };

    // LDS byte addresses of this lane's A fragment (row block 0, ring slot 0) and B fragment (column block 0, buffer 0)
    uint32_t af_addr[2], bf_addr[2];
    {
        const int ra = wm * 64 + ns, rb_ = wn * 64 + ns;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            af_addr[q] = uint32_t((ra * 8 + ((q * 4 + kg) ^ lds_swizzle_key_step1(ra))) * 16);
            bf_addr[q] = uint32_t(Cfg::kBBase + (rb_ * 8 + ((q * 4 + kg) ^ lds_swizzle_key_step1(rb_))) * 16);
        }
    }
    int4v_t af[2][4], bf[2][4];
    auto read_frags = [&](int4v_t (&dst)[4], uint32_t addr) {
        dst[0] = lds_read_b128_early<0 * 2048>(addr);
        dst[1] = lds_read_b128_early<1 * 2048>(addr);
        dst[2] = lds_read_b128_early<2 * 2048>(addr);
        dst[3] = lds_read_b128_early<3 * 2048>(addr);
    };
    auto mfmas = [&](int4v_t (&fa)[4], int4v_t (&fb)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int rb = 0; rb < 4; ++rb)
                acc[rb][t] = T::mfma(__builtin_bit_cast(uint4, fa[rb]), __builtin_bit_cast(uint4, fb[t]), acc[rb][t]);
    };

    // Schedule. One barrier per stage, in the middle: M(s). Stage s runs as
    //   H1(s): MFMAs of k-step 0 with the widening of stage s + 1 (bytes read during H2(s-1)) in their shadow, then
    //          the two tile writes into the other buffer
    //   M(s):  own LDS traffic done, own loads of H2(s-2) landed, barrier
    //   H2(s): reads of the bytes of stage s + 2 and of the k-step 0 fragments of stage s + 1; MFMAs of k-step 1 with
    //          the loads of activations s + 3 and packed rows s + 4 between them; then the reads of the k-step 1
    //          fragments of stage s + 1 into the registers just consumed
    // so every LDS read has half a stage to land and the only LDS traffic between the last MFMA of H1 and the barrier
    // is the two writes. Ring slot of stage x is (x - s_begin) % 3 for activations and packed rows, tile buffer
    // (x - s_begin) % 2.
    auto mfmas_half = [&](int4v_t (&fa)[4], int4v_t (&fb)[4], int t0) {
#pragma unroll
        for (int t = t0; t < t0 + 2; ++t)
#pragma unroll
            for (int rb = 0; rb < 4; ++rb)
                acc[rb][t] = T::mfma(__builtin_bit_cast(uint4, fa[rb]), __builtin_bit_cast(uint4, fb[t]), acc[rb][t]);
    };
    load_raw(s_begin, 0);
    load_a(s_begin, 0, std::false_type());
    load_raw(s_begin + 1, 1);
    load_a(s_begin + 1, 1, std::false_type());
    load_raw(s_begin + 2, 2);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __builtin_amdgcn_s_barrier();
    read_raw(0);
    lds_wait_keep_newer<0>(bytes, sc2);
    dequant();
    lds_write_b128(bw_addr[0], chunk[0]);
    lds_write_b128(bw_addr[1], chunk[1]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    load_a(s_begin + 2, 2, std::false_type());
    load_raw(s_begin + 3, 0);
    read_raw(1);
    auto active_loop = [&](auto all_tag) {
        read_frags(af[0], af_addr[0]);
        read_frags(bf[0], bf_addr[0]);
        read_frags(af[1], af_addr[1]);
        read_frags(bf[1], bf_addr[1]);
        for (int s = s_begin, slot = 0, buf = 0; s < s_end; ++s) {
            const int slot1 = slot == 2 ? 0 : slot + 1, slot2 = slot >= 1 ? slot - 1 : 2;
            const uint32_t a_next = uint32_t(slot1 * Cfg::kASlotBytes), b_other = uint32_t((buf ^ 1) * Cfg::kBBufBytes);
            // H1
            lds_wait_keep_newer<8>(bytes, sc2);
            lds_wait_keep_newer<8>(af[0], bf[0]);
            dequant();
            mfmas(af[0], bf[0]);
            // the two waves of a SIMD run in step: widening must sit in the shadow of this wave's own MFMAs, or the
            // MFMA pipe idles while both widen
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // four VALU
            }
            __builtin_amdgcn_sched_barrier(0);
            lds_write_b128(bw_addr[0] + b_other, chunk[0]);
            lds_write_b128(bw_addr[1] + b_other, chunk[1]);
            lds_wait_keep_newer<0>(af[1], bf[1]);
            wait_older_loads(all_tag);
            __builtin_amdgcn_s_barrier();
            // H2
            read_raw(slot2);
            read_frags(af[0], af_addr[0] + a_next);
            read_frags(bf[0], bf_addr[0] + b_other);
            __builtin_amdgcn_sched_barrier(0);
            mfmas_half(af[1], bf[1], 0);
            __builtin_amdgcn_sched_barrier(0);
            load_a(s + 3, slot, all_tag);
            load_raw(s + 4, slot1);
            __builtin_amdgcn_sched_barrier(0);
            mfmas_half(af[1], bf[1], 2);
            __builtin_amdgcn_sched_barrier(0);
            read_frags(af[1], af_addr[1] + a_next);
            read_frags(bf[1], bf_addr[1] + b_other);
            slot = slot1;
            buf ^= 1;
        }
        // drain: the reads issued for the stage past the end are not used, but their registers must not be reused
        // before they have landed
        lds_wait_keep_newer<0>(af[0], bf[0]);
        lds_wait_keep_newer<0>(af[1], bf[1]);
    };
    if (a_cnt == Cfg::kAChunks) {  // then the wave is active too
        active_loop(std::true_type());
    } else if (wave_active) {
        active_loop(std::false_type());
    } else {
        // same loads, widening, writes and barriers; no fragments, no MFMAs
        for (int s = s_begin, slot = 0, buf = 0; s < s_end; ++s) {
            const int slot1 = slot == 2 ? 0 : slot + 1, slot2 = slot >= 1 ? slot - 1 : 2;
            const uint32_t b_other = uint32_t((buf ^ 1) * Cfg::kBBufBytes);
            lds_wait_keep_newer<0>(bytes, sc2);
            dequant();
            lds_write_b128(bw_addr[0] + b_other, chunk[0]);
            lds_write_b128(bw_addr[1] + b_other, chunk[1]);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            wait_older_loads(std::false_type());
            __builtin_amdgcn_s_barrier();
            read_raw(slot2);
            load_a(s + 3, slot, std::false_type());
            load_raw(s + 4, slot1);
            slot = slot1;
            buf ^= 1;
        }
    }
    lds_wait_keep_newer<0>(bytes, sc2);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // LDS must not be released with loads in flight
    __builtin_amdgcn_sched_barrier(0);

    if (split) {
        uint32_t rows_valid = 0;  // row blocks of this wave that reach into the matrix
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) rows_valid |= uint32_t(m0 + wm * 64 + rb * 16 < m) << rb;
        if (!fix(acc, rows_valid)) return;
    }

    const int col = n0 + wn * 64 + ns * 4;  // first of this lane's 4 columns
    if (col >= n) return;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = m0 + wm * 64 + rb * 16 + kg * 4 + v;
            if (row < m) {
                uint2 o;
                o.x = uint32_t(T::from_f32(acc[rb][0][v])) | (uint32_t(T::from_f32(acc[rb][1][v])) << 16);
                o.y = uint32_t(T::from_f32(acc[rb][2][v])) | (uint32_t(T::from_f32(acc[rb][3][v])) << 16);
                *reinterpret_cast<uint2 *>(c + int64_t(row) * n + col) = o;
            }
        }
}

// STREAM false: one work item per workgroup (a tile, or one of `tail_parts` equal K ranges of a tail tile). STREAM true:
// the grid is `concurrent` workgroups per XCD and a workgroup computes its run of (tile, stage) units of the XCD's
// region (gemm_tiling.h: runs across the tiles), piece by piece; `tail_stride` is then the stride of the per-XCD blocks
// of tile counters, and `partials` holds two pieces per workgroup.
template <int DT, bool STREAM>
__global__ __launch_bounds__(512, 1) void gemm_w4a16_lds_kernel(
    const uint16_t *__restrict__ a, int64_t lda, const uint8_t *__restrict__ w, const uint16_t *__restrict__ scales,
    uint16_t *__restrict__ c, int m, int k, int n, int group, int tiles_m, int tiles_n, int xm, int xn, int concurrent,
    int tail_parts, int tail_stride, float *__restrict__ partials, uint32_t *__restrict__ counters) {
    using Cfg = GemmW4LdsCfg;
    extern __shared__ uint4 lds[];
    int *s_last = reinterpret_cast<int *>(lds + Cfg::kRingBytes / 16);
    const int stages = k / kBK;
    if constexpr (!STREAM) {
        GemmWorkItem item;
        if (!gemm_work_item(tiles_m, tiles_n, xm, xn, concurrent, tail_parts, tail_stride, &item)) return;
        gemm_w4a16_lds_tile<DT>(a, lda, w, scales, c, m, k, n, group, item.tile_m, item.tile_n, (stages * item.part) / item.parts,
                                (stages * (item.part + 1)) / item.parts, item.parts > 1, [&](auto &acc, uint32_t rows_valid) {
                                    return gemm_k_split_fixup<Cfg::kThreads>(acc, item, partials, counters, s_last, rows_valid);
                                });
    } else {
        constexpr int kTileFloats = Cfg::kBM * Cfg::kBN;
        const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;  // workgroup b runs on XCD b % 8
        const GemmRegion reg = gemm_region_of_xcd(tiles_m, tiles_n, xm, xn, xcd);
        const int units = reg.rows * reg.cols * stages;
        if (units == 0) return;
        const int hi = gemm_stream_bound(units, stages, concurrent, j + 1);
        for (int local = gemm_stream_bound(units, stages, concurrent, j) / stages; local * stages < hi; ++local) {
            const GemmStreamPiece piece = gemm_stream_piece(units, stages, concurrent, j, local);
            int tile_m, tile_n;
            gemm_tile_of_region(reg, local, &tile_m, &tile_n);
            gemm_w4a16_lds_tile<DT>(a, lda, w, scales, c, m, k, n, group, tile_m, tile_n, piece.s_begin, piece.s_end, piece.parts > 1,
                                    [&](auto &acc, uint32_t rows_valid) {
                                        const auto piece_at = [&](int p) {
                                            const int jp = piece.first + p;
                                            return partials + int64_t((jp * 8 + xcd) * 2 + gemm_stream_kind(units, stages, concurrent, jp, local)) * kTileFloats;
                                        };
                                        return gemm_stream_fixup<Cfg::kThreads>(acc, piece.parts, piece_at(piece.part), piece_at,
                                                                                counters + xcd * tail_stride + local, s_last, rows_valid);
                                    });
            __syncthreads();  // every wave is done with the rings before the next piece's loads write them
        }
    }
}

template <int DT>
void launch_lds(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n, int64_t lda,
                int group, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    using Cfg = GemmW4LdsCfg;
    const int tiles_m = int(cdiv(m, Cfg::kBM)), tiles_n = int(cdiv(n, Cfg::kBN));
    constexpr int kConcurrent = 32;
    const GemmTiling tiling = make_gemm_tiling(tiles_m, tiles_n, kConcurrent);
    // one part of one tile exchanged = 256 KiB through memory, about 0.05 us of the chip's bandwidth; a tile's compute
    // time is about 74 us at K = 4096 (measured: M = 512, all 172 tiles in 4 parts: 82 -> 104 us; M = 1024, 88 tail
    // tiles in 2 parts: 146 -> 121 us)
    GemmTail tail = make_gemm_tail_by_rounds(tiling, kConcurrent, 4, 0.0007 * 4096.0 / double(k));
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    while (tail.parts > 1 &&
           (k / kBK < 8 * tail.parts || ws.scratch_bytes < int64_t(8) * tail.max_tiles * tail.parts * Cfg::kBM * Cfg::kBN * 4))
        --tail.parts;
    const int64_t grid = gemm_grid_with_tail(tiling, kConcurrent, tail);
    QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
    // Runs across the tiles instead (gemm_tiling.h), one workgroup per CU, when the busiest XCD has a few tiles more than
    // a whole number of rounds: measured against the plan above at K = 4096, N = 11008, the run plan costs about a third
    // of a round whatever the size (a second prologue per workgroup and 128 KiB per piece through memory), so it wins
    // where the few tail tiles would cost half a round (M = 768, 33 tiles per XCD: 123 -> 105 us; M = 1536, 65: 194 ->
    // 187 us) and nowhere else (M = 512, 22 tiles on 32 CUs: 80 against 78 us with a third of the CUs idle; M = 1024: 129
    // against 127 us; M = 4096: 450 against 416 us, the workgroups of a region no longer walk K in step and share less
    // in the L2)
    const int stages = int(k / kBK);
    int fewest = tiling.region_tiles;
    for (int x = 0; x < 8; ++x) fewest = std::min(fewest, gemm_region_tiles(tiling, x));
    const int rest = tiling.region_tiles % kConcurrent;
    const bool stream_pays = tiling.region_tiles > kConcurrent && tiling.region_tiles < 3 * kConcurrent && rest >= 1 && rest <= kConcurrent / 8;
    const bool stream_ok = fewest > 0 && int64_t(fewest) * stages >= int64_t(kConcurrent) * kGemmStreamMinShare &&
                           int64_t(8) * tiling.region_tiles <= kExchangeLostWord &&
                           ws.scratch_bytes >= int64_t(8) * kConcurrent * 2 * Cfg::kBM * Cfg::kBN * 4;
    if (stream_ok && stream_pays) {
        allow_dynamic_lds(reinterpret_cast<const void *>(gemm_w4a16_lds_kernel<DT, true>), Cfg::kLdsBytes);
        launch(gemm_w4a16_lds_kernel<DT, true>, dim3(8 * kConcurrent), dim3(Cfg::kThreads), size_t(Cfg::kLdsBytes), stream,
               static_cast<const uint16_t *>(a), lda, static_cast<const uint8_t *>(w), static_cast<const uint16_t *>(scales),
               static_cast<uint16_t *>(c), int(m), int(k), int(n), group, tiles_m, tiles_n, tiling.xm, tiling.xn, kConcurrent, 1,
               tiling.region_tiles, reinterpret_cast<float *>(ws.scratch), ws.counters);
        return;
    }
    allow_dynamic_lds(reinterpret_cast<const void *>(gemm_w4a16_lds_kernel<DT, false>), Cfg::kLdsBytes);
    launch(gemm_w4a16_lds_kernel<DT, false>, dim3(uint32_t(grid)), dim3(Cfg::kThreads), size_t(Cfg::kLdsBytes), stream,
           static_cast<const uint16_t *>(a), lda, static_cast<const uint8_t *>(w), static_cast<const uint16_t *>(scales),
           static_cast<uint16_t *>(c), int(m), int(k), int(n), group, tiles_m, tiles_n, tiling.xm, tiling.xn, kConcurrent,
           tail.parts, tail.max_tiles, reinterpret_cast<float *>(ws.scratch), ws.counters);
}

}  // namespace

bool gemm_w4a16_supported(const void *a, const void *w, const void *scales, const void *c, int64_t k, int64_t n,
                          int64_t lda, int group) {
    return (k % 8 == 0) && (lda % 8 == 0) && (n % 8 == 0) && (group % 32 == 0) && aligned(a, 16) && aligned(w, 4) &&
           aligned(scales, 16) && aligned(c, 16);
}

void gemm_w4a16_launch(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n,
                       int64_t lda, int group, int dtype, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    const bool fast = (k % kBK == 0) && (group % kBK == 0) && k * (n / 2) < (int64_t(1) << 31) - (1 << 20) &&
                      (m * lda + k) * 2 < (int64_t(1) << 31) - (1 << 20) && (k / group) * n * 2 < (int64_t(1) << 31);
    // Measured on K = 4096, N = 11008, M = 33 .. 4096: the kernel that widens once per workgroup (256-row tiles) is
    // ahead except where its tall tiles leave a second or third tile row mostly empty (3 or 5 tile rows of 128).
    const int64_t rows128 = cdiv(m, 128);
    if (fast && n % 32 == 0 && rows128 != 3 && rows128 != 5) {
        if (dtype == HIDET_QMM_F16) launch_lds<HIDET_QMM_F16>(a, w, scales, c, m, k, n, lda, group, workspace, workspace_bytes, stream);
        else launch_lds<HIDET_QMM_BF16>(a, w, scales, c, m, k, n, lda, group, workspace, workspace_bytes, stream);
        return;
    }
    if (fast) {
        // workgroup tile 128 x 256: 4 waves of 64 x 128, two workgroups per CU
        if (dtype == HIDET_QMM_F16) launch_cfg16<HIDET_QMM_F16, 4, 2, 2, 2>(a, w, scales, c, m, k, n, lda, group, workspace, workspace_bytes, stream);
        else launch_cfg16<HIDET_QMM_BF16, 4, 2, 2, 2>(a, w, scales, c, m, k, n, lda, group, workspace, workspace_bytes, stream);
        return;
    }
    // 128 x 256 tiles (2 waves of 128 x 128) when they fill the chip, 64 x 256 tiles otherwise
    const bool big = cdiv(m, 128) * cdiv(n, 256) >= 512;
    if (dtype == HIDET_QMM_F16) {
        if (big) launch_cfg<HIDET_QMM_F16, 8, 1, 2>(a, w, scales, c, m, k, n, lda, group, stream);
        else launch_cfg<HIDET_QMM_F16, 4, 1, 2>(a, w, scales, c, m, k, n, lda, group, stream);
    } else {
        if (big) launch_cfg<HIDET_QMM_BF16, 8, 1, 2>(a, w, scales, c, m, k, n, lda, group, stream);
        else launch_cfg<HIDET_QMM_BF16, 4, 1, 2>(a, w, scales, c, m, k, n, lda, group, stream);
    }
}

}  // namespace qmm
