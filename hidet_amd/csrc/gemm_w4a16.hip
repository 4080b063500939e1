// Group-wise W4A16 GEMM (M > 64): c[m, n] = sum_g scale[g, n] * sum_{k in g} a[m, k] * q[k, n] on
// bf16 / fp16 MFMA with fp32 accumulation.
//
// As in the int8 GEMM the packed weights go straight from global memory into registers: lane (kg, ns)
// loads one dword (8 columns) of rows 8kg .. 8kg+7 per 32-row k-step, a wave covers 128 columns.  Each
// nibble is dequantised exactly as the definition says: u = nibble ^ 8 = q + 8 is widened with
// v_cvt_f32_ubyte, one fma gives q * scale = u * scale - 8 * scale in fp32 and v_cvt_pk rounds two
// of them to the 16-bit type, which is bit for bit the dequantised weight `dtype(q) * scale`.  The eight
// values of one column over eight rows are the B operand of a 16x16x32 MFMA.  A wave owns RB*16 rows
// x 128 columns; the activation tile goes through swizzled, double-buffered LDS.
#include "common.h"

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

}  // namespace

bool gemm_w4a16_supported(const void *a, const void *w, const void *scales, const void *c, int64_t k, int64_t n,
                          int64_t lda, int group) {
    return (k % 8 == 0) && (lda % 8 == 0) && (n % 8 == 0) && (group % 32 == 0) && aligned(a, 16) && aligned(w, 4) &&
           aligned(scales, 16) && aligned(c, 16);
}

void gemm_w4a16_launch(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n,
                       int64_t lda, int group, int dtype, hipStream_t stream) {
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
