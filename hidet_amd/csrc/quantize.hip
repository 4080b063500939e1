// Quantization kernels: symmetric int8/int16 quantize + dequantize over a [outer, reduce, inner]
// view, group-wise signed int4 with nibble packing, and per-tensor float8 e4m3.
//
// Every division and rounding here is IEEE (no fast-math, no reciprocal approximation): the codes
// and scales must match the CPU definition bit for bit.
#include "common.h"
#include "numeric.h"

namespace qmm {
namespace {


__global__ void fill_u32_kernel(uint32_t *p, int64_t n, uint32_t v) {
    int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// amax over the middle axis of [outer, R, inner] when inner > 1 (strided reduction).
// grid (ceil(inner/64), outer, row_splits); 256 threads = 4 row lanes x 64 columns.
template <int DT>
__global__ __launch_bounds__(256) void amax_strided_kernel(const void *__restrict__ w, uint32_t *__restrict__ amax_bits,
                                                           int64_t R, int64_t inner, int64_t rows_per_split,
                                                           int use_atomic) {
    __shared__ float red[4][64];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t col = int64_t(blockIdx.x) * 64 + tx;
    const int64_t o = blockIdx.y;
    const int64_t r0 = int64_t(blockIdx.z) * rows_per_split;
    const int64_t r1 = min(R, r0 + rows_per_split);
    float m = 0.0f;
    if (col < inner) {
        const int64_t base = o * R * inner + col;
        int64_t r = r0 + ty;
        for (; r + 28 < r1; r += 32) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = load_as_f32<DT>(w, base + (r + 4 * i) * inner);
#pragma unroll
            for (int i = 0; i < 8; ++i) m = fmaxf(m, fabsf(v[i]));
        }
        for (; r < r1; r += 4) m = fmaxf(m, fabsf(load_as_f32<DT>(w, base + r * inner)));
    }
    red[ty][tx] = m;
    __syncthreads();
    if (ty == 0 && col < inner) {
        m = fmaxf(fmaxf(red[0][tx], red[1][tx]), fmaxf(red[2][tx], red[3][tx]));
        // |x| >= 0: the unsigned order of the bit patterns is the order of the values
        if (use_atomic) atomicMax(&amax_bits[o * inner + col], __float_as_uint(m));
        else amax_bits[o * inner + col] = __float_as_uint(m);
    }
}

// amax over the last axis of [outer, R] (inner == 1): one wave per row, 4 rows per block.
template <int DT>
__global__ __launch_bounds__(256) void amax_contig_kernel(const void *__restrict__ w, uint32_t *__restrict__ amax_bits,
                                                          int64_t outer, int64_t R) {
    const int lane = threadIdx.x & 63;
    const int64_t row = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= outer) return;
    float m = 0.0f;
    for (int64_t r = lane; r < R; r += 64) m = fmaxf(m, fabsf(load_as_f32<DT>(w, row * R + r)));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if (lane == 0) amax_bits[row] = __float_as_uint(m);
}

template <int QT>
__device__ __forceinline__ void store_code(void *q, int64_t i, float r) {
    if (QT == HIDET_QMM_I8) {
        static_cast<int8_t *>(q)[i] = static_cast<int8_t>(fminf(fmaxf(r, -128.0f), 127.0f));
    } else {
        static_cast<int16_t *>(q)[i] = static_cast<int16_t>(fminf(fmaxf(r, -32768.0f), 32767.0f));
    }
}

// Four-element forms (numel a multiple of 4, 16-byte aligned input, 4-byte aligned codes).
template <int DT>
__device__ __forceinline__ void load4_as_f32(const void *p, int64_t i4, float (&x)[4]) {
    if (DT == HIDET_QMM_F32) {
        const float4 v = *reinterpret_cast<const float4 *>(static_cast<const float *>(p) + i4 * 4);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    } else {
        const uint2 v = *reinterpret_cast<const uint2 *>(static_cast<const uint16_t *>(p) + i4 * 4);
        const uint16_t h[4] = {uint16_t(v.x), uint16_t(v.x >> 16), uint16_t(v.y), uint16_t(v.y >> 16)};
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = DT == HIDET_QMM_F16 ? f16_bits_to_f32(h[e]) : bf16_bits_to_f32(h[e]);
    }
}

// code = saturating_cast(round(rnd(w / scale))), scale = rnd(amax / qmax), rnd = round to w's dtype. `round` is what
// the reference's GPU lowering of round() does for the dtype: ties away from zero for float32 (roundf,
// python/hidet/ir/primitives/hip/math/float32.py:40), ties to even for float16 (hrint, hip/math/float16.py:42) and
// bfloat16 (hrint, cuda/math/bfloat16.py:29; the reference has no HIP bfloat16 math set). Its CPU half types round ties
// away instead (include/hidet/runtime/cpu/float16.h:747-750): a float16 quotient of exactly n + 0.5 - common, since
// float16 has a spacing of 1/16 between 64 and 128 - differs by one code between the two targets.
template <int DT>
__device__ __forceinline__ float round_code(float q) {
    return DT == HIDET_QMM_F32 ? roundf(q) : rintf(q);
}

template <int DT, int QT>
__global__ __launch_bounds__(256) void quantize_kernel(const void *__restrict__ w, const uint32_t *__restrict__ amax_bits,
                                                       void *__restrict__ q, void *__restrict__ scale, int64_t R,
                                                       int64_t inner, int64_t total) {
    const float qmax = QT == HIDET_QMM_I8 ? 127.0f : 32767.0f;
    int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int64_t o = i / (R * inner);
    const int64_t rem = i - o * R * inner;
    const int64_t r = rem / inner, c = rem - r * inner;
    const float amax = __uint_as_float(amax_bits[o * inner + c]);
    const float s = round_to<DT>(amax / qmax);
    if (r == 0) store_from_f32<DT>(scale, o * inner + c, s);
    float code = 0.0f;
    if (s != 0.0f) code = round_code<DT>(round_to<DT>(load_as_f32<DT>(w, i) / s));
    store_code<QT>(q, i, code);
}

// Same arithmetic, four consecutive elements of the innermost axis per thread (inner a multiple of 4, tensors aligned
// for the 4-element accesses): one index division per four elements, 16- or 8-byte loads, 4- or 8-byte code stores.
// ALONG_REDUCE (inner == 1, reduce a multiple of 4): the four elements lie along the reduced axis and share one scale;
// R is then reduce / 4 and inner4 is unused.
template <int DT, int QT, bool ALONG_REDUCE>
__global__ __launch_bounds__(256) void quantize4_kernel(const void *__restrict__ w, const uint32_t *__restrict__ amax_bits,
                                                        void *__restrict__ q, void *__restrict__ scale, int64_t R,
                                                        int64_t inner4, int64_t total4) {
    const float qmax = QT == HIDET_QMM_I8 ? 127.0f : 32767.0f;
    const int64_t i4 = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i4 >= total4) return;
    int64_t r, sidx;
    uint32_t abits[4];
    if (ALONG_REDUCE) {
        sidx = i4 / R;
        r = i4 - sidx * R;
        abits[0] = abits[1] = abits[2] = abits[3] = amax_bits[sidx];
    } else {
        const int64_t row = i4 / inner4;  // o * R + r
        const int64_t c4 = i4 - row * inner4;
        const int64_t o = row / R;
        r = row - o * R;
        sidx = (o * inner4 + c4) * 4;
        const uint4 ab = *reinterpret_cast<const uint4 *>(amax_bits + sidx);
        abits[0] = ab.x; abits[1] = ab.y; abits[2] = ab.z; abits[3] = ab.w;
    }
    float x[4];
    if (DT == HIDET_QMM_F32) {
        const float4 v = *reinterpret_cast<const float4 *>(static_cast<const float *>(w) + i4 * 4);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    } else {
        const uint2 v = *reinterpret_cast<const uint2 *>(static_cast<const uint16_t *>(w) + i4 * 4);
        const uint16_t h[4] = {uint16_t(v.x), uint16_t(v.x >> 16), uint16_t(v.y), uint16_t(v.y >> 16)};
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = DT == HIDET_QMM_F16 ? f16_bits_to_f32(h[e]) : bf16_bits_to_f32(h[e]);
    }
    float code[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float s = round_to<DT>(__uint_as_float(abits[e]) / qmax);
        if (r == 0 && (!ALONG_REDUCE || e == 0)) store_from_f32<DT>(scale, sidx + (ALONG_REDUCE ? 0 : e), s);
        code[e] = s != 0.0f ? round_code<DT>(round_to<DT>(x[e] / s)) : 0.0f;
    }
    if (QT == HIDET_QMM_I8) {
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) packed |= uint32_t(uint8_t(int8_t(fminf(fmaxf(code[e], -128.0f), 127.0f)))) << (8 * e);
        static_cast<uint32_t *>(q)[i4] = packed;
    } else {
        uint2 packed;
        uint32_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = uint32_t(uint16_t(int16_t(fminf(fmaxf(code[e], -32768.0f), 32767.0f))));
        packed.x = h[0] | (h[1] << 16);
        packed.y = h[2] | (h[3] << 16);
        static_cast<uint2 *>(q)[i4] = packed;
    }
}

// Same arithmetic for [outer, R, inner] with inner a multiple of 4, laid out so that nothing is recomputed per element:
// grid (ceil(inner / 256), ceil(R / kQuantRows), outer), 256 threads = 4 row lanes x 64 column quads. A thread keeps its
// four columns, works out their four scales once (the element-per-thread kernels divide amax / qmax again for every
// element and pay two 64-bit index divisions per thread) and walks kQuantRows / 4 rows with 16-byte loads.
constexpr int kQuantRows = 32;
template <int DT, int QT>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const void *__restrict__ w, const uint32_t *__restrict__ amax_bits,
                                                            void *__restrict__ q, void *__restrict__ scale, int64_t R,
                                                            int64_t inner4) {
    const float qmax = QT == HIDET_QMM_I8 ? 127.0f : 32767.0f;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t c4 = int64_t(blockIdx.x) * 64 + tx;
    if (c4 >= inner4) return;
    const int64_t o = blockIdx.z;
    const int64_t sidx = (o * inner4 + c4) * 4;
    const uint4 ab = *reinterpret_cast<const uint4 *>(amax_bits + sidx);
    const uint32_t abits[4] = {ab.x, ab.y, ab.z, ab.w};
    float s[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] = round_to<DT>(__uint_as_float(abits[e]) / qmax);
    if (blockIdx.y == 0 && ty == 0) {
#pragma unroll
        for (int e = 0; e < 4; ++e) store_from_f32<DT>(scale, sidx + e, s[e]);
    }
    const int64_t r_end = min(R, (int64_t(blockIdx.y) + 1) * kQuantRows);
    for (int64_t r = int64_t(blockIdx.y) * kQuantRows + ty; r < r_end; r += 4) {
        const int64_t i4 = (o * R + r) * inner4 + c4;
        float x[4], code[4];
        load4_as_f32<DT>(w, i4, x);
#pragma unroll
        for (int e = 0; e < 4; ++e) code[e] = s[e] != 0.0f ? round_code<DT>(round_to<DT>(x[e] / s[e])) : 0.0f;
        if (QT == HIDET_QMM_I8) {
            uint32_t packed = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) packed |= uint32_t(uint8_t(int8_t(fminf(fmaxf(code[e], -128.0f), 127.0f)))) << (8 * e);
            static_cast<uint32_t *>(q)[i4] = packed;
        } else {
            uint32_t h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = uint32_t(uint16_t(int16_t(fminf(fmaxf(code[e], -32768.0f), 32767.0f))));
            static_cast<uint2 *>(q)[i4] = uint2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        }
    }
}

// inner == 1 (one scale per row, e.g. an embedding table): one workgroup per row keeps the whole row in registers
// between the amax pass and the quantization, so the tensor is read once. Rows of up to 256 * 4 * NV elements, a
// multiple of 4, 16-byte aligned. Same arithmetic as above.
template <int DT, int QT, int NV>
__global__ __launch_bounds__(256) void quantize_row_fused_kernel(const void *__restrict__ w, void *__restrict__ q,
                                                                 void *__restrict__ scale, int64_t R4) {
    __shared__ float red[4];
    const float qmax = QT == HIDET_QMM_I8 ? 127.0f : 32767.0f;
    const int tid = threadIdx.x;
    const int64_t base4 = int64_t(blockIdx.x) * R4;
    float x[NV][4];
    float m = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t j = int64_t(v) * 256 + tid;
        x[v][0] = x[v][1] = x[v][2] = x[v][3] = 0.0f;
        if (j < R4) load4_as_f32<DT>(w, base4 + j, x[v]);
#pragma unroll
        for (int e = 0; e < 4; ++e) m = fmaxf(m, fabsf(x[v][e]));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = round_to<DT>(m / qmax);
    if (tid == 0) store_from_f32<DT>(scale, blockIdx.x, s);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int64_t j = int64_t(v) * 256 + tid;
        if (j >= R4) continue;
        float code[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) code[e] = s != 0.0f ? round_code<DT>(round_to<DT>(x[v][e] / s)) : 0.0f;
        if (QT == HIDET_QMM_I8) {
            uint32_t packed = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) packed |= uint32_t(uint8_t(int8_t(fminf(fmaxf(code[e], -128.0f), 127.0f)))) << (8 * e);
            static_cast<uint32_t *>(q)[base4 + j] = packed;
        } else {
            uint32_t h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = uint32_t(uint16_t(int16_t(fminf(fmaxf(code[e], -32768.0f), 32767.0f))));
            static_cast<uint2 *>(q)[base4 + j] = uint2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        }
    }
}

template <int QT, int ST>
__global__ __launch_bounds__(256) void dequantize_kernel(const void *__restrict__ q, const void *__restrict__ scale,
                                                         void *__restrict__ w, int64_t R, int64_t inner, int64_t total) {
    int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int64_t o = i / (R * inner);
    const int64_t c = (i - o * R * inner) % inner;
    const float code = QT == HIDET_QMM_I8 ? float(static_cast<const int8_t *>(q)[i]) : float(static_cast<const int16_t *>(q)[i]);
    store_from_f32<ST>(w, i, round_to<ST>(code * load_as_f32<ST>(scale, o * inner + c)));
}

// Four consecutive elements per thread: along the innermost axis (inner4 = inner / 4, one scale each) or, with
// ALONG_REDUCE (inner == 1, R = reduce / 4), along the reduced axis (one scale for all four).
template <int QT, int ST, bool ALONG_REDUCE>
__global__ __launch_bounds__(256) void dequantize4_kernel(const void *__restrict__ q, const void *__restrict__ scale,
                                                          void *__restrict__ w, int64_t R, int64_t inner4, int64_t total4) {
    const int64_t i4 = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i4 >= total4) return;
    float code[4], sc[4];
    if (QT == HIDET_QMM_I8) {
        const uint32_t v = static_cast<const uint32_t *>(q)[i4];
#pragma unroll
        for (int e = 0; e < 4; ++e) code[e] = float(int8_t(v >> (8 * e)));
    } else {
        const uint2 v = static_cast<const uint2 *>(q)[i4];
        code[0] = float(int16_t(v.x)); code[1] = float(int16_t(v.x >> 16));
        code[2] = float(int16_t(v.y)); code[3] = float(int16_t(v.y >> 16));
    }
    if (ALONG_REDUCE) {
        sc[0] = sc[1] = sc[2] = sc[3] = load_as_f32<ST>(scale, i4 / R);
    } else {
        const int64_t row = i4 / inner4;
        const int64_t sidx = ((row / R) * inner4 + (i4 - row * inner4)) * 4;
        load4_as_f32<ST>(scale, sidx / 4, sc);
    }
    float out[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = round_to<ST>(code[e] * sc[e]);
    if (ST == HIDET_QMM_F32) {
        static_cast<float4 *>(w)[i4] = float4{out[0], out[1], out[2], out[3]};
    } else {
        uint32_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = ST == HIDET_QMM_F16 ? f32_to_f16_bits(out[e]) : f32_to_bf16_bits(out[e]);
        static_cast<uint2 *>(w)[i4] = uint2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
    }
}

// Group-wise int4: grid (ceil(n/128), k/group); 256 threads = 4 row lanes x 64 column pairs.
// scale32 = amax / 7 and code = clamp(round_half_away(w / scale32), -7, 7) in float32; two codes per
// byte along n, low nibble first; the stored scale is scale32 rounded to the scale dtype.
template <int ST>
__global__ __launch_bounds__(256) void group_quantize_int4_kernel(const float *__restrict__ w, uint8_t *__restrict__ packed,
                                                                  void *__restrict__ scales, int64_t n, int group) {
    __shared__ float red[4][128];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t c0 = int64_t(blockIdx.x) * 128 + 2 * tx;
    const int64_t g = blockIdx.y;
    const int64_t rbase = g * group;
    const bool ok = c0 < n;  // n is even: the pair is in or out together
    float m0 = 0.0f, m1 = 0.0f;
    if (ok) {
        for (int r = ty; r < group; r += 4) {
            float2 v = *reinterpret_cast<const float2 *>(w + (rbase + r) * n + c0);
            m0 = fmaxf(m0, fabsf(v.x));
            m1 = fmaxf(m1, fabsf(v.y));
        }
    }
    red[ty][2 * tx] = m0;
    red[ty][2 * tx + 1] = m1;
    __syncthreads();
    if (!ok) return;
    m0 = fmaxf(fmaxf(red[0][2 * tx], red[1][2 * tx]), fmaxf(red[2][2 * tx], red[3][2 * tx]));
    m1 = fmaxf(fmaxf(red[0][2 * tx + 1], red[1][2 * tx + 1]), fmaxf(red[2][2 * tx + 1], red[3][2 * tx + 1]));
    const float s0 = m0 / 7.0f, s1 = m1 / 7.0f;
    if (ty == 0) {
        store_from_f32<ST>(scales, g * n + c0, round_to<ST>(s0));
        store_from_f32<ST>(scales, g * n + c0 + 1, round_to<ST>(s1));
    }
    for (int r = ty; r < group; r += 4) {
        float2 v = *reinterpret_cast<const float2 *>(w + (rbase + r) * n + c0);
        float q0 = s0 == 0.0f ? 0.0f : fminf(fmaxf(roundf(v.x / s0), -7.0f), 7.0f);
        float q1 = s1 == 0.0f ? 0.0f : fminf(fmaxf(roundf(v.y / s1), -7.0f), 7.0f);
        packed[((rbase + r) * n + c0) >> 1] = uint8_t((int(q0) & 0xF) | ((int(q1) & 0xF) << 4));
    }
}

// ---- per-tensor float8 e4m3 -------------------------------------------------------------------

template <int DT>
__global__ __launch_bounds__(256) void amax_all_kernel(const void *__restrict__ x, uint32_t *__restrict__ amax_bits, int64_t numel) {
    __shared__ float red[4];
    float m = 0.0f;
    for (int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x; i < numel; i += int64_t(gridDim.x) * 256)
        m = fmaxf(m, fabsf(load_as_f32<DT>(x, i)));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        atomicMax(amax_bits, __float_as_uint(m));
    }
}

template <int DT>
__global__ __launch_bounds__(256) void fp8_quantize_kernel(const void *__restrict__ x, const uint32_t *__restrict__ amax_bits,
                                                           uint8_t *__restrict__ codes, float *__restrict__ scale, int64_t numel) {
    const float s = __uint_as_float(*amax_bits) / 448.0f;
    int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i == 0) *scale = s;
    if (i >= numel) return;
    codes[i] = s == 0.0f ? uint8_t(0) : f32_to_e4m3(load_as_f32<DT>(x, i) / s);
}

template <int DT>
__global__ __launch_bounds__(256) void amax_all4_kernel(const void *__restrict__ x, uint32_t *__restrict__ amax_bits, int64_t numel4) {
    __shared__ float red[4];
    float m = 0.0f;
    // chunks of 256 threads x 8 independent vector loads, contiguous per workgroup: with one load in flight per thread
    // this pass ran at 1.9 TB/s
    constexpr int kLoads = 8;
    if (DT != HIDET_QMM_F32 && (numel4 & 1) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        // 16-bit input: 16 bytes = 8 values per load; |x| as an integer compare on the 15 value bits (same order as the
        // floats for finite values; the reduction below continues in float)
        const int64_t numel8 = numel4 >> 1;
        constexpr uint32_t kInfBits = DT == HIDET_QMM_F16 ? 0x7C00u : 0x7F80u;
        uint32_t mb = 0;
        for (int64_t base = int64_t(blockIdx.x) * (256 * kLoads); base < numel8; base += int64_t(gridDim.x) * (256 * kLoads)) {
            uint4 v[kLoads];
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
                const int64_t i = base + j * 256 + threadIdx.x;
                v[j] = uint4{0u, 0u, 0u, 0u};
                if (i < numel8) v[j] = static_cast<const uint4 *>(x)[i];
            }
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
                const uint32_t w4[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t lo = w4[e] & 0x7FFFu, hi = (w4[e] >> 16) & 0x7FFFu;
                    mb = max(mb, max(lo > kInfBits ? 0u : lo, hi > kInfBits ? 0u : hi));  // a NaN is skipped, as fmaxf skips it
                }
            }
        }
        m = DT == HIDET_QMM_F16 ? f16_bits_to_f32(uint16_t(mb)) : bf16_bits_to_f32(uint16_t(mb));
    } else {
        for (int64_t base = int64_t(blockIdx.x) * (256 * kLoads); base < numel4; base += int64_t(gridDim.x) * (256 * kLoads)) {
            float v[kLoads][4];
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
                const int64_t i = base + j * 256 + threadIdx.x;
                v[j][0] = v[j][1] = v[j][2] = v[j][3] = 0.0f;
                if (i < numel4) load4_as_f32<DT>(x, i, v[j]);
            }
#pragma unroll
            for (int j = 0; j < kLoads; ++j)
                m = fmaxf(fmaxf(m, fmaxf(fabsf(v[j][0]), fabsf(v[j][1]))), fmaxf(fabsf(v[j][2]), fabsf(v[j][3])));
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        atomicMax(amax_bits, __float_as_uint(m));
    }
}

// Small tensors (the activations of a decode step): one workgroup of 1024 threads keeps up to 65536 elements in registers
// between the amax and the conversion - one launch instead of three. Same arithmetic as fp8_quantize4_kernel.
template <int DT>
__global__ __launch_bounds__(1024) void fp8_quantize_small_kernel(const void *__restrict__ x, uint32_t *__restrict__ codes,
                                                                  float *__restrict__ scale, int numel4) {
    __shared__ float red[16];
    const int tid = threadIdx.x;
    float v[16][4];
    float m = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int i = j * 1024 + tid;
        v[j][0] = v[j][1] = v[j][2] = v[j][3] = 0.0f;
        if (i < numel4) load4_as_f32<DT>(x, i, v[j]);
#pragma unroll
        for (int e = 0; e < 4; ++e) m = fmaxf(m, fabsf(v[j][e]));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    m = red[0];
#pragma unroll
    for (int wv = 1; wv < 16; ++wv) m = fmaxf(m, red[wv]);
    const float s = m / 448.0f;
    if (tid == 0) *scale = s;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int i = j * 1024 + tid;
        if (i >= numel4) continue;
        uint32_t packed = 0;
        if (s != 0.0f) {
            float q[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) q[e] = fminf(fmaxf(v[j][e] / s, -448.0f), 448.0f);
            int p = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
            p = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], p, true);
            packed = uint32_t(p);
        }
        codes[i] = packed;
    }
}

// The quotient is clamped to +-448 (what saturation means for a format whose largest finite value is 448) and converted
// by the hardware's round-to-nearest-even OCP e4m3 conversion, two values per instruction.
template <int DT>
__global__ __launch_bounds__(256) void fp8_quantize4_kernel(const void *__restrict__ x, const uint32_t *__restrict__ amax_bits,
                                                            uint32_t *__restrict__ codes, float *__restrict__ scale, int64_t numel4) {
    const float s = __uint_as_float(*amax_bits) / 448.0f;
    if (blockIdx.x == 0 && threadIdx.x == 0) *scale = s;
    // four independent vector loads per thread (a workgroup converts 1024 consecutive groups of four values)
    float v[4][4];
    const int64_t base = int64_t(blockIdx.x) * 1024 + threadIdx.x;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (base + j * 256 < numel4) load4_as_f32<DT>(x, base + j * 256, v[j]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t i = base + j * 256;
        if (i >= numel4) continue;
        uint32_t packed = 0;
        if (s != 0.0f) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[j][e] = fminf(fmaxf(v[j][e] / s, -448.0f), 448.0f);
            int p = __builtin_amdgcn_cvt_pk_fp8_f32(v[j][0], v[j][1], 0, false);
            p = __builtin_amdgcn_cvt_pk_fp8_f32(v[j][2], v[j][3], p, true);
            packed = uint32_t(p);
        }
        codes[i] = packed;
    }
}

template <typename F>
void dispatch_float(int dt, F &&f) {
    switch (dt) {
        case HIDET_QMM_F32: f(std::integral_constant<int, HIDET_QMM_F32>()); break;
        case HIDET_QMM_F16: f(std::integral_constant<int, HIDET_QMM_F16>()); break;
        case HIDET_QMM_BF16: f(std::integral_constant<int, HIDET_QMM_BF16>()); break;
        default: QMM_FAIL("expected a float32, float16 or bfloat16 dtype code, got " << dt);
    }
}

}  // namespace
}  // namespace qmm

using namespace qmm;

HIDET_API void hidet_symmetric_quantize(const void *w, void *wq, void *scale, int64_t outer, int64_t reduce,
                                        int64_t inner, int w_dtype, int q_dtype, void *workspace,
                                        int64_t workspace_bytes, void *stream_) {
    QMM_ENTRY_BEGIN
    QMM_CHECK(q_dtype == HIDET_QMM_I8 || q_dtype == HIDET_QMM_I16, "quant_type must be int8 or int16, got code " << q_dtype);
    QMM_CHECK(outer >= 0 && reduce >= 0 && inner >= 0, "negative extent");
    const int64_t total = outer * reduce * inner;
    const int64_t nscale = outer * inner;
    if (nscale == 0) return;
    QMM_CHECK(scale && (total == 0 || (w && wq)), "null tensor pointer");
    QMM_CHECK(inner < (int64_t(1) << 31) * 64 && outer < 65536 * int64_t(4), "extent too large");
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    QMM_CHECK(ws.scratch_bytes >= nscale * 4, "workspace too small: its scratch part (three quarters of what follows the first 64 KiB) must hold "
                                                  << nscale * 4 << " bytes, got a workspace of " << workspace_bytes);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    uint32_t *amax_bits = reinterpret_cast<uint32_t *>(ws.scratch);
    dispatch_float(w_dtype, [&](auto dt) {
        constexpr int DT = decltype(dt)::value;
        {
            // rows that fit a workgroup's registers: one pass
            const int esize0 = DT == HIDET_QMM_F32 ? 4 : 2, qsize0 = q_dtype == HIDET_QMM_I8 ? 1 : 2;
            if (inner == 1 && reduce > 0 && reduce % 4 == 0 && reduce <= 256 * 4 * 16 && outer < (int64_t(1) << 31) &&
                aligned(w, 4 * esize0) && aligned(wq, 4 * qsize0) && aligned(scale, esize0)) {
                auto go = [&](auto kern) { launch(kern, dim3(uint32_t(outer)), dim3(256), 0, stream, w, wq, scale, reduce / 4); };
                const bool small = reduce <= 256 * 4 * 4;
                if (q_dtype == HIDET_QMM_I8) small ? go(quantize_row_fused_kernel<DT, HIDET_QMM_I8, 4>) : go(quantize_row_fused_kernel<DT, HIDET_QMM_I8, 16>);
                else small ? go(quantize_row_fused_kernel<DT, HIDET_QMM_I16, 4>) : go(quantize_row_fused_kernel<DT, HIDET_QMM_I16, 16>);
                return;
            }
        }
        if (reduce == 0) {
            launch_aux(fill_u32_kernel, dim3(cdiv(nscale, 256)), dim3(256), 0, stream, amax_bits, nscale, 0u);
        } else if (inner == 1) {
            launch(amax_contig_kernel<DT>, dim3(cdiv(outer, 4)), dim3(256), 0, stream, w, amax_bits, outer, reduce);
        } else {
            QMM_CHECK(outer <= 65535, "outer extent " << outer << " exceeds the grid limit");
            const int64_t col_blocks = cdiv(inner, 64);
            int64_t splits = 1;
            if (col_blocks * outer < 1024) splits = std::min<int64_t>(cdiv(1024, col_blocks * outer), cdiv(reduce, 64));
            splits = std::max<int64_t>(1, std::min<int64_t>(splits, 65535));
            const int64_t rows_per_split = cdiv(cdiv(reduce, splits), 4) * 4;
            splits = cdiv(reduce, rows_per_split);
            if (splits > 1) launch_aux(fill_u32_kernel, dim3(cdiv(nscale, 256)), dim3(256), 0, stream, amax_bits, nscale, 0u);
            launch(amax_strided_kernel<DT>, dim3(col_blocks, outer, splits), dim3(256), 0, stream, w, amax_bits, reduce,
                   inner, rows_per_split, int(splits > 1));
        }
        if (total == 0) return;
        const int esize = DT == HIDET_QMM_F32 ? 4 : 2, qsize = q_dtype == HIDET_QMM_I8 ? 1 : 2;
        const bool vec_ok = aligned(w, 4 * esize) && aligned(wq, 4 * qsize) && aligned(scale, esize);
        if (vec_ok && inner % 4 == 0) {
            const int64_t row_blocks = cdiv(reduce, kQuantRows);
            if (row_blocks <= 65535 && outer <= 65535) {
                const dim3 grid(uint32_t(cdiv(inner / 4, 64)), uint32_t(row_blocks), uint32_t(outer));
                if (q_dtype == HIDET_QMM_I8)
                    launch(quantize_rows_kernel<DT, HIDET_QMM_I8>, grid, dim3(256), 0, stream, w, amax_bits, wq, scale, reduce, inner / 4);
                else
                    launch(quantize_rows_kernel<DT, HIDET_QMM_I16>, grid, dim3(256), 0, stream, w, amax_bits, wq, scale, reduce, inner / 4);
                return;
            }
            if (q_dtype == HIDET_QMM_I8)
                launch(quantize4_kernel<DT, HIDET_QMM_I8, false>, dim3(cdiv(total / 4, 256)), dim3(256), 0, stream, w, amax_bits,
                       wq, scale, reduce, inner / 4, total / 4);
            else
                launch(quantize4_kernel<DT, HIDET_QMM_I16, false>, dim3(cdiv(total / 4, 256)), dim3(256), 0, stream, w, amax_bits,
                       wq, scale, reduce, inner / 4, total / 4);
            return;
        }
        if (vec_ok && inner == 1 && reduce % 4 == 0) {
            if (q_dtype == HIDET_QMM_I8)
                launch(quantize4_kernel<DT, HIDET_QMM_I8, true>, dim3(cdiv(total / 4, 256)), dim3(256), 0, stream, w, amax_bits,
                       wq, scale, reduce / 4, int64_t(0), total / 4);
            else
                launch(quantize4_kernel<DT, HIDET_QMM_I16, true>, dim3(cdiv(total / 4, 256)), dim3(256), 0, stream, w, amax_bits,
                       wq, scale, reduce / 4, int64_t(0), total / 4);
            return;
        }
        if (q_dtype == HIDET_QMM_I8)
            launch(quantize_kernel<DT, HIDET_QMM_I8>, dim3(cdiv(total, 256)), dim3(256), 0, stream, w, amax_bits, wq, scale,
                   reduce, inner, total);
        else
            launch(quantize_kernel<DT, HIDET_QMM_I16>, dim3(cdiv(total, 256)), dim3(256), 0, stream, w, amax_bits, wq, scale,
                   reduce, inner, total);
    });
    if (reduce == 0) {
        // no elements: scale = 0 still has to be written
        dispatch_float(w_dtype, [&](auto dt) {
            constexpr int DT = decltype(dt)::value;
            if (DT == HIDET_QMM_F32) launch_aux(fill_u32_kernel, dim3(cdiv(nscale, 256)), dim3(256), 0, stream, static_cast<uint32_t *>(scale), nscale, 0u);
            else launch_aux(fill_u32_kernel, dim3(cdiv(cdiv(nscale, 2), 256)), dim3(256), 0, stream, static_cast<uint32_t *>(scale), cdiv(nscale, 2), 0u);
        });
    }
    QMM_ENTRY_END
}

HIDET_API void hidet_symmetric_dequantize(const void *wq, const void *scale, void *w, int64_t outer, int64_t reduce,
                                          int64_t inner, int q_dtype, int s_dtype, void *stream_) {
    QMM_ENTRY_BEGIN
    QMM_CHECK(q_dtype == HIDET_QMM_I8 || q_dtype == HIDET_QMM_I16, "quantized dtype must be int8 or int16, got code " << q_dtype);
    const int64_t total = outer * reduce * inner;
    if (total == 0) return;
    QMM_CHECK(w && wq && scale, "null tensor pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    dispatch_float(s_dtype, [&](auto dt) {
        constexpr int ST = decltype(dt)::value;
        const int esize = ST == HIDET_QMM_F32 ? 4 : 2, qsize = q_dtype == HIDET_QMM_I8 ? 1 : 2;
        const bool vec_ok = aligned(w, 4 * esize) && aligned(wq, 4 * qsize) && aligned(scale, 4 * esize);
        auto go4 = [&](auto kern, int64_t r4, int64_t in4) {
            launch(kern, dim3(cdiv(total / 4, 256)), dim3(256), 0, stream, wq, scale, w, r4, in4, total / 4);
        };
        if (vec_ok && inner % 4 == 0) {
            if (q_dtype == HIDET_QMM_I8) go4(dequantize4_kernel<HIDET_QMM_I8, ST, false>, reduce, inner / 4);
            else go4(dequantize4_kernel<HIDET_QMM_I16, ST, false>, reduce, inner / 4);
            return;
        }
        if (vec_ok && inner == 1 && reduce % 4 == 0) {
            if (q_dtype == HIDET_QMM_I8) go4(dequantize4_kernel<HIDET_QMM_I8, ST, true>, reduce / 4, int64_t(0));
            else go4(dequantize4_kernel<HIDET_QMM_I16, ST, true>, reduce / 4, int64_t(0));
            return;
        }
        if (q_dtype == HIDET_QMM_I8)
            launch(dequantize_kernel<HIDET_QMM_I8, ST>, dim3(cdiv(total, 256)), dim3(256), 0, stream, wq, scale, w, reduce, inner, total);
        else
            launch(dequantize_kernel<HIDET_QMM_I16, ST>, dim3(cdiv(total, 256)), dim3(256), 0, stream, wq, scale, w, reduce, inner, total);
    });
    QMM_ENTRY_END
}

HIDET_API void hidet_group_quantize_int4(const void *w, void *packed, void *scales, int64_t k, int64_t n, int group_size,
                                         int w_dtype, int s_dtype, void *stream_) {
    QMM_ENTRY_BEGIN
    QMM_CHECK(w_dtype == HIDET_QMM_F32, "group_quantize_int4 expects float32 weights, got dtype code " << w_dtype);
    QMM_CHECK(group_size > 0 && k % group_size == 0, "K (" << k << ") must be a multiple of the group size (" << group_size << ")");
    QMM_CHECK(n % 2 == 0, "N (" << n << ") must be even: two codes are packed per byte");
    if (k == 0 || n == 0) return;
    QMM_CHECK(w && packed && scales, "null tensor pointer");
    QMM_CHECK(aligned(w, 8), "weight pointer must be 8-byte aligned");
    QMM_CHECK(k / group_size <= 65535, "too many groups");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    dispatch_float(s_dtype, [&](auto dt) {
        constexpr int ST = decltype(dt)::value;
        launch(group_quantize_int4_kernel<ST>, dim3(cdiv(n, 128), k / group_size), dim3(256), 0, stream,
               static_cast<const float *>(w), static_cast<uint8_t *>(packed), scales, n, group_size);
    });
    QMM_ENTRY_END
}

HIDET_API void hidet_fp8_quantize_per_tensor(const void *x, void *codes, void *scale, int64_t numel, int x_dtype,
                                             void *workspace, int64_t workspace_bytes, void *stream_) {
    QMM_ENTRY_BEGIN
    QMM_CHECK(scale, "null scale pointer");
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    QMM_CHECK(ws.scratch_bytes >= 4, "workspace too small");
    QMM_CHECK(numel == 0 || (x && codes), "null tensor pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    uint32_t *amax_bits = reinterpret_cast<uint32_t *>(ws.scratch);
    dispatch_float(x_dtype, [&](auto dt) {
        constexpr int DT = decltype(dt)::value;
        const int esize = DT == HIDET_QMM_F32 ? 4 : 2;
        if (numel > 0 && numel <= 65536 && numel % 4 == 0 && aligned(x, 4 * esize) && aligned(codes, 4)) {
            launch(fp8_quantize_small_kernel<DT>, dim3(1), dim3(1024), 0, stream, x, static_cast<uint32_t *>(codes),
                   static_cast<float *>(scale), int(numel / 4));
            return;
        }
        launch_aux(fill_u32_kernel, dim3(1), dim3(64), 0, stream, amax_bits, int64_t(1), 0u);
        if (numel > 0 && numel % 4 == 0 && aligned(x, 4 * esize) && aligned(codes, 4)) {
            const int64_t n4 = numel / 4;
            // at most 512 workgroups: each ends with one atomic on the same word, and 4096 of them took longer than the reads
            launch(amax_all4_kernel<DT>, dim3(std::min<int64_t>(cdiv(n4, 2048), 512)), dim3(256), 0, stream, x, amax_bits, n4);
            launch(fp8_quantize4_kernel<DT>, dim3(cdiv(n4, 1024)), dim3(256), 0, stream, x, amax_bits,
                   static_cast<uint32_t *>(codes), static_cast<float *>(scale), n4);
            return;
        }
        if (numel > 0) {
            const int64_t blocks = std::min<int64_t>(cdiv(numel, 256 * 8), 512);  // one atomic on one word per workgroup
            launch(amax_all_kernel<DT>, dim3(blocks), dim3(256), 0, stream, x, amax_bits, numel);
        }
        launch(fp8_quantize_kernel<DT>, dim3(std::max<int64_t>(1, cdiv(numel, 256))), dim3(256), 0, stream, x, amax_bits,
               static_cast<uint8_t *>(codes), static_cast<float *>(scale), numel);
    });
    QMM_ENTRY_END
}
