// Device-side element access and rounding helpers keyed by the ABI's dtype codes.
#pragma once
#include "common.h"

namespace qmm {

template <int DT>
__device__ __forceinline__ float load_as_f32(const void *p, int64_t i) {
    if (DT == HIDET_QMM_F32) return static_cast<const float *>(p)[i];
    if (DT == HIDET_QMM_F16) return f16_bits_to_f32(static_cast<const uint16_t *>(p)[i]);
    return bf16_bits_to_f32(static_cast<const uint16_t *>(p)[i]);
}

// Round a float32 value to the precision of DT (nearest even) and return it widened again.
template <int DT>
__device__ __forceinline__ float round_to(float x) {
    if (DT == HIDET_QMM_F32) return x;
    if (DT == HIDET_QMM_F16) return f16_bits_to_f32(f32_to_f16_bits(x));
    return bf16_bits_to_f32(f32_to_bf16_bits(x));
}

// Store a value that is already representable in DT.
template <int DT>
__device__ __forceinline__ void store_from_f32(void *p, int64_t i, float x) {
    if (DT == HIDET_QMM_F32) static_cast<float *>(p)[i] = x;
    else if (DT == HIDET_QMM_F16) static_cast<uint16_t *>(p)[i] = f32_to_f16_bits(x);
    else static_cast<uint16_t *>(p)[i] = f32_to_bf16_bits(x);
}

// float32 -> OCP e4m3fn code: round to nearest even, saturate to +-448 (infinities too), NaN -> 0x7F.
// Integer arithmetic only, so the result does not depend on any conversion instruction's mode.
__device__ __forceinline__ uint8_t f32_to_e4m3(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return uint8_t(sign | 0x7Fu);
    if (a >= 0x43E00000u) return uint8_t(sign | 0x7Eu);  // >= 448
    if (a <= 0x3A800000u) return uint8_t(sign);          // <= 2^-10: rounds to zero (tie goes to even)
    const int e = int(a >> 23) - 127;
    uint32_t man = a & 0x7FFFFFu;
    uint32_t shift, base;
    if (e >= -6) {
        shift = 20;
        base = uint32_t(e + 7) << 3;
    } else {  // subnormal target: unit 2^-9
        man |= 0x800000u;
        shift = uint32_t(14 - e);
        base = 0;
    }
    const uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t r = base + q;
    if (rem > half || (rem == half && (q & 1u))) r += 1;
    return uint8_t(sign | r);
}

__device__ __forceinline__ float e4m3_to_f32(uint8_t c) {
    const uint32_t sign = uint32_t(c & 0x80u) << 24;
    const uint32_t e = (c >> 3) & 0xFu, m = c & 7u;
    float v;
    if (e == 0) v = float(m) * 0.001953125f;  // m * 2^-9
    else if (e == 15 && m == 7) v = __uint_as_float(0x7FC00000u);
    else v = __uint_as_float(((e + 120u) << 23) | (m << 20));
    return __uint_as_float(__float_as_uint(v) | sign);
}

// float32 -> OCP e5m2 code: round to nearest even, finite values and infinities saturate to +-57344 (0x7B), NaN -> 0x7F:
// what the reference's float8_e5m2 type does on conversion (include/hidet/runtime/cuda/float8_e5m2.h:6, the
// saturate-to-finite constructor of the vendor's e5m2 type). Integer arithmetic only.
__device__ __forceinline__ uint8_t f32_to_e5m2(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return uint8_t(sign | 0x7Fu);
    if (a >= 0x47600000u) return uint8_t(sign | 0x7Bu);  // >= 57344
    if (a <= 0x37000000u) return uint8_t(sign);          // <= 2^-17: rounds to zero (tie goes to even)
    const int e = int(a >> 23) - 127;
    uint32_t man = a & 0x7FFFFFu;
    uint32_t shift, base;
    if (e >= -14) {
        shift = 21;
        base = uint32_t(e + 15) << 2;
    } else {  // subnormal target: unit 2^-16
        man |= 0x800000u;
        shift = uint32_t(7 - e);
        base = 0;
    }
    const uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t r = base + q;
    if (rem > half || (rem == half && (q & 1u))) r += 1;
    if (r > 0x7Bu) r = 0x7Bu;  // rounded up past the largest finite value
    return uint8_t(sign | r);
}

// An e5m2 code is the upper byte of the float16 with the same value.
__device__ __forceinline__ float e5m2_to_f32(uint8_t c) { return f16_bits_to_f32(uint16_t(uint16_t(c) << 8)); }

// Element formats of the fp8 MFMA (its cbsz / blgp fields).
constexpr int kFmtE4M3 = 0, kFmtE5M2 = 1;
template <int FMT>
__device__ __forceinline__ float fp8_to_f32(uint8_t c) { return FMT == kFmtE5M2 ? e5m2_to_f32(c) : e4m3_to_f32(c); }

// One output element from float32, for the element-wise epilogues.
template <int OUT>
__device__ __forceinline__ void store_out(void *c, int64_t o, float v) {
    if (OUT == HIDET_QMM_F32) static_cast<float *>(c)[o] = v;
    else if (OUT == HIDET_QMM_BF16) static_cast<uint16_t *>(c)[o] = f32_to_bf16_bits(v);
    else if (OUT == HIDET_QMM_F16) static_cast<uint16_t *>(c)[o] = f32_to_f16_bits(v);
    else if (OUT == HIDET_QMM_E5M2) static_cast<uint8_t *>(c)[o] = f32_to_e5m2(v);
    else static_cast<uint8_t *>(c)[o] = f32_to_e4m3(v);
}

}  // namespace qmm
