// Group-wise int4 weights: how a 4-bit code becomes a 16-bit float of the activation type inside the decode kernels.
// A two's-complement nibble with its top bit flipped, u = nibble ^ 8 = q + 8, or-ed under the bit pattern of 2^7
// (bfloat16, 7 mantissa bits) or 2^10 (float16) is the float 128 + u = 136 + q or 1024 + u = 1032 + q; kMagic does both
// (the xor with 8 and the exponent) for two codes at bits 0-3 and 16-19 of a register.  The constant is removed after
// the MFMA with kBias * sum_k a[m, k].
#pragma once
#include "common.h"
#include "numeric.h"

namespace qmm {

template <int DT>
struct W4Traits;
template <>
struct W4Traits<HIDET_QMM_BF16> {
    static constexpr uint32_t kMagic = 0x43084308u;
    static constexpr float kBias = 136.0f;
    static constexpr uint16_t kOne = 0x3F80;
    static __device__ __forceinline__ float4_t mfma(const uint4 &a, const uint4 &b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t b) { return bf16_bits_to_f32(b); }
};
template <>
struct W4Traits<HIDET_QMM_F16> {
    static constexpr uint32_t kMagic = 0x64086408u;
    static constexpr float kBias = 1032.0f;
    static constexpr uint16_t kOne = 0x3C00;
    static __device__ __forceinline__ float4_t mfma(const uint4 &a, const uint4 &b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(uint16_t b) { return f16_bits_to_f32(b); }
};

}  // namespace qmm
