// Driver around the REFERENCE's own CPU half type -- TEST INFRASTRUCTURE ONLY.
//
// This file contains no reference code: it #includes include/hidet/runtime/cpu/float16.h
// from the reference checkout at build time (see the Makefile's `ref` target, output in
// oracle/_ref/) and exposes its conversions, its operators and the loop nest the
// reference's CPU scheduler emits for symmetric_quant_matmul, so that the restatement in
// cpu_ref.c can be compared with the real type bit for bit.
#include <cstdint>
#include <hidet/runtime/cpu/float16.h>

#define REF_API extern "C" __attribute__((visibility("default")))

static inline half from_bits(uint16_t b) { return half(b, half::from_bits()); }

REF_API uint16_t ref_f32_to_f16(float f) { return half(f).x; }
REF_API float ref_f16_to_f32(uint16_t h) { return float(from_bits(h)); }
REF_API uint16_t ref_half_mul(uint16_t a, uint16_t b) { return (from_bits(a) * from_bits(b)).x; }
REF_API uint16_t ref_half_add(uint16_t a, uint16_t b) { return (from_bits(a) + from_bits(b)).x; }
REF_API uint16_t ref_half_div(uint16_t a, uint16_t b) { return (from_bits(a) / from_bits(b)).x; }
REF_API uint16_t ref_half_round(uint16_t a) { return std::round(from_bits(a)).x; }

// c[i,j] = sum_k a[i,k] * (half(w[k,j]) * scale[j]) with a half accumulator: the expression of
// graph/ops/quant/matmul.py:57-72 evaluated as the CPU auto-scheduler does
// (ir/schedulers/base.py:347-371), one output element per flattened loop iteration.
REF_API void ref_quant_matmul_cpu(const uint16_t *a, const int8_t *w, const uint16_t *scale, uint16_t *c, int64_t m,
                                  int64_t k, int64_t n) {
    for (int64_t o = 0; o < m * n; ++o) {
        int64_t i = o / n, j = o % n;
        half acc = half(0.0f);
        for (int64_t kk = 0; kk < k; ++kk)
            acc = acc + from_bits(a[i * k + kk]) * (half((float)w[kk * n + j]) * from_bits(scale[j]));
        c[o] = acc.x;
    }
}

// symmetric.py:23-47 for a half matrix w[rows, cols] reduced over axis 0: scale = amax / 127 and
// code = (int8) round(w / scale), each operator on the reference's half type.
REF_API void ref_symmetric_quantize_f16_axis0(const uint16_t *w, int64_t rows, int64_t cols, int8_t *codes,
                                              uint16_t *scale) {
    for (int64_t c = 0; c < cols; ++c) {
        half m = half(0.0f);
        for (int64_t r = 0; r < rows; ++r) {
            half v = from_bits(w[r * cols + c]);
            half av = float(v) >= 0.0f ? v : -v;
            if (float(av) > float(m)) m = av;
        }
        half s = m / half(127.0f);
        scale[c] = s.x;
        for (int64_t r = 0; r < rows; ++r)
            codes[r * cols + c] = float(s) == 0.0f ? 0 : (int8_t)float(std::round(from_bits(w[r * cols + c]) / s));
    }
}
