/*
 * C restatement of the reference's quantized-matmul arithmetic -- TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker and the CPU baseline for the HIP kernels.  Nothing in the
 * product library links or calls it.  Each function cites the reference file:line it
 * follows (paths relative to the reference checkout).
 *
 * Built strictly (no -ffast-math) so that divisions and roundings are IEEE.  The timing
 * loop nest that mimics the reference's CPU build flags lives in cpu_baseline.c.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "half_sw.h"

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API uint16_t oracle_f32_to_f16(float f) { return half_from_f32(f); }
ORACLE_API float oracle_f16_to_f32(uint16_t h) { return half_to_f32(h); }

ORACLE_API float oracle_roundf(float x) { return roundf(x); }

/* ---- symmetric quantization of a float32 matrix w[rows, cols] --------------------------
 * graph/ops/quant/symmetric.py:23-47: amax over the reduced axis, scale = amax / qmax,
 * code = (int) round(w / scale), all in float32 (w's dtype), ties away from zero
 * (ir/primitives/cpu/math/float32.py:40).  reduce_axis 0: one scale per column; 1: per row.
 * code_bytes is 1 (int8) or 2 (int16).  amax == 0 gives scale 0 and code 0 (the reference
 * leaves 0/0 undefined). */
ORACLE_API void oracle_symmetric_quantize_f32(const float *w, int64_t rows, int64_t cols, int reduce_axis,
                                              int qmax, int code_bytes, void *codes, float *scale) {
    int64_t ns = reduce_axis == 0 ? cols : rows;
    for (int64_t s = 0; s < ns; ++s) scale[s] = 0.0f;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float v = fabsf(w[r * cols + c]);
            int64_t s = reduce_axis == 0 ? c : r;
            if (v > scale[s]) scale[s] = v;
        }
    for (int64_t s = 0; s < ns; ++s) scale[s] = scale[s] / (float)qmax;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float sc = scale[reduce_axis == 0 ? c : r];
            float q = sc == 0.0f ? 0.0f : roundf(w[r * cols + c] / sc);
            if (code_bytes == 1) ((int8_t *)codes)[r * cols + c] = (int8_t)q;
            else ((int16_t *)codes)[r * cols + c] = (int16_t)q;
        }
}

/* ---- W8A16 parity target: dequantize (float16) then matmul with float32 accumulation ---
 * graph/ops/quant/matmul.py:57-72 for the operand order: wd = f16(f16(q) * scale) first,
 * then sum_k a * wd.  Products of two float16 values are exact in float32. */
ORACLE_API void oracle_quant_matmul_f32acc(const uint16_t *a, const int8_t *w, const uint16_t *scale, uint16_t *c,
                                           int64_t m, int64_t k, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t j0 = 0; j0 < n; j0 += 64) {
        int64_t jn = n - j0 < 64 ? n - j0 : 64;
        float sc[64], acc[64];
        for (int64_t j = 0; j < jn; ++j) sc[j] = half_to_f32(scale[j0 + j]);
        for (int64_t i = 0; i < m; ++i) {
            for (int64_t j = 0; j < jn; ++j) acc[j] = 0.0f;
            for (int64_t kk = 0; kk < k; ++kk) {
                float av = half_to_f32(a[i * k + kk]);
                const int8_t *wr = w + kk * n + j0;
                for (int64_t j = 0; j < jn; ++j) {
                    float wd = half_to_f32(half_from_f32((float)wr[j] * sc[j]));
                    acc[j] += av * wd;
                }
            }
            for (int64_t j = 0; j < jn; ++j) c[i * n + j0 + j] = half_from_f32(acc[j]);
        }
    }
}

/* ---- the reference's CPU route, strict build -------------------------------------------
 * One output element per iteration of a flattened parallel loop, serial k, every multiply
 * and add rounded to float16, float16 accumulator (ir/schedulers/cpu/scheduler.py:24-52,
 * ir/schedulers/base.py:347-371, backend/codegen.py:573-592,
 * include/hidet/runtime/cpu/float16.h:424-444). */
ORACLE_API void oracle_quant_matmul_ref_cpu(const uint16_t *a, const int8_t *w, const uint16_t *scale, uint16_t *c,
                                            int64_t m, int64_t k, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t o = 0; o < m * n; ++o) {
        int64_t i = o / n, j = o % n;
        float sc = half_to_f32(scale[j]);
        uint16_t acc = 0;
        for (int64_t kk = 0; kk < k; ++kk) {
            /* cast(weight, f16) is exact for int8 */
            uint16_t wd = half_from_f32((float)w[kk * n + j] * sc);
            uint16_t pr = half_from_f32(half_to_f32(a[i * k + kk]) * half_to_f32(wd));
            acc = half_from_f32(half_to_f32(acc) + half_to_f32(pr));
        }
        c[o] = acc;
    }
}
