/*
 * Timing restatement of the reference's CPU route for symmetric_quant_matmul -- TEST
 * INFRASTRUCTURE ONLY: it is the benchmark's CPU baseline, never the product.
 *
 * Same loop nest as oracle_quant_matmul_ref_cpu, but this file is compiled with the flag
 * set the reference's CPU build uses (backend/build.py:318-350: -O3 -mavx2 -m64
 * -ffast-math -fopenmp; -march=native is left out because the library is built on one
 * machine and timed on another).  The software `half` arithmetic is kept, as the
 * reference's generated code uses include/hidet/runtime/cpu/float16.h:424-444.
 */
#include <stdint.h>
#include <omp.h>

#include "half_sw.h"

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_baseline_threads(void) { return omp_get_max_threads(); }

/* a f16 [m,k], w i8 [k,n], scale f16 [n] -> c f16 [m,n]; rows [row_begin,row_end) only, so a
 * bounded sample of a large problem can be timed. */
ORACLE_API void oracle_baseline_quant_matmul(const uint16_t *a, const int8_t *w, const uint16_t *scale, uint16_t *c,
                                             int64_t m, int64_t k, int64_t n, int64_t col_begin, int64_t col_end) {
    int64_t nc = col_end - col_begin;
#pragma omp parallel for schedule(static)
    for (int64_t o = 0; o < m * nc; ++o) {
        int64_t i = o / nc, j = col_begin + o % nc;
        float sc = half_to_f32(scale[j]);
        uint16_t acc = 0;
        for (int64_t kk = 0; kk < k; ++kk) {
            uint16_t wd = half_from_f32((float)w[kk * n + j] * sc);
            uint16_t pr = half_from_f32(half_to_f32(a[i * k + kk]) * half_to_f32(wd));
            acc = half_from_f32(half_to_f32(acc) + half_to_f32(pr));
        }
        c[i * n + j] = acc;
    }
}
