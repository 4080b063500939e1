// Entry points of the FP8 matmuls: argument checks and the choice of kernel family.
#include "common.h"

namespace qmm {
bool skinny_fp8_supported(const void *b, int64_t k, int64_t ldb);
void skinny_fp8_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                       int out_dtype, const void *scale_a, const void *scale_b, hipStream_t stream);
void gemm_fp8_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                     int out_dtype, const void *scale_a, const void *scale_b, void *workspace, int64_t workspace_bytes,
                     hipStream_t stream);
void gemm_fp8_scaled_launch(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m,
                            int64_t n, int64_t k, int out_dtype, bool e5m2, void *workspace, int64_t workspace_bytes,
                            hipStream_t stream);
void skinny_fp8_e5m2_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                            int out_dtype, const void *scale_a, const void *scale_b, hipStream_t stream);
void gemm_fp8_e5m2_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                          int out_dtype, const void *scale_a, const void *scale_b, hipStream_t stream);
void skinny_fp8_block_scaled_launch(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m,
                                    int64_t n, int64_t k, int out_dtype, bool e5m2, hipStream_t stream);
}  // namespace qmm

using namespace qmm;

// The workspace is optional here (NULL: tiles are never computed in K ranges); when given it starts with the 64 KiB of
// arrival counters, which are zero between calls.
static void check_workspace(const void *workspace, int64_t workspace_bytes) {
    QMM_CHECK(workspace_bytes >= 0, "negative workspace size");
    QMM_CHECK(workspace == nullptr || aligned(workspace, 16), "the workspace must be 16-byte aligned");
}

static void check_out_dtype(int out_dtype) {
    QMM_CHECK(out_dtype == HIDET_QMM_F32 || out_dtype == HIDET_QMM_F16 || out_dtype == HIDET_QMM_BF16 || out_dtype == HIDET_QMM_E4M3,
              "output dtype must be float32, float16, bfloat16 or float8_e4m3, got code " << out_dtype);
}

HIDET_API void hidet_matmul_f8(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda,
                               int64_t ldb, int out_dtype, const void *scale_a, const void *scale_b, void *workspace,
                               int64_t workspace_bytes, void *stream_) {
    QMM_ENTRY_BEGIN
    check_out_dtype(out_dtype);
    QMM_CHECK(m >= 0 && n >= 0 && k >= 0, "negative extent: m=" << m << " n=" << n << " k=" << k);
    QMM_CHECK(lda >= k && ldb >= k, "row strides (" << lda << ", " << ldb << ") must be at least K (" << k << ")");
    QMM_CHECK(k < (int64_t(1) << 31) && n < (int64_t(1) << 31) && m < (int64_t(1) << 31), "extent exceeds 2^31");
    if (m == 0 || n == 0) return;
    QMM_CHECK(c && (k == 0 || (a && b)), "null tensor pointer");
    check_workspace(workspace, workspace_bytes);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (m <= 16 && skinny_fp8_supported(b, k, ldb))
        skinny_fp8_launch(a, b, c, m, n, k, lda, ldb, out_dtype, scale_a, scale_b, stream);
    else
        gemm_fp8_launch(a, b, c, m, n, k, lda, ldb, out_dtype, scale_a, scale_b, workspace, workspace_bytes, stream);
    QMM_ENTRY_END
}

HIDET_API void hidet_matmul_f8_e5m2(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda,
                                    int64_t ldb, int out_dtype, const void *scale_a, const void *scale_b, void *stream_) {
    QMM_ENTRY_BEGIN
    QMM_CHECK(out_dtype == HIDET_QMM_F32 || out_dtype == HIDET_QMM_F16 || out_dtype == HIDET_QMM_BF16 || out_dtype == HIDET_QMM_E5M2,
              "output dtype must be float32, float16, bfloat16 or float8_e5m2, got code " << out_dtype);
    QMM_CHECK(m >= 0 && n >= 0 && k >= 0, "negative extent: m=" << m << " n=" << n << " k=" << k);
    QMM_CHECK(lda >= k && ldb >= k, "row strides (" << lda << ", " << ldb << ") must be at least K (" << k << ")");
    QMM_CHECK(k < (int64_t(1) << 31) && n < (int64_t(1) << 31) && m < (int64_t(1) << 31), "extent exceeds 2^31");
    if (m == 0 || n == 0) return;
    QMM_CHECK(c && (k == 0 || (a && b)), "null tensor pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (m <= 16 && skinny_fp8_supported(b, k, ldb))
        skinny_fp8_e5m2_launch(a, b, c, m, n, k, lda, ldb, out_dtype, scale_a, scale_b, stream);
    else
        gemm_fp8_e5m2_launch(a, b, c, m, n, k, lda, ldb, out_dtype, scale_a, scale_b, stream);
    QMM_ENTRY_END
}

// Checks and kernel choice of the block-scaled matmul; `e5m2`: both operands float8_e5m2, else float8_e4m3.
static void f8_scaled_dispatch(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m, int64_t n,
                               int64_t k, int out_dtype, bool e5m2, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    if (e5m2)
        QMM_CHECK(out_dtype == HIDET_QMM_F32 || out_dtype == HIDET_QMM_F16 || out_dtype == HIDET_QMM_BF16 || out_dtype == HIDET_QMM_E5M2,
                  "output dtype must be float32, float16, bfloat16 or float8_e5m2, got code " << out_dtype);
    else
        check_out_dtype(out_dtype);
    QMM_CHECK(m >= 0 && n >= 0 && k >= 0, "negative extent: m=" << m << " n=" << n << " k=" << k);
    QMM_CHECK(k % 128 == 0 && n % 128 == 0,
              "block-scaled matmul needs K and N to be multiples of the 128 x 128 scale block, got K=" << k << " N=" << n);
    QMM_CHECK(k < (int64_t(1) << 31) && n < (int64_t(1) << 31) && m < (int64_t(1) << 31), "extent exceeds 2^31");
    if (m == 0 || n == 0) return;
    QMM_CHECK(a && b && c && scale_a && scale_b, "null tensor pointer");
    QMM_CHECK(k > 0, "K must be positive");
    QMM_CHECK(aligned(a, 16) && aligned(b, 16) && aligned(c, 16), "tensors must be 16-byte aligned");
    check_workspace(workspace, workspace_bytes);
    if (m <= 16)  // decode: the bandwidth-bound kernel, one pass over b
        skinny_fp8_block_scaled_launch(a, b, scale_a, scale_b, c, m, n, k, out_dtype, e5m2, stream);
    else
        gemm_fp8_scaled_launch(a, b, scale_a, scale_b, c, m, n, k, out_dtype, e5m2, workspace, workspace_bytes, stream);
}

HIDET_API void hidet_matmul_f8_scaled(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c,
                                      int64_t m, int64_t n, int64_t k, int out_dtype, void *workspace, int64_t workspace_bytes,
                                      void *stream_) {
    QMM_ENTRY_BEGIN
    f8_scaled_dispatch(a, b, scale_a, scale_b, c, m, n, k, out_dtype, false, workspace, workspace_bytes, static_cast<hipStream_t>(stream_));
    QMM_ENTRY_END
}

HIDET_API void hidet_matmul_f8_scaled_e5m2(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c,
                                           int64_t m, int64_t n, int64_t k, int out_dtype, void *workspace,
                                           int64_t workspace_bytes, void *stream_) {
    QMM_ENTRY_BEGIN
    f8_scaled_dispatch(a, b, scale_a, scale_b, c, m, n, k, out_dtype, true, workspace, workspace_bytes, static_cast<hipStream_t>(stream_));
    QMM_ENTRY_END
}
