// Entry point of the group-wise W4A16 matmul: argument checks and the choice of kernel family.
#include "common.h"

namespace qmm {
void skinny_w4a16_launch(const void *a, const void *w, const void *scales, const void *bias, void *c, int64_t m, int64_t k,
                         int64_t n, int64_t lda, int group, int dtype, int parallel_k_parts, void *workspace,
                         int64_t workspace_bytes, hipStream_t stream);
bool gemm_w4a16_supported(const void *a, const void *w, const void *scales, const void *c, int64_t k, int64_t n,
                          int64_t lda, int group);
void gemm_w4a16_launch(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n,
                       int64_t lda, int group, int dtype, void *workspace, int64_t workspace_bytes, hipStream_t stream);
bool skinny_w4a16_nk_supported(const void *a, const void *w, int64_t k, int64_t lda, int64_t ldw, int group);
void skinny_w4a16_nk_launch(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k, int64_t n,
                            int64_t lda, int64_t ldw, int group, int dtype, hipStream_t stream);
}  // namespace qmm

using namespace qmm;

namespace {

// c[i, j] = T(f32(c[i, j]) + f32(bias[j])): the add that follows the MFMA GEMM when a bias is given (the GEMM has stored
// its result rounded to the output type, so this is the second of the two roundings the bandwidth-bound kernels apply
// in their epilogue).
template <int DT>
__global__ __launch_bounds__(256) void add_bias_rows_kernel(uint16_t *__restrict__ c, const uint16_t *__restrict__ bias, int64_t m, int64_t n) {
    const int64_t o = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (o >= m * n) return;
    const float sum = (DT == HIDET_QMM_F16 ? f16_bits_to_f32(c[o]) : bf16_bits_to_f32(c[o])) +
                      (DT == HIDET_QMM_F16 ? f16_bits_to_f32(bias[o % n]) : bf16_bits_to_f32(bias[o % n]));
    c[o] = DT == HIDET_QMM_F16 ? f32_to_f16_bits(sum) : f32_to_bf16_bits(sum);
}

void w4a16_dispatch(const void *a, const void *w, const void *scales, const void *bias, void *c, int64_t m, int64_t k, int64_t n,
                    int64_t lda, int group_size, int dtype, int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                    void *stream_);

}  // namespace

HIDET_API void hidet_symmetric_quant_matmul_w4a16(const void *a, const void *w, const void *scales, void *c, int64_t m,
                                                  int64_t k, int64_t n, int64_t lda, int group_size, int dtype,
                                                  int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                                                  void *stream_) {
    QMM_ENTRY_BEGIN
    w4a16_dispatch(a, w, scales, nullptr, c, m, k, n, lda, group_size, dtype, parallel_k_parts, workspace, workspace_bytes, stream_);
    QMM_ENTRY_END
}

HIDET_API void hidet_symmetric_quant_matmul_w4a16_bias(const void *a, const void *w, const void *scales, const void *bias, void *c,
                                                       int64_t m, int64_t k, int64_t n, int64_t lda, int group_size, int dtype,
                                                       int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                                                       void *stream_) {
    QMM_ENTRY_BEGIN
    QMM_CHECK(bias != nullptr || n == 0, "null bias pointer");
    w4a16_dispatch(a, w, scales, bias, c, m, k, n, lda, group_size, dtype, parallel_k_parts, workspace, workspace_bytes, stream_);
    QMM_ENTRY_END
}

namespace {
void w4a16_dispatch(const void *a, const void *w, const void *scales, const void *bias, void *c, int64_t m, int64_t k, int64_t n,
                    int64_t lda, int group_size, int dtype, int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                    void *stream_) {
    QMM_CHECK(dtype == HIDET_QMM_BF16 || dtype == HIDET_QMM_F16,
              "activations and scales must be bfloat16 or float16, got dtype code " << dtype);
    QMM_CHECK(m >= 0 && k >= 0 && n >= 0, "negative extent: m=" << m << " k=" << k << " n=" << n);
    QMM_CHECK(group_size > 0 && k % group_size == 0,
              "K (" << k << ") must be a multiple of the group size (" << group_size << ")");
    QMM_CHECK(n % 2 == 0, "N (" << n << ") must be even: two codes are packed per byte");
    QMM_CHECK(lda >= k, "row stride of a (" << lda << ") is smaller than K (" << k << ")");
    QMM_CHECK(k < (int64_t(1) << 31) && n < (int64_t(1) << 31) && m < (int64_t(1) << 31), "extent exceeds 2^31");
    QMM_CHECK(parallel_k_parts >= 0, "parallel_k_parts must be >= 0");
    if (m == 0 || n == 0) return;
    QMM_CHECK(a && c && (k == 0 || (w && scales)), "null tensor pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    // one or two 16-row passes of the bandwidth-bound kernel (19 us each at K=4096, N=11008) beat the MFMA GEMM
    // (46 us up to M=128); beyond 32 rows the GEMM wins
    if (m > 32 && k > 0 && gemm_w4a16_supported(a, w, scales, c, k, n, lda, group_size)) {
        gemm_w4a16_launch(a, w, scales, c, m, k, n, lda, group_size, dtype, workspace, workspace_bytes, stream);
        if (bias != nullptr) {
            // a few microseconds next to a GEMM of 35 and more; the decode-sized calls below add the bias in their epilogue
            QMM_CHECK(m * n < (int64_t(1) << 39), "output too large for the bias pass");
            if (dtype == HIDET_QMM_F16)
                launch(add_bias_rows_kernel<HIDET_QMM_F16>, dim3(uint32_t(cdiv(m * n, 256))), dim3(256), 0, stream,
                       static_cast<uint16_t *>(c), static_cast<const uint16_t *>(bias), m, n);
            else
                launch(add_bias_rows_kernel<HIDET_QMM_BF16>, dim3(uint32_t(cdiv(m * n, 256))), dim3(256), 0, stream,
                       static_cast<uint16_t *>(c), static_cast<const uint16_t *>(bias), m, n);
        }
    } else {
        skinny_w4a16_launch(a, w, scales, bias, c, m, k, n, lda, group_size, dtype, parallel_k_parts, workspace, workspace_bytes,
                            stream);
    }
}
}  // namespace

HIDET_API void hidet_symmetric_quant_matmul_w4a16_nk(const void *a, const void *w_nk, const void *scales, void *c, int64_t m,
                                                     int64_t k, int64_t n, int64_t lda, int64_t ldw, int group_size, int dtype,
                                                     void *stream_) {
    QMM_ENTRY_BEGIN
    QMM_CHECK(dtype == HIDET_QMM_BF16 || dtype == HIDET_QMM_F16,
              "activations and scales must be bfloat16 or float16, got dtype code " << dtype);
    QMM_CHECK(m >= 0 && k >= 0 && n >= 0, "negative extent: m=" << m << " k=" << k << " n=" << n);
    QMM_CHECK(group_size > 0 && k % group_size == 0,
              "K (" << k << ") must be a multiple of the group size (" << group_size << ")");
    QMM_CHECK(lda >= k, "row stride of a (" << lda << ") is smaller than K (" << k << ")");
    QMM_CHECK(2 * ldw >= k, "row stride of w_nk (" << ldw << " bytes) is smaller than K / 2 (" << k / 2 << ")");
    QMM_CHECK(k < (int64_t(1) << 31) && n < (int64_t(1) << 31) && m < (int64_t(1) << 31), "extent exceeds 2^31");
    if (m == 0 || n == 0) return;
    QMM_CHECK(a && c && w_nk && scales, "null tensor pointer");
    QMM_CHECK(skinny_w4a16_nk_supported(a, w_nk, k, lda, ldw, group_size),
              "the K-contiguous int4 kernel needs K a multiple of 128, a group size of 128 times a power of two, 16-byte "
              "aligned rows of w_nk and of a: k=" << k << " group=" << group_size << " lda=" << lda << " ldw=" << ldw);
    skinny_w4a16_nk_launch(a, w_nk, scales, c, m, k, n, lda, ldw, group_size, dtype, static_cast<hipStream_t>(stream_));
    QMM_ENTRY_END
}
