// Entry point of the W8A16 matmul: argument checks and the choice of kernel family.
#include "common.h"

namespace qmm {
void skinny_w8a16_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                         int64_t n, int64_t lda, int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                         bool strict_workspace, hipStream_t stream);
bool gemm_w8a16_supported(const void *a, const void *w, const void *c, int64_t m, int64_t k, int64_t n, int64_t lda);
void gemm_w8a16_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                       int64_t n, int64_t lda, void *workspace, int64_t workspace_bytes, hipStream_t stream);
bool skinny_w8a16_nk_supported(const void *w, int64_t k, int64_t ldw);
void skinny_w8a16_nk_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                            int64_t n, int64_t lda, int64_t ldw, hipStream_t stream);
bool gemm_w8a16_nk_supported(const void *a, const void *w, const void *c, int64_t m, int64_t k, int64_t n, int64_t lda,
                             int64_t ldw);
void gemm_w8a16_nk_launch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                          int64_t n, int64_t lda, int64_t ldw, void *workspace, int64_t workspace_bytes, hipStream_t stream);
}

using namespace qmm;

namespace {

// Checks and kernel choice shared by the two row-major entry points. `strict_workspace`: a bandwidth-bound launch whose
// K split does not fit the scratch memory is an error instead of a launch with fewer K slices.
void w8a16_dispatch(const void *a, const void *w, const void *scale, const void *bias, void *c, int64_t m, int64_t k, int64_t n,
                    int64_t lda, int parallel_k_parts, void *workspace, int64_t workspace_bytes, bool strict_workspace,
                    hipStream_t stream) {
    QMM_CHECK(m >= 0 && k >= 0 && n >= 0, "negative extent: m=" << m << " k=" << k << " n=" << n);
    QMM_CHECK(lda >= k, "row stride of a (" << lda << ") is smaller than K (" << k << ")");
    QMM_CHECK(k < (int64_t(1) << 31) && n < (int64_t(1) << 31) && m < (int64_t(1) << 31), "extent exceeds 2^31");
    QMM_CHECK(parallel_k_parts >= 0, "parallel_k_parts must be >= 0");
    if (m == 0 || n == 0) return;
    QMM_CHECK(a && w && scale && c, "null tensor pointer");
    QMM_CHECK(aligned(a, 2) && aligned(scale, 2) && aligned(c, 2) && aligned(bias, 2), "float16 tensors must be 2-byte aligned");
    // Up to 16 rows one pass of the bandwidth-bound kernel serves; beyond that every 16 rows would cost another pass
    // over the weights, and the MFMA GEMM with its K split and its empty row blocks left out takes over (K=4096, N=11008,
    // weights from HBM: 17 us at M=17..32, 20 us at M=64, 29 us at M=128). For 9 to 16 rows the bandwidth-bound kernel is
    // ahead of the GEMM on every shape measured (4096 x 11008: 13.5 - 14.1 against 16.5 us; 8192 x 8192: 16.9 - 18.2
    // against 22.4; 8192 x 28672: 42.6 - 43.8 against 49).
    if (m > 16 && k > 0 && gemm_w8a16_supported(a, w, c, m, k, n, lda))
        gemm_w8a16_launch(a, w, scale, bias, c, m, k, n, lda, workspace, workspace_bytes, stream);
    else
        skinny_w8a16_launch(a, w, scale, bias, c, m, k, n, lda, parallel_k_parts, workspace, workspace_bytes, strict_workspace,
                            stream);
}

// Checks and kernel choice shared by the two entry points for K-contiguous weights.
void w8a16_nk_dispatch(const void *a, const void *w_nk, const void *scale, const void *bias, void *c, int64_t m, int64_t k,
                       int64_t n, int64_t lda, int64_t ldw, void *workspace, int64_t workspace_bytes, hipStream_t stream) {
    QMM_CHECK(m >= 0 && k >= 0 && n >= 0, "negative extent: m=" << m << " k=" << k << " n=" << n);
    QMM_CHECK(lda >= k && ldw >= k, "row strides (" << lda << ", " << ldw << ") must be at least K (" << k << ")");
    QMM_CHECK(k < (int64_t(1) << 31) && n < (int64_t(1) << 31) && m < (int64_t(1) << 31), "extent exceeds 2^31");
    QMM_CHECK(workspace_bytes >= 0 && (workspace == nullptr || aligned(workspace, 16)),
              "the workspace must be 16-byte aligned (or NULL: no tile is computed in K ranges)");
    if (m == 0 || n == 0) return;
    QMM_CHECK(a && w_nk && scale && c, "null tensor pointer");
    QMM_CHECK(aligned(a, 2) && aligned(scale, 2) && aligned(c, 2) && aligned(bias, 2), "float16 tensors must be 2-byte aligned");
    QMM_CHECK(skinny_w8a16_nk_supported(w_nk, k, ldw),
              "K-contiguous weights need K and the row stride to be multiples of 16 and a 16-byte aligned pointer, got K=" << k
                                                                                                                         << " ldw=" << ldw);
    // more than one pass of 16 rows: the MFMA GEMM reading the same layout, where its conditions hold
    if (m > 16 && gemm_w8a16_nk_supported(a, w_nk, c, m, k, n, lda, ldw))
        gemm_w8a16_nk_launch(a, w_nk, scale, bias, c, m, k, n, lda, ldw, workspace ? workspace : nullptr,
                             workspace ? workspace_bytes : 0, stream);
    else
        skinny_w8a16_nk_launch(a, w_nk, scale, bias, c, m, k, n, lda, ldw, stream);
}

// Scratch memory of hidet_symmetric_quant_matmul_f16_i8_static, used exactly like a caller's workspace of that size
// (counters, mailbox, scratch). One copy per GPU, loaded with the library's code object (zero-filled then; the kernels
// return every counter and every mailbox word they used to zero).
constexpr int64_t kStaticScratchBytes = HIDET_QMM_STATIC_SCRATCH_BYTES;
static_assert(kStaticScratchBytes > kCounterBytes && kStaticScratchBytes % 256 == 0, "counters plus partial tiles");
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, looked up on the first call there
std::mutex g_scratch_mu;

// The device address of this GPU's copy of `scratch`. In host code the array's name is only a handle for the runtime's
// symbol lookup, never a pointer a kernel may be given.
void *static_scratch_of_current_device() {
    int device = -1;
    QMM_HIP(hipGetDevice(&device));
    QMM_CHECK(device >= 0 && device < kMaxDevices, "device ordinal " << device << " out of range");
    std::lock_guard<std::mutex> guard(g_scratch_mu);
    if (g_scratch_ptr[device] == nullptr) {
        void *ptr = nullptr;
        QMM_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        QMM_CHECK(ptr != nullptr && aligned(ptr, 256), "the runtime returned no usable address for the static scratch array");
        g_scratch_ptr[device] = ptr;
    }
    return g_scratch_ptr[device];
}

}  // namespace

HIDET_API void hidet_symmetric_quant_matmul_f16_i8(const void *a, const void *w, const void *scale, void *c, int64_t m,
                                                   int64_t k, int64_t n, int64_t lda, int parallel_k_parts,
                                                   void *workspace, int64_t workspace_bytes, void *stream_) {
    QMM_ENTRY_BEGIN
    w8a16_dispatch(a, w, scale, nullptr, c, m, k, n, lda, parallel_k_parts, workspace, workspace_bytes, false,
                   static_cast<hipStream_t>(stream_));
    QMM_ENTRY_END
}

HIDET_API int64_t hidet_qmm_static_scratch_bytes(void) { return kStaticScratchBytes; }

namespace {
__global__ __launch_bounds__(256) void zero_fill_kernel(uint4 *__restrict__ dst, int64_t count) {
    for (int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x; i < count; i += int64_t(gridDim.x) * 256) dst[i] = uint4{0u, 0u, 0u, 0u};
}
}  // namespace

HIDET_API int hidet_qmm_exchange_status(const void *workspace, int64_t workspace_bytes, void *stream_) {
    try {
        const void *base = workspace;
        if (base == nullptr) {
            base = static_scratch_of_current_device();
            workspace_bytes = kStaticScratchBytes;
        }
        hipStream_t stream = static_cast<hipStream_t>(stream_);
        uint32_t word = 0;
        if (workspace_bytes >= kCounterBytes)  // else: no counter block, no exchange ever ran on it
            QMM_HIP(hipMemcpyAsync(&word, static_cast<const uint32_t *>(base) + kExchangeLostWord, sizeof(word), hipMemcpyDeviceToHost, stream));
        QMM_HIP(hipStreamSynchronize(stream));
        return word != 0u ? 1 : 0;
    } catch (const std::exception &e) {
        hidet_set_last_error(e.what());
    } catch (...) {
        hidet_set_last_error("unknown error");
    }
    return -1;
}

HIDET_API void hidet_qmm_exchange_reset(void *workspace, int64_t workspace_bytes, void *stream_) {
    QMM_ENTRY_BEGIN
    if (workspace == nullptr) {
        workspace = static_scratch_of_current_device();
        workspace_bytes = kStaticScratchBytes;
    }
    QMM_CHECK(aligned(workspace, 16), "the workspace must be 16-byte aligned");
    const Workspace ws = split_workspace(workspace, workspace_bytes);
    if (ws.counters == nullptr) return;
    // a fill kernel, not a memset node: callers may capture this into a graph
    const int64_t count = (kCounterBytes + ws.mailbox_bytes) / 16;
    launch_aux(zero_fill_kernel, dim3(uint32_t(std::min<int64_t>(2048, cdiv(count, 256)))), dim3(256), 0, static_cast<hipStream_t>(stream_),
               static_cast<uint4 *>(workspace), count);
    QMM_ENTRY_END
}

HIDET_API void hidet_symmetric_quant_matmul_f16_i8_static(const void *a, const void *w, const void *scale, void *c, int64_t m,
                                                          int64_t k, int64_t n, int64_t lda, int parallel_k_parts,
                                                          void *stream_) {
    QMM_ENTRY_BEGIN
    void *ptr = static_scratch_of_current_device();
    w8a16_dispatch(a, w, scale, nullptr, c, m, k, n, lda, parallel_k_parts, ptr, kStaticScratchBytes, true,
                   static_cast<hipStream_t>(stream_));
    QMM_ENTRY_END
}

HIDET_API void hidet_symmetric_quant_matmul_f16_i8_bias(const void *a, const void *w, const void *scale, const void *bias,
                                                        void *c, int64_t m, int64_t k, int64_t n, int64_t lda,
                                                        int parallel_k_parts, void *workspace, int64_t workspace_bytes,
                                                        void *stream_) {
    QMM_ENTRY_BEGIN
    w8a16_dispatch(a, w, scale, bias, c, m, k, n, lda, parallel_k_parts, workspace, workspace_bytes, false,
                   static_cast<hipStream_t>(stream_));
    QMM_ENTRY_END
}

HIDET_API void hidet_symmetric_quant_matmul_f16_i8_nk(const void *a, const void *w_nk, const void *scale, void *c, int64_t m,
                                                      int64_t k, int64_t n, int64_t lda, int64_t ldw, void *workspace,
                                                      int64_t workspace_bytes, void *stream_) {
    QMM_ENTRY_BEGIN
    w8a16_nk_dispatch(a, w_nk, scale, nullptr, c, m, k, n, lda, ldw, workspace, workspace_bytes, static_cast<hipStream_t>(stream_));
    QMM_ENTRY_END
}

HIDET_API void hidet_symmetric_quant_matmul_f16_i8_nk_bias(const void *a, const void *w_nk, const void *scale, const void *bias,
                                                           void *c, int64_t m, int64_t k, int64_t n, int64_t lda, int64_t ldw,
                                                           void *workspace, int64_t workspace_bytes, void *stream_) {
    QMM_ENTRY_BEGIN
    w8a16_nk_dispatch(a, w_nk, scale, bias, c, m, k, n, lda, ldw, workspace, workspace_bytes, static_cast<hipStream_t>(stream_));
    QMM_ENTRY_END
}
