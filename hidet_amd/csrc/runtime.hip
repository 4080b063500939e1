// Error state, library facts and the timing hook of libhidet_qmm.so.
#include "common.h"

namespace {
struct ErrorState {
    bool has_error = false;
    std::string msg;
};
ErrorState &error_state() {
    static thread_local ErrorState s;
    return s;
}
}  // namespace

namespace qmm {
TimingSlot &timing_slot() {
    static thread_local TimingSlot s;
    return s;
}
}  // namespace qmm

// Thread-local, read-once error string: the convention of src/hidet/runtime/logging.cpp:14-36.
HIDET_API void hidet_set_last_error(const char *msg) {
    ErrorState &s = error_state();
    if (s.has_error) fprintf(stderr, "Warning: hidet error state has been overridden: %s\n", s.msg.c_str());
    s.has_error = true;
    s.msg = msg ? msg : "";
}

HIDET_API const char *hidet_get_last_error(void) {
    ErrorState &s = error_state();
    if (!s.has_error) return nullptr;
    s.has_error = false;
    return s.msg.c_str();
}

HIDET_API int hidet_qmm_abi_version(void) { return HIDET_QMM_ABI_VERSION; }
HIDET_API const char *hidet_qmm_arch(void) { return "gfx950"; }
HIDET_API int64_t hidet_qmm_min_workspace_bytes(void) { return int64_t(96) << 20; }

HIDET_API void *hidet_qmm_event_create(void) {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) {
        hidet_set_last_error("hipEventCreate failed");
        return nullptr;
    }
    return e;
}

HIDET_API void hidet_qmm_event_destroy(void *event) {
    if (event) (void)hipEventDestroy(static_cast<hipEvent_t>(event));
}

HIDET_API void hidet_qmm_event_record(void *event, void *stream) {
    QMM_ENTRY_BEGIN
    QMM_HIP(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
    QMM_ENTRY_END
}

HIDET_API void hidet_qmm_event_synchronize(void *event) {
    QMM_ENTRY_BEGIN
    QMM_HIP(hipEventSynchronize(static_cast<hipEvent_t>(event)));
    QMM_ENTRY_END
}

HIDET_API float hidet_qmm_event_elapsed_ms(void *start, void *stop) {
    float ms = -1.0f;
    hipError_t e = hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop));
    if (e != hipSuccess) {
        hidet_set_last_error(hipGetErrorString(e));
        return -1.0f;
    }
    return ms;
}

HIDET_API void hidet_qmm_arm_timing(void *start_event, void *stop_event) {
    qmm::TimingSlot &ts = qmm::timing_slot();
    ts.start = static_cast<hipEvent_t>(start_event);
    ts.stop = static_cast<hipEvent_t>(stop_event);
}

// ---- measurement: what a kernel that only reads can get out of the memory system -----------------------------------
namespace {
constexpr int kProbeBlockBytes = 32768;  // 256 threads x 8 loads x 16 bytes, contiguous per workgroup

__global__ __launch_bounds__(256) void read_probe_kernel(const uint4 *__restrict__ src, uint32_t *__restrict__ sink) {
    const uint4 *p = src + int64_t(blockIdx.x) * (kProbeBlockBytes / 16) + threadIdx.x;
    uint4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = p[j * 256];
    uint32_t acc = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc += v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
    if (acc == 0x9E3779B9u) sink[0] = acc;  // practically never true; keeps the loads alive
}
}  // namespace

HIDET_API void hidet_qmm_read_probe(const void *src, int64_t bytes, void *sink, void *stream) {
    QMM_ENTRY_BEGIN
    QMM_CHECK(src && sink && qmm::aligned(src, 16), "null or misaligned pointer");
    QMM_CHECK(bytes > 0 && bytes % kProbeBlockBytes == 0 && bytes / kProbeBlockBytes < (int64_t(1) << 31),
              "the size must be a positive multiple of " << kProbeBlockBytes << " bytes, got " << bytes);
    qmm::launch(read_probe_kernel, dim3(uint32_t(bytes / kProbeBlockBytes)), dim3(256), 0, static_cast<hipStream_t>(stream),
                static_cast<const uint4 *>(src), static_cast<uint32_t *>(sink));
    QMM_ENTRY_END
}
