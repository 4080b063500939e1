// Error state and library facts of libhidet_qmm.so.
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
bool error_pending() { return error_state().has_error; }
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
HIDET_API int64_t hidet_qmm_workspace_bytes_for_scratch(int64_t scratch_bytes) {
    if (scratch_bytes < 0) scratch_bytes = 0;
    const auto scratch_of = [](int64_t bytes) { return qmm::split_workspace(reinterpret_cast<void *>(uintptr_t(256)), bytes).scratch_bytes; };
    // the mailbox takes a quarter of what follows the counters, 16 MiB at most, rounded down to a multiple of 256: a
    // third on top of the scratch bytes is enough, and the rounding can only leave a few bytes to give back
    int64_t bytes = qmm::kCounterBytes + std::min(scratch_bytes + qmm::kMaxMailboxBytes, (scratch_bytes * 4 + 2) / 3);
    while (scratch_of(bytes) < scratch_bytes) ++bytes;
    while (bytes > qmm::kCounterBytes && scratch_of(bytes - 1) >= scratch_bytes) --bytes;
    return bytes;
}
