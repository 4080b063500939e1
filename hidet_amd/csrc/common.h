// Shared host/device helpers for the quantized-matmul library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <exception>
#include <map>
#include <mutex>
#include <set>
#include <sstream>
#include <string>

#include "../../include/hidet_qmm.h"

#define HIDET_API extern "C" __attribute__((visibility("default")))

namespace qmm {

// Thrown inside an entry point, turned into the thread-local last-error string at the boundary.
struct Error : std::exception {
    std::string msg;
    explicit Error(std::string m) : msg(std::move(m)) {}
    const char *what() const noexcept override { return msg.c_str(); }
};

struct Thrower {
    std::ostringstream os;
    Thrower(const char *file, int line) { os << file << ":" << line << ": "; }
    [[noreturn]] void raise() { throw Error(os.str()); }
};

#define QMM_FAIL(...)                         \
    do {                                      \
        ::qmm::Thrower _t(__FILE__, __LINE__); \
        _t.os << __VA_ARGS__;                 \
        _t.raise();                           \
    } while (0)

#define QMM_CHECK(cond, ...)                  \
    do {                                      \
        if (!(cond)) QMM_FAIL(__VA_ARGS__);   \
    } while (0)

#define QMM_HIP(call)                                                                   \
    do {                                                                                \
        hipError_t _e = (call);                                                         \
        if (_e != hipSuccess) QMM_FAIL(#call << " failed: " << hipGetErrorString(_e));  \
    } while (0)

// Body of every extern "C" entry point: nothing may propagate across the C boundary.
#define QMM_ENTRY_BEGIN try {
#define QMM_ENTRY_END                            \
    }                                            \
    catch (const std::exception &e) {            \
        hidet_set_last_error(e.what());          \
        return;                                  \
    }                                            \
    catch (...) {                                \
        hidet_set_last_error("unknown error");   \
        return;                                  \
    }

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline size_t dtype_bytes(int dt) {
    switch (dt) {
        case HIDET_QMM_F32: return 4;
        case HIDET_QMM_F16:
        case HIDET_QMM_BF16:
        case HIDET_QMM_I16: return 2;
        case HIDET_QMM_I8:
        case HIDET_QMM_E4M3: return 1;
        default: QMM_FAIL("unknown dtype code " << dt);
    }
}

// One-shot timing hook: when a (start, stop) event pair is armed on this thread, the next main
// kernel launch records its own begin/end timestamps into them (hipExtLaunchKernelGGL).
struct TimingSlot {
    hipEvent_t start = nullptr, stop = nullptr;
};
TimingSlot &timing_slot();
// true while this thread's last-error string has not been read (it stays set)
bool error_pending();

template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t shmem, hipStream_t stream, Args... args) {
    TimingSlot &ts = timing_slot();
    if (ts.start != nullptr) {
        hipEvent_t s = ts.start, e = ts.stop;
        ts.start = ts.stop = nullptr;
        hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, s, e, 0, static_cast<KArgs>(args)...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, shmem, stream, static_cast<KArgs>(args)...);
    }
    QMM_HIP(hipGetLastError());
}

// A kernel that uses more than 64 KiB of dynamic LDS has to be told so once per device before its first launch there.
inline void allow_dynamic_lds(const void *kernel, int bytes) {
    if (bytes <= 65536) return;
    static std::mutex mu;
    static std::set<std::pair<const void *, int>> done;
    int device = 0;
    QMM_HIP(hipGetDevice(&device));
    std::lock_guard<std::mutex> guard(mu);
    if (done.count({kernel, device})) return;
    QMM_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    done.insert({kernel, device});
}

// Compute units of the current device, read once per device.
inline int device_cus() {
    static std::mutex mu;
    static std::map<int, int> known;
    int device = 0;
    QMM_HIP(hipGetDevice(&device));
    std::lock_guard<std::mutex> guard(mu);
    auto it = known.find(device);
    if (it != known.end()) return it->second;
    int cus = 0;
    QMM_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    known[device] = cus;
    return cus;
}

// Helper kernels (fills, conversions) never consume the timing slot.
template <typename... KArgs, typename... Args>
inline void launch_aux(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t shmem, hipStream_t stream, Args... args) {
    hipLaunchKernelGGL(kernel, grid, block, shmem, stream, static_cast<KArgs>(args)...);
    QMM_HIP(hipGetLastError());
}

// ---- device-side numeric helpers ---------------------------------------------------------------

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int int8v_t __attribute__((ext_vector_type(8)));
typedef int int4v_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint4v_t __attribute__((ext_vector_type(4)));

// A caller-provided workspace has three parts. The first 64 KiB hold arrival counters of cross-workgroup exchanges
// (always returned to zero by the kernel that used them). The mailbox behind them - a quarter of the rest, at most
// 16 MiB - belongs to the split-K exchange of the bandwidth-bound kernels, which finds it all zero and leaves it all
// zero. What follows is plain scratch (partial tiles of the GEMMs, column maxima of the quantizers) whose contents
// nobody relies on between launches.
constexpr int64_t kCounterBytes = 64 << 10;
constexpr int64_t kMaxMailboxBytes = 16 << 20;
// Word of the counter block (in its last 256 bytes, far behind the arrival counters) that a collector of the split-K
// exchange sets when it gives up waiting for a partial tile. It stays set until hidet_qmm_exchange_reset.
constexpr int kExchangeLostWord = 16320;
// Re-reads of the mailbox after which a collector gives up: about a second of polling. Tests lower it from the host to
// drive the give-up path without a kernel that waits for long.
constexpr int kExchangeSpinLimit = 1 << 20;
inline std::atomic<int> &exchange_spin_limit() {
    static std::atomic<int> limit{kExchangeSpinLimit};
    return limit;
}

struct Workspace {
    uint32_t *counters = nullptr;
    float *mailbox = nullptr;
    int64_t mailbox_bytes = 0;
    char *scratch = nullptr;
    int64_t scratch_bytes = 0;
};

inline Workspace split_workspace(void *workspace, int64_t bytes) {
    Workspace v;
    if (workspace == nullptr || bytes < kCounterBytes) return v;
    const int64_t rest = bytes - kCounterBytes;
    v.counters = static_cast<uint32_t *>(workspace);
    v.mailbox_bytes = std::min(kMaxMailboxBytes, rest / 4) / 256 * 256;
    v.mailbox = reinterpret_cast<float *>(static_cast<char *>(workspace) + kCounterBytes);
    v.scratch = static_cast<char *>(workspace) + kCounterBytes + v.mailbox_bytes;
    v.scratch_bytes = rest - v.mailbox_bytes;
    return v;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

// float32 -> bfloat16 bits, round to nearest even (NaN kept quiet)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    _Float16 h = static_cast<_Float16>(f);  // v_cvt_f16_f32: round to nearest even
    return __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) { return static_cast<float>(__builtin_bit_cast(_Float16, b)); }

// The float16 output of the int8 matmul with the optional bias of its epilogue: the product is rounded to float16 and the
// bias is added to that value with a second rounding - what the reference's fused epilogue computes, which applies the add
// to the value the template stores (python/hidet/graph/ops/quant/matmul_f16_i8.py:95-99) - so a fused call and the
// matmul followed by an add give the same bits. `bias` of a call without one is -0.0f, which changes nothing (not even
// the sign of a zero).
__device__ __forceinline__ _Float16 scaled_biased_f16(float acc, float scale, float bias) {
    const _Float16 product = _Float16(acc * scale);
    return _Float16(float(product) + bias);
}
// The bfloat16 form (bits): the matmul's bfloat16 result, then the add rounded to bfloat16 again.
__device__ __forceinline__ uint16_t biased_bf16_bits(float acc, float bias) {
    return f32_to_bf16_bits(bf16_bits_to_f32(f32_to_bf16_bits(acc)) + bias);
}

}  // namespace qmm
