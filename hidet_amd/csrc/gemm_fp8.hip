// FP8 e4m3 GEMM: c[m, n] = cast(alpha * sum_k a[m, k] * b[n, k]), both operands K-contiguous, fp32
// accumulation on the CDNA4 block-scaled MFMA (v_mfma_scale_f32_16x16x128_f8f6f4 with unit block
// scales, the form that runs fp8 at twice the rate of the plain fp8 MFMA).  alpha = scale_a * scale_b
// (per-tensor float32 scales read from device memory) or 1.
//
// Workgroup tile 256 x 256, four waves of 128 x 128, k-step 128 bytes.  Both operand tiles are staged
// through LDS as rows of 128 bytes = eight 16-byte chunks, XOR-swizzled by row so that the 32-byte
// fragment reads of 16 consecutive rows spread over all banks; two buffers, one barrier per k-step,
// the next step's global loads in flight during the 64 MFMAs of the current one.  The MFMA is issued
// with the b tile as its row operand: a lane then holds 4 consecutive output columns of one row and
// stores them together.
#include "common.h"
#include "numeric.h"

namespace qmm {
namespace {

constexpr int kBM = 256, kBN = 256, kBKB = 128;  // tile and k-step in bytes (= fp8 elements)
constexpr int kThreads = 256;
constexpr int kStageChunks = (kBM + kBN) * 8;      // 16-byte chunks per stage (A rows then B rows)
constexpr int kChunksPerThread = kStageChunks / kThreads;  // 16
constexpr int kLdsBytes = 2 * kStageChunks * 16;   // 128 KiB

__device__ __forceinline__ float4_t mfma_fp8_k128(const uint4 &r0, const uint4 &r1, const uint4 &c0, const uint4 &c1, float4_t acc) {
    int8v_t rv, cv;
    rv[0] = int(r0.x); rv[1] = int(r0.y); rv[2] = int(r0.z); rv[3] = int(r0.w);
    rv[4] = int(r1.x); rv[5] = int(r1.y); rv[6] = int(r1.z); rv[7] = int(r1.w);
    cv[0] = int(c0.x); cv[1] = int(c0.y); cv[2] = int(c0.z); cv[3] = int(c0.w);
    cv[4] = int(c1.x); cv[5] = int(c1.y); cv[6] = int(c1.z); cv[7] = int(c1.w);
    // formats 0/0 = e4m3 x e4m3; block scales 0x7F = 2^0
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rv, cv, acc, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
}

template <int OUT>
__device__ __forceinline__ void store4(void *c, int64_t idx, float4_t v) {
    if (OUT == HIDET_QMM_F32) {
        *reinterpret_cast<float4_t *>(static_cast<float *>(c) + idx) = v;
    } else if (OUT == HIDET_QMM_BF16) {
        uint2 o;
        o.x = uint32_t(f32_to_bf16_bits(v[0])) | (uint32_t(f32_to_bf16_bits(v[1])) << 16);
        o.y = uint32_t(f32_to_bf16_bits(v[2])) | (uint32_t(f32_to_bf16_bits(v[3])) << 16);
        *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(c) + idx) = o;
    } else if (OUT == HIDET_QMM_F16) {
        uint2 o;
        o.x = uint32_t(f32_to_f16_bits(v[0])) | (uint32_t(f32_to_f16_bits(v[1])) << 16);
        o.y = uint32_t(f32_to_f16_bits(v[2])) | (uint32_t(f32_to_f16_bits(v[3])) << 16);
        *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(c) + idx) = o;
    } else {
        const uint32_t o = uint32_t(f32_to_e4m3(v[0])) | (uint32_t(f32_to_e4m3(v[1])) << 8) |
                           (uint32_t(f32_to_e4m3(v[2])) << 16) | (uint32_t(f32_to_e4m3(v[3])) << 24);
        *reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(c) + idx) = o;
    }
}

template <int OUT>
__global__ __launch_bounds__(kThreads, 1) void gemm_fp8_kernel(const uint8_t *__restrict__ a, int64_t lda,
                                                               const uint8_t *__restrict__ b, int64_t ldb,
                                                               void *__restrict__ c, int m, int n, int k,
                                                               const float *__restrict__ scale_a,
                                                               const float *__restrict__ scale_b, int tiles_m, int tiles_n) {
    extern __shared__ uint4 lds[];  // [2][kStageChunks]

    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int cb_begin = (tiles_n * xcd) / 8, cb_end = (tiles_n * (xcd + 1)) / 8;
    if (local >= (cb_end - cb_begin) * tiles_m) return;
    const int m0 = (local % tiles_m) * kBM;
    const int n0 = (cb_begin + local / tiles_m) * kBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int kg = lane >> 4, ls = lane & 15;

    float4_t acc[8][8];  // [row block of a][column block of b]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    // staging: chunk id = j * 256 + tid -> tile row id / 8 (A rows 0..255, then B rows 256..511),
    // LDS position id % 8 holds the row's chunk (position ^ (row & 7))
    uint4 stage[kChunksPerThread];
    auto load_stage = [&](int kbase) {
#pragma unroll
        for (int j = 0; j < kChunksPerThread; ++j) {
            const int id = j * kThreads + tid;
            const int row = id >> 3, pos = id & 7;
            const int chunk = pos ^ (row & 7);
            const int kb = kbase + chunk * 16;
            stage[j] = uint4{0u, 0u, 0u, 0u};
            if (j < kChunksPerThread / 2) {
                const int r = m0 + row;
                if (r < m && kb < k) stage[j] = *reinterpret_cast<const uint4 *>(a + int64_t(r) * lda + kb);
            } else {
                const int r = n0 + row - kBM;
                if (r < n && kb < k) stage[j] = *reinterpret_cast<const uint4 *>(b + int64_t(r) * ldb + kb);
            }
        }
    };
    auto store_stage = [&](int buf) {
#pragma unroll
        for (int j = 0; j < kChunksPerThread; ++j) lds[buf * kStageChunks + j * kThreads + tid] = stage[j];
    };

    load_stage(0);
    store_stage(0);
    __syncthreads();

    const int steps = (k + kBKB - 1) / kBKB;
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        const bool more = s + 1 < steps;
        if (more) load_stage((s + 1) * kBKB);
        const uint4 *la = lds + buf * kStageChunks;
        const uint4 *lb = la + kBM * 8;
        uint4 bf[8][2];  // the 8 column-block fragments of b
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int r = wn * 128 + j * 16 + ls;
            bf[j][0] = lb[r * 8 + ((2 * kg) ^ (r & 7))];
            bf[j][1] = lb[r * 8 + ((2 * kg + 1) ^ (r & 7))];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = wm * 128 + i * 16 + ls;
            const uint4 a0 = la[r * 8 + ((2 * kg) ^ (r & 7))];
            const uint4 a1 = la[r * 8 + ((2 * kg + 1) ^ (r & 7))];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[i][j] = mfma_fp8_k128(bf[j][0], bf[j][1], a0, a1, acc[i][j]);
        }
        if (more) store_stage(buf ^ 1);
        __syncthreads();
    }

    // acc[i][j][v] = c[m0 + wm*128 + i*16 + ls][n0 + wn*128 + j*16 + 4*kg + v]
    float alpha = 1.0f;
    if (scale_a != nullptr) alpha *= *scale_a;
    if (scale_b != nullptr) alpha *= *scale_b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = m0 + wm * 128 + i * 16 + ls;
        if (row < m) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int col = n0 + wn * 128 + j * 16 + 4 * kg;
                if (col < n) {  // n % 4 == 0
                    float4_t v = acc[i][j];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] *= alpha;
                    store4<OUT>(c, int64_t(row) * n + col, v);
                }
            }
        }
    }
}

// Fallback for shapes the tiled kernel cannot take: one thread per output element.
template <int OUT>
__global__ __launch_bounds__(256) void naive_fp8_kernel(const uint8_t *__restrict__ a, int64_t lda, const uint8_t *__restrict__ b,
                                                        int64_t ldb, void *__restrict__ c, int64_t m, int64_t n, int64_t k,
                                                        const float *__restrict__ scale_a, const float *__restrict__ scale_b) {
    const int64_t o = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (o >= m * n) return;
    const int64_t i = o / n, j = o - i * n;
    float acc = 0.f;
    for (int64_t kk = 0; kk < k; ++kk) acc += e4m3_to_f32(a[i * lda + kk]) * e4m3_to_f32(b[j * ldb + kk]);
    if (scale_a != nullptr) acc *= (*scale_a) * (scale_b != nullptr ? *scale_b : 1.0f);
    else if (scale_b != nullptr) acc *= *scale_b;
    if (OUT == HIDET_QMM_F32) static_cast<float *>(c)[o] = acc;
    else if (OUT == HIDET_QMM_BF16) static_cast<uint16_t *>(c)[o] = f32_to_bf16_bits(acc);
    else if (OUT == HIDET_QMM_F16) static_cast<uint16_t *>(c)[o] = f32_to_f16_bits(acc);
    else static_cast<uint8_t *>(c)[o] = f32_to_e4m3(acc);
}

template <typename F>
void dispatch_out(int out_dtype, F &&f) {
    switch (out_dtype) {
        case HIDET_QMM_F32: f(std::integral_constant<int, HIDET_QMM_F32>()); break;
        case HIDET_QMM_F16: f(std::integral_constant<int, HIDET_QMM_F16>()); break;
        case HIDET_QMM_BF16: f(std::integral_constant<int, HIDET_QMM_BF16>()); break;
        case HIDET_QMM_E4M3: f(std::integral_constant<int, HIDET_QMM_E4M3>()); break;
        default: QMM_FAIL("unsupported output dtype code " << out_dtype);
    }
}

}  // namespace

void gemm_fp8_launch(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                     int out_dtype, const void *scale_a, const void *scale_b, hipStream_t stream) {
    const uint8_t *ap = static_cast<const uint8_t *>(a), *bp = static_cast<const uint8_t *>(b);
    const float *sa = static_cast<const float *>(scale_a), *sb = static_cast<const float *>(scale_b);
    const bool tiled = (k % 16 == 0) && (lda % 16 == 0) && (ldb % 16 == 0) && (n % 4 == 0) && aligned(a, 16) &&
                       aligned(b, 16) && aligned(c, 16) && k > 0;
    dispatch_out(out_dtype, [&](auto o) {
        constexpr int OUT = decltype(o)::value;
        if (!tiled) {
            launch(naive_fp8_kernel<OUT>, dim3(cdiv(m * n, 256)), dim3(256), 0, stream, ap, lda, bp, ldb, c, m, n, k, sa, sb);
            return;
        }
        const int tiles_m = int(cdiv(m, kBM)), tiles_n = int(cdiv(n, kBN));
        const int64_t grid = int64_t(8) * cdiv(tiles_n, 8) * tiles_m;
        QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
        static bool attr_set = false;  // one flag per output type (the lambda is instantiated per type)
        if (!attr_set) {
            QMM_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_fp8_kernel<OUT>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));
            attr_set = true;
        }
        launch(gemm_fp8_kernel<OUT>, dim3(uint32_t(grid)), dim3(kThreads), size_t(kLdsBytes), stream, ap, lda, bp, ldb, c,
               int(m), int(n), int(k), sa, sb, tiles_m, tiles_n);
    });
}

}  // namespace qmm
