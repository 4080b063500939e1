// Block-scaled FP8 e4m3 GEMM (DeepSeek-style): for every K block of 128
//   c[m, n] += (sum_{k in block} a[m, k] * b[n, k]) * scale_a[kb, m] * scale_b[n / 128, kb]
// with scale_a float32 [K/128, M] (M contiguous) and scale_b float32 [N/128, K/128].
//
// Workgroup tile 128 x 128 (one scale_b entry per k block), four waves of 64 x 64, k-step 128 bytes
// through swizzled double-buffered LDS as in the per-tensor kernel.  Each k block is multiplied into a
// scratch accumulator (one 16x16x128 MFMA per 16 x 16 block) and folded into the running sum with its
// two scales on the vector ALU.
#include "common.h"
#include "numeric.h"

namespace qmm {
namespace {

constexpr int kT = 128;  // tile rows, tile columns and k-step bytes
constexpr int kThreads = 256;
constexpr int kStageChunks = 2 * kT * 8;
constexpr int kChunksPerThread = kStageChunks / kThreads;  // 8
constexpr int kLdsBytes = 2 * kStageChunks * 16;           // 64 KiB

template <int OUT>
__global__ __launch_bounds__(kThreads, 1) void gemm_fp8_scaled_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                                      const float *__restrict__ scale_a,
                                                                      const float *__restrict__ scale_b, void *__restrict__ c,
                                                                      int m, int n, int k, int tiles_m) {
    extern __shared__ uint4 lds[];
    const int m0 = (blockIdx.x % tiles_m) * kT;
    const int nb = blockIdx.x / tiles_m;
    const int n0 = nb * kT;
    const int kblocks = k / 128;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int kg = lane >> 4, ls = lane & 15;

    float4_t total[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) total[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    uint4 stage[kChunksPerThread];
    auto load_stage = [&](int kbase) {
#pragma unroll
        for (int j = 0; j < kChunksPerThread; ++j) {
            const int id = j * kThreads + tid;
            const int row = id >> 3, pos = id & 7;
            const int kb = kbase + (pos ^ (row & 7)) * 16;
            stage[j] = uint4{0u, 0u, 0u, 0u};
            if (j < kChunksPerThread / 2) {
                if (m0 + row < m) stage[j] = *reinterpret_cast<const uint4 *>(a + int64_t(m0 + row) * k + kb);
            } else {
                if (n0 + row - kT < n) stage[j] = *reinterpret_cast<const uint4 *>(b + int64_t(n0 + row - kT) * k + kb);
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

    for (int s = 0; s < kblocks; ++s) {
        const int buf = s & 1;
        const bool more = s + 1 < kblocks;
        if (more) load_stage((s + 1) * 128);
        // scale of this k block for the lane's 4 rows (one per row block) and the tile's column block
        const float sb = scale_b[int64_t(nb) * kblocks + s];
        float f[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = m0 + wm * 64 + i * 16 + ls;
            f[i] = row < m ? scale_a[int64_t(s) * m + row] * sb : 0.f;
        }
        const uint4 *la = lds + buf * kStageChunks;
        const uint4 *lb = la + kT * 8;
        uint4 bf[4][2];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = wn * 64 + j * 16 + ls;
            bf[j][0] = lb[r * 8 + ((2 * kg) ^ (r & 7))];
            bf[j][1] = lb[r * 8 + ((2 * kg + 1) ^ (r & 7))];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = wm * 64 + i * 16 + ls;
            const uint4 a0 = la[r * 8 + ((2 * kg) ^ (r & 7))];
            const uint4 a1 = la[r * 8 + ((2 * kg + 1) ^ (r & 7))];
            int8v_t cv;
            cv[0] = int(a0.x); cv[1] = int(a0.y); cv[2] = int(a0.z); cv[3] = int(a0.w);
            cv[4] = int(a1.x); cv[5] = int(a1.y); cv[6] = int(a1.z); cv[7] = int(a1.w);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int8v_t rv;
                rv[0] = int(bf[j][0].x); rv[1] = int(bf[j][0].y); rv[2] = int(bf[j][0].z); rv[3] = int(bf[j][0].w);
                rv[4] = int(bf[j][1].x); rv[5] = int(bf[j][1].y); rv[6] = int(bf[j][1].z); rv[7] = int(bf[j][1].w);
                const float4_t part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    rv, cv, float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
#pragma unroll
                for (int v = 0; v < 4; ++v) total[i][j][v] += part[v] * f[i];
            }
        }
        if (more) store_stage(buf ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = m0 + wm * 64 + i * 16 + ls;
        if (row >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + wn * 64 + j * 16 + 4 * kg;
            if (col >= n) continue;
            const int64_t o = int64_t(row) * n + col;
            const float4_t v = total[i][j];
            if (OUT == HIDET_QMM_F32) {
                *reinterpret_cast<float4_t *>(static_cast<float *>(c) + o) = v;
            } else if (OUT == HIDET_QMM_BF16) {
                uint2 w2;
                w2.x = uint32_t(f32_to_bf16_bits(v[0])) | (uint32_t(f32_to_bf16_bits(v[1])) << 16);
                w2.y = uint32_t(f32_to_bf16_bits(v[2])) | (uint32_t(f32_to_bf16_bits(v[3])) << 16);
                *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(c) + o) = w2;
            } else if (OUT == HIDET_QMM_F16) {
                uint2 w2;
                w2.x = uint32_t(f32_to_f16_bits(v[0])) | (uint32_t(f32_to_f16_bits(v[1])) << 16);
                w2.y = uint32_t(f32_to_f16_bits(v[2])) | (uint32_t(f32_to_f16_bits(v[3])) << 16);
                *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(c) + o) = w2;
            } else {
                *reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(c) + o) =
                    uint32_t(f32_to_e4m3(v[0])) | (uint32_t(f32_to_e4m3(v[1])) << 8) | (uint32_t(f32_to_e4m3(v[2])) << 16) |
                    (uint32_t(f32_to_e4m3(v[3])) << 24);
            }
        }
    }
}

}  // namespace

void gemm_fp8_scaled_launch(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m,
                            int64_t n, int64_t k, int out_dtype, hipStream_t stream) {
    const int tiles_m = int(cdiv(m, kT)), tiles_n = int(n / 128);
    const int64_t grid = int64_t(tiles_m) * tiles_n;
    QMM_CHECK(grid < (int64_t(1) << 31), "problem too large for one launch");
    auto go = [&](auto kern) {
        launch(kern, dim3(uint32_t(grid)), dim3(kThreads), size_t(kLdsBytes), stream, static_cast<const uint8_t *>(a),
               static_cast<const uint8_t *>(b), static_cast<const float *>(scale_a), static_cast<const float *>(scale_b), c,
               int(m), int(n), int(k), tiles_m);
    };
    switch (out_dtype) {
        case HIDET_QMM_F32: go(gemm_fp8_scaled_kernel<HIDET_QMM_F32>); break;
        case HIDET_QMM_F16: go(gemm_fp8_scaled_kernel<HIDET_QMM_F16>); break;
        case HIDET_QMM_BF16: go(gemm_fp8_scaled_kernel<HIDET_QMM_BF16>); break;
        case HIDET_QMM_E4M3: go(gemm_fp8_scaled_kernel<HIDET_QMM_E4M3>); break;
        default: QMM_FAIL("unsupported output dtype code " << out_dtype);
    }
}

}  // namespace qmm
