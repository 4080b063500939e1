/*
 * C ABI of libhidet_qmm.so: MI355X (gfx950) kernels for Hidet's quantized-matmul operator path.
 *
 * Conventions (the ones Hidet's runtime applies to every compiled task library):
 *   - every symbol is extern "C", default visibility, prefixed `hidet_`
 *     (reference: include/hidet/runtime/common.h:16-18, python/hidet/backend/codegen.py:60-70);
 *   - entry points return void; a failure is reported through the thread-local, read-once
 *     last-error string, which the caller polls after every call
 *     (reference: python/hidet/backend/codegen.py:72-93, python/hidet/runtime/compiled_module.py:79-102);
 *   - arguments are inputs first, then outputs, as raw device pointers, followed by explicit
 *     extents; the caller owns every buffer, outputs included, and keeps it alive until the stream
 *     has run the work (reference: python/hidet/runtime/compiled_task.py:146-207);
 *   - work is enqueued asynchronously on the hipStream_t passed as the last argument (the
 *     reference keeps one process-global stream, src/hidet/runtime/hip/context.cpp:35-41; here it
 *     is explicit per call, so there is no global state besides the error string);
 *   - scratch memory comes from the caller as (workspace, workspace_bytes) instead of the
 *     reference's grow-only global request_hip_workspace (src/hidet/runtime/hip/context.cpp:43-57).
 *     The workspace must be zero-filled once when it is allocated.  Its first 64 KiB are arrival counters and the
 *     next quarter of what remains (16 MiB at most) is the mailbox through which the bandwidth-bound kernels
 *     exchange split-K partial sums: the kernels leave every counter and every mailbox word they use at zero
 *     again.  The rest is plain scratch.  Two calls that overlap in time (different streams) must not share a
 *     workspace, and nothing else may write to one while a call is in flight.
 *     In bytes: counters = 65536; mailbox = min(16 MiB, (workspace_bytes - 65536) / 4) rounded down to a multiple of 256;
 *     scratch = workspace_bytes - 65536 - mailbox.  What each entry point needs of it:
 *       hidet_symmetric_quantize          scratch >= 4 * outer * inner bytes (an error otherwise);
 *       hidet_fp8_quantize_per_tensor     scratch >= 4 bytes (an error otherwise);
 *       hidet_symmetric_quant_matmul_f16_i8[_bias], hidet_symmetric_quant_matmul_w4a16[_bias] with up to 16 rows
 *                                         mailbox >= 1024 * min(m, 16) bytes per workgroup of the K split, at most 256
 *                                         workgroups unless parallel_k_parts asks for more (4 MiB serve every automatic
 *                                         plan); with less the kernels use fewer workgroups, never an error;
 *       the same with more rows, hidet_matmul_f8, hidet_matmul_f8_scaled, the _nk matmuls
 *                                         scratch: 64 KiB per tile computed in K ranges times the ranges (optional: with
 *                                         less, fewer or no tiles are split; hidet_qmm_min_workspace_bytes() serves
 *                                         every shape); hidet_symmetric_quant_matmul_w4a16 with a few hundred to a few
 *                                         thousand rows: 64 MiB for its plan of equal runs of work per workgroup
 *                                         (optional: with less it computes whole tiles and equal K ranges).
 *     hidet_qmm_workspace_bytes_for_scratch(s) returns the smallest workspace whose scratch part holds s bytes.
 *
 * All tensors are dense row-major.  No function allocates device memory; none but hidet_qmm_exchange_status synchronises.
 */
#ifndef HIDET_QMM_H
#define HIDET_QMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: the workspace gained the mailbox (see above and hidet_qmm_workspace_bytes_for_scratch); measurement hooks moved to
 * hidet_qmm_bench.h; hidet_qmm_exchange_status / hidet_qmm_exchange_reset added. */
#define HIDET_QMM_ABI_VERSION 2

/* element type codes */
enum {
    HIDET_QMM_F32 = 0,
    HIDET_QMM_F16 = 1,
    HIDET_QMM_BF16 = 2,
    HIDET_QMM_I8 = 3,
    HIDET_QMM_I16 = 4,
    HIDET_QMM_E4M3 = 5, /* OCP float8 e4m3fn: max 448, no infinities */
    HIDET_QMM_E5M2 = 6  /* OCP float8 e5m2: max 57344 */
};

/* ---- error state: same two symbols, same semantics as the reference runtime ------------------
 * replaces include/hidet/runtime/logging.h:60-63 and src/hidet/runtime/logging.cpp:20-36.
 * hidet_get_last_error returns the message once and clears it; NULL when there is none. */
void hidet_set_last_error(const char *msg);
const char *hidet_get_last_error(void);

/* ---- library facts ---------------------------------------------------------------------------*/
int hidet_qmm_abi_version(void);
const char *hidet_qmm_arch(void);            /* "gfx950" */
/* A workspace of this size lets every entry point use the K split it would choose for the shapes of a 4096- to 8192-wide
 * transformer; with less (or with very wide outputs) the kernels use fewer K slices, down to none, never an error. */
int64_t hidet_qmm_min_workspace_bytes(void);
/* The smallest workspace_bytes whose scratch part (what follows the counters and the mailbox) holds scratch_bytes. */
int64_t hidet_qmm_workspace_bytes_for_scratch(int64_t scratch_bytes);

/* ---- health of the split-K exchange ------------------------------------------------------------------
 * The bandwidth-bound kernels sum their K slices through the workspace's mailbox: a workgroup that holds a column tile's
 * last rows polls the mailbox for the partial tiles of the others.  The poll is bounded; if a partial tile never shows
 * up (a workspace that was not zero-filled, two overlapping calls on one workspace, a device fault) the workgroup
 * writes NaN to its outputs, sets a flag in the workspace and returns, and the mailbox may be left with stale words that
 * would corrupt later calls.  No counterpart in the reference, whose split-K parts are separate outputs summed by a
 * second operator (python/hidet/graph/ops/quant/resolve.py:99).
 * hidet_qmm_exchange_status waits for `stream`, then returns 1 if any launch on this workspace gave up since the last
 * reset, 0 if none did, -1 on an error (last-error string).  hidet_qmm_exchange_reset enqueues kernels on `stream` that
 * zero the counters, the flag and the mailbox; call it after a status of 1, with no other call on the workspace in
 * flight.  workspace == NULL names the current device's array of hidet_symmetric_quant_matmul_f16_i8_static. */
int hidet_qmm_exchange_status(const void *workspace, int64_t workspace_bytes, void *stream);
void hidet_qmm_exchange_reset(void *workspace, int64_t workspace_bytes, void *stream);

/* ---- symmetric quantize / dequantize ---------------------------------------------------------
 * replaces the auto-scheduled kernels of SymmetricQuantizationTask / SymmetricDeQuantizationTask
 * (python/hidet/graph/ops/quant/symmetric.py:23-61).  The tensor is viewed as [outer, reduce, inner]
 * with the reduced axes folded into `reduce`; scale is [outer, inner] in w's dtype.
 *   scale = max|w| / qmax, wq = saturating_cast(round(w / scale)), evaluated in w's dtype (float32, float16 or
 *   bfloat16); round is the reference's GPU lowering for that dtype: ties away from zero for float32
 *   (python/hidet/ir/primitives/hip/math/float32.py:40), ties to even for float16 and bfloat16
 *   (hip/math/float16.py:42, cuda/math/bfloat16.py:29); a slice of zeros gives scale 0 and codes 0.
 * q_dtype is HIDET_QMM_I8 or HIDET_QMM_I16. */
void hidet_symmetric_quantize(const void *w, void *wq, void *scale, int64_t outer, int64_t reduce, int64_t inner,
                              int w_dtype, int q_dtype, void *workspace, int64_t workspace_bytes, void *stream);
/* w = cast(wq, scale dtype) * scale */
void hidet_symmetric_dequantize(const void *wq, const void *scale, void *w, int64_t outer, int64_t reduce,
                                int64_t inner, int q_dtype, int s_dtype, void *stream);

/* ---- W8A16: c[m, n] = sum_k a[m, k] * (f16(w[k, n]) * scale[n]) --------------------------------
 * replaces SymmetricQuantizedMatmulTask (python/hidet/graph/ops/quant/matmul.py:24-74) and the
 * tuned CUDA template SymmetricQuantizedMatmulF16I8Task with its split-K sum
 * (python/hidet/graph/ops/quant/matmul_f16_i8.py:30-93, resolve.py:99).
 * a: float16 [m, k] with row stride lda (elements); w: int8 [k, n]; scale: float16 [n]; c: float16 [m, n].
 * fp32 accumulation.  parallel_k_parts: 0 lets the library choose the K split, > 0 is a hint. */
void hidet_symmetric_quant_matmul_f16_i8(const void *a, const void *w, const void *scale, void *c, int64_t m,
                                         int64_t k, int64_t n, int64_t lda, int parallel_k_parts, void *workspace,
                                         int64_t workspace_bytes, void *stream);
/* The same two operators with the bias of a linear layer added in the epilogue: c = f16(f16(acc * scale[n]) + bias[n]),
 * the bits the matmul followed by a float16 add gives (the reference's fused epilogue adds to the stored float16 value
 * as well); bias float16 [n] (NULL: none).  No counterpart in the reference's operator signature; it is the fused form of
 * the epilogue the reference's template admits (allow_epilogue, python/hidet/graph/ops/quant/matmul_f16_i8.py:95-99), so
 * that a rewritten nn.Linear with bias is one launch. */
void hidet_symmetric_quant_matmul_f16_i8_bias(const void *a, const void *w, const void *scale, const void *bias, void *c,
                                              int64_t m, int64_t k, int64_t n, int64_t lda, int parallel_k_parts,
                                              void *workspace, int64_t workspace_bytes, void *stream);
void hidet_symmetric_quant_matmul_f16_i8_nk_bias(const void *a, const void *w_nk, const void *scale, const void *bias, void *c,
                                                 int64_t m, int64_t k, int64_t n, int64_t lda, int64_t ldw, void *workspace,
                                                 int64_t workspace_bytes, void *stream);
/* The same operator for callers that can neither allocate device memory nor pass a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose tasks
 * take their scratch from the runtime's grow-only request_hip_workspace).  Same arguments, checks, kernels and results
 * as hidet_symmetric_quant_matmul_f16_i8 called with a workspace of HIDET_QMM_STATIC_SCRATCH_BYTES; the scratch memory
 * is an array of that size inside the library's device code, one copy per GPU for the life of the process.  The call
 * allocates and frees nothing.  Up to 16 rows (and whenever the bandwidth-bound kernel is chosen) a shape whose K split
 * needs more mailbox memory than the array's share of it (a quarter: 4 MiB) is rejected with an error that names the
 * bytes needed; taller matrices always run, in as many K ranges as fit the scratch part.  Every call on one GPU uses the same array: calls that overlap in
 * time on one GPU (two streams, two threads) race; calls ordered by a stream or by events do not.  The device the
 * stream belongs to must be current.  The first call on a device looks up the array's address (hipGetSymbolAddress):
 * make it outside any stream capture; later calls only launch kernels and may be captured. */
#define HIDET_QMM_STATIC_SCRATCH_BYTES ((16 << 20) + (64 << 10))
int64_t hidet_qmm_static_scratch_bytes(void);
void hidet_symmetric_quant_matmul_f16_i8_static(const void *a, const void *w, const void *scale, void *c, int64_t m,
                                                int64_t k, int64_t n, int64_t lda, int parallel_k_parts, void *stream);
/* The same operator for a weight that is stored K-contiguous: w_nk[n * ldw + k] = w[k, n] (the [K, N] operand held
 * with strides (1, ldw); what torch's nn.Linear keeps, and what a matmul with transpose_b=True reads,
 * python/hidet/graph/ops/matmul/matmul.py:37-38, python/hidet/graph/frontend/torch/register_functions.py:165-167).
 * The reference's quantized operator has no such form (its rewrite rule re-emits the matmul without transpose_b,
 * python/hidet/graph/transforms/graph_patterns/quant/linear.py:43-49).  The reduction then runs along the
 * contiguous axis: up to 16 rows take the bandwidth-bound kernels, which need no workspace; more rows the MFMA GEMM
 * reading this layout (K a multiple of 64; the workspace is optional, NULL means no tile is computed in K ranges,
 * which matters below a few hundred rows).  K and ldw multiples of 16, w_nk 16-byte aligned. */
void hidet_symmetric_quant_matmul_f16_i8_nk(const void *a, const void *w_nk, const void *scale, void *c, int64_t m,
                                            int64_t k, int64_t n, int64_t lda, int64_t ldw, void *workspace,
                                            int64_t workspace_bytes, void *stream);

/* ---- group-wise W4A16 (benchmark configuration; the reference has no operator for it) -----------
 * Conventions inherited from the reference: int4b is signed with max 7, so the symmetric rule of
 * python/hidet/graph/ops/quant/symmetric.py:32-41 gives scale = amax / 7; sub-byte tensors are packed
 * along the innermost axis, element o in byte o / 2 at bit (o % 2) * 4
 * (python/hidet/transforms/lower_integer_subbyte.py:103-113), i.e. byte [k, j] = q[k, 2j] | q[k, 2j+1] << 4;
 * scales are [K / group, N] as in the reference's test kernel (tests/cute_kernel/quantized_linear.py:692-699).
 *
 * hidet_group_quantize_int4: w float32 [k, n] -> packed uint8 [k, n/2], scales [k/group, n] (s_dtype:
 * bfloat16 or float16); scale32 = amax / 7 and code = clamp(round_half_away(w / scale32), -7, 7) in float32. */
void hidet_group_quantize_int4(const void *w, void *packed, void *scales, int64_t k, int64_t n, int group_size,
                               int w_dtype, int s_dtype, void *stream);
/* c[m, n] = sum_g scales[g, n] * sum_{k in g} a[m, k] * q[k, n]; a, scales, c share `dtype` (bfloat16 or
 * float16); fp32 accumulation. */
void hidet_symmetric_quant_matmul_w4a16(const void *a, const void *w, const void *scales, void *c, int64_t m, int64_t k,
                                        int64_t n, int64_t lda, int group_size, int dtype, int parallel_k_parts,
                                        void *workspace, int64_t workspace_bytes, void *stream);
/* The same with bias[n] (of `dtype`, not NULL) added to the rounded result, c = dtype(dtype(sum) + bias): the bits of
 * the matmul followed by an add, as for the int8 operator (hidet_symmetric_quant_matmul_f16_i8_bias). Up to 32 rows the
 * add rides in the kernel's epilogue; above, a short element-wise pass follows the GEMM. */
void hidet_symmetric_quant_matmul_w4a16_bias(const void *a, const void *w, const void *scales, const void *bias, void *c,
                                             int64_t m, int64_t k, int64_t n, int64_t lda, int group_size, int dtype,
                                             int parallel_k_parts, void *workspace, int64_t workspace_bytes, void *stream);
/* The same operator on weights repacked for decode: w_nk is uint8 [n, k/2] with row stride ldw bytes, row n holding
 * the k codes of output column n; inside every 32-bit word (8 consecutive k) nibble i is code 2i for i < 4 and code
 * 2(i-4)+1 for i >= 4 (hidet_amd.graph.ops.quant.to_decode_layout_int4 repacks). scales stay [k/group, n]. No
 * counterpart in the reference, like the operator itself; the layout is the int4 analogue of the transpose_b=True
 * weight of python/hidet/graph/ops/matmul/matmul.py:37-38. Needs k a multiple of 128, a group size of 128 times a
 * power of two and 16-byte aligned rows; meant for decode: every 16 rows of a are one more pass over the weights.
 * No workspace. */
void hidet_symmetric_quant_matmul_w4a16_nk(const void *a, const void *w_nk, const void *scales, void *c, int64_t m,
                                           int64_t k, int64_t n, int64_t lda, int64_t ldw, int group_size, int dtype,
                                           void *stream);

/* ---- per-tensor float8 e4m3 quantization (benchmark configuration) --------------------------------
 * scale[0] = max|x| / 448 (float32, written to device memory), codes = e4m3(x / scale), round to nearest
 * even, saturating; e4m3 limits from python/hidet/ir/dtypes/floats.py:108-110. */
void hidet_fp8_quantize_per_tensor(const void *x, void *codes, void *scale, int64_t numel, int x_dtype,
                                   void *workspace, int64_t workspace_bytes, void *stream);

/* ---- FP8 e4m3 matmul: c[m, n] = cast(alpha * sum_k a[m, k] * b[n, k]) ------------------------------
 * replaces MatmulF8Task (python/hidet/graph/ops/matmul/matmul_f8.py:132-175, 693-742): a is [m, k] and b is
 * [n, k], both K-major e4m3 with row strides lda / ldb (bytes = elements); fp32 accumulation; out_dtype is the
 * element type of c (float8_e4m3, float16, bfloat16 or float32).  scale_a / scale_b are optional pointers to
 * one float32 each in device memory (per-tensor scales of the benchmark configuration); alpha is their
 * product, NULL counts as 1 (the reference's unscaled task).  No shape has to be a tile multiple.
 * `workspace` (optional, may be NULL; same buffer and rules as for the int8 matmul: zero-initialised once, at
 * least hidet_qmm_min_workspace_bytes() serves every shape, one per stream) lets matrices of a few hundred
 * rows be computed in K ranges by several workgroups per tile, summed in a fixed order; it stands in for the
 * workspace the reference's compiled tasks request from the runtime (src/hidet/runtime/hip/context.cpp:43-57). */
void hidet_matmul_f8(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                     int out_dtype, const void *scale_a, const void *scale_b, void *workspace, int64_t workspace_bytes,
                     void *stream);
/* The same task for float8_e5m2 operands (the reference accepts both operands e4m3 or both e5m2,
 * python/hidet/graph/ops/matmul/matmul_f8.py:709-712): same arguments and meaning as hidet_matmul_f8 without the
 * workspace; out_dtype float8_e5m2, float16, bfloat16 or float32 (conversion to e5m2 rounds to nearest even and
 * saturates at +-57344). Served by the MFMA's bf8 format on a plainer kernel than the e4m3 one. */
void hidet_matmul_f8_e5m2(const void *a, const void *b, void *c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                          int out_dtype, const void *scale_a, const void *scale_b, void *stream);
/* replaces MatmulF8ScaledTask (python/hidet/graph/ops/matmul/matmul_f8.py:357-454, 632-636): per K block of
 * 128, c += (sum_{k in block} a * b) * scale_a[kb, m] * scale_b[n / 128, kb]; scale_a float32 [k/128, m],
 * scale_b float32 [n/128, k/128]; a [m, k] and b [n, k] dense. */
void hidet_matmul_f8_scaled(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m,
                            int64_t n, int64_t k, int out_dtype, void *workspace, int64_t workspace_bytes, void *stream);
/* The same task for float8_e5m2 operands (MatmulF8ScaledTask asserts only that both operands have the same dtype,
 * python/hidet/graph/ops/matmul/matmul_f8.py:386-389, and _matmul_f8 admits both-e5m2 for the scaled form too, :709-712):
 * same arguments and meaning; out_dtype float8_e5m2, float16, bfloat16 or float32. Same kernels with the MFMA's bf8
 * operand format. */
void hidet_matmul_f8_scaled_e5m2(const void *a, const void *b, const void *scale_a, const void *scale_b, void *c, int64_t m,
                                 int64_t n, int64_t k, int out_dtype, void *workspace, int64_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HIDET_QMM_H */
