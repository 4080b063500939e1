/*
 * Measurement and test hooks of libhidet_qmm.so.  Nothing here is part of the operator path: bench.py, the profiles and
 * the tests bind these symbols; a host that only runs the operators needs hidet_qmm.h alone.  Same conventions as
 * there (extern "C", errors through hidet_get_last_error).  None has a counterpart in the reference except where noted.
 */
#ifndef HIDET_QMM_BENCH_H
#define HIDET_QMM_BENCH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- timing hook ---------------------------------------------------------------------------------
 * hidet_qmm_arm_timing makes the NEXT compute-kernel launch issued from this thread record its
 * own begin and end into the two events (the dispatch's timestamps, without launch gaps).  The
 * role of the reference's CompiledFunction.profile (python/hidet/runtime/compiled_module.py:106-147). */
void *hidet_qmm_event_create(void);
void hidet_qmm_event_destroy(void *event);
void hidet_qmm_event_record(void *event, void *stream);
void hidet_qmm_event_synchronize(void *event);
float hidet_qmm_event_elapsed_ms(void *start, void *stop);
void hidet_qmm_arm_timing(void *start_event, void *stop_event);

/* launches `launches` W8A16 matmuls (hidet_symmetric_quant_matmul_f16_i8 with parallel_k_parts = 0, one activation block a
 * [m, k] against weights[i % ring], scales[i % ring] into outs[i % ring]) back to back from one native loop, launch i
 * recording its own begin and end into start_events[i] / stop_events[i] (both arrays may be NULL: untimed).  What a timed
 * pass of a benchmark needs so that the host interpreter's time per call (about as long as a decode kernel runs) does not
 * drain the stream's queue between two launches.  An error ends the loop and is reported as usual. */
void hidet_qmm_gemv_ring_timed(const void *a, const void *const *weights, const void *const *scales, void *const *outs, int ring,
                               int launches, int64_t m, int64_t k, int64_t n, int64_t lda, void *workspace,
                               int64_t workspace_bytes, void *const *start_events, void *const *stop_events, void *stream);

/* ---- kernels that only read ------------------------------------------------------------------------
 * One kernel that reads `bytes` (a multiple of 32768) from src with 16-byte loads, 32 KiB contiguous per workgroup,
 * and does nothing else (sink: 4 bytes of device memory, practically never written).  Timed through the hook above it
 * gives the rate at which this memory system delivers a matrix of that size to a kernel: the ceiling of the decode
 * kernels at their real sizes, next to the 8 TB/s of the data sheet. */
void hidet_qmm_read_probe(const void *src, int64_t bytes, void *sink, void *stream);
/* The loads of the W8A16 decode kernel over an int8 matrix w[k, n] without its arithmetic and its exchange: the
 * (256-column tile, row) space in workgroups x 8 equal runs, one per wave of 512-thread workgroups, walked in steps of
 * 32 rows with one step (8 non-temporal 16-byte loads per lane, each wave instruction covering four 256-byte row
 * segments n bytes apart) in flight.  contiguous != 0 reads the same bytes per wave as 1 KiB pieces instead.  K a
 * multiple of 32, N a multiple of 256.  What this takes is the floor under the decode kernel's time for its access
 * pattern; the difference to hidet_qmm_read_probe is the price of the [K, N] layout. */
void hidet_qmm_pattern_probe(const void *w, int64_t k, int64_t n, int workgroups, int contiguous, void *sink, void *stream);

/* ---- test hook -------------------------------------------------------------------------------------
 * Re-reads of the mailbox after which a collector of the split-K exchange gives up (process-wide, applies to launches
 * made afterwards; negative restores the default of about a second of polling).  Tests set 0 to reach the give-up path
 * of hidet_qmm_exchange_status with kernels that all finish at once. */
void hidet_qmm_set_exchange_spin_limit(int limit);

#ifdef __cplusplus
}
#endif
#endif /* HIDET_QMM_BENCH_H */
