/*
 * mtq_measure.h -- measurement aids of libmtq_hip.so.
 *
 * Nothing in this header is part of the drop-in boundary (include/mtq.h): these entry
 * points have no kernel of the reference behind them. They exist so that a bench driver
 * can (a) bring the card's clocks to their sustained level before a timed region, as the
 * reference's runner does at start-up (GpuRunner::wake_dvfs,
 * crates/metaltile-std/src/runner.rs:280-284), (b) record the shader clock a timed region
 * ran at, and (c) calibrate hardware-counter readings and launch-size ceilings against
 * kernels of known size. Same conventions as mtq.h (0 or a negative MTQ_ERR_* code,
 * mtq_last_error()), same stream, mtq_init first.
 */
#ifndef MTQ_MEASURE_H
#define MTQ_MEASURE_H

#include "mtq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Sustained full-grid load: the cache-flush dispatch of mtq_flush_cache repeated until at least
 * `min_gpu_ms` milliseconds of GPU time have passed (at most 4096 dispatches), so that a timed
 * region that follows does not measure the clock ramp of a card coming out of idle. The
 * counterpart of GpuRunner::wake_dvfs (crates/metaltile-std/src/runner.rs:280-284: 64 flush
 * dispatches at start-up), sized by time instead of by count. *gpu_ms (may be NULL) receives the
 * GPU time spent, *dispatches (may be NULL) the number of dispatches. */
MTQ_API int mtq_wake_clocks(double min_gpu_ms, double *gpu_ms, int *dispatches);

/* One reading of the shader clock. A single wave runs a chain of `valu_ops` dependent 32-bit
 * integer adds (each issues in 4 shader clocks on a 16-lane SIMD) between two readings of the
 * constant-rate counter, so sclk_mhz = 4 * valu_ops / elapsed. counter_mhz is the rate of the
 * shader's own cycle counter (the clock64() of device code) against the constant-rate counter over
 * the same interval, reported beside it as a second reading. */
typedef struct mtq_clock_sample {
    double sclk_mhz;        /* shader clock from the dependent-add chain */
    double counter_mhz;     /* rate of the shader cycle counter */
    double probe_us;        /* length of the probe on the constant-rate counter */
    double wall_clock_mhz;  /* rate of the constant-rate counter (runtime attribute) */
    uint64_t valu_ops;      /* adds in the chain */
} mtq_clock_sample;
/* Enqueues the probe on the library's stream behind whatever is queued there, waits for it and
 * fills *out: called right after a timed region it reads the clock that region ended at. */
MTQ_API int mtq_clock_probe(mtq_clock_sample *out);

/* Plain device-to-device copy kernel of `bytes` (a multiple of 16), enqueued
 * `repeat` times; avg_us (may be NULL) receives the mean GPU duration. No
 * counterpart in the reference: it is the known-size kernel hardware-counter
 * readings are calibrated against. */
MTQ_API int mtq_copy_kernel(void *dst, const void *src, size_t bytes, int repeat, double *avg_us);

/* Measurement aid, no counterpart in the reference: a kernel that only reads. `repeat` passes over the n_srcs
 * buffers of `bytes` bytes each (bytes % 16 == 0) are enqueued back to back on the library's stream, one launch per
 * buffer, `workgroups` (0 = 2048) workgroups of 256 threads with `in_flight` (1, 2, 4, 8; 0 = 8) 16-byte loads in
 * flight per thread (nontemporal != 0: loads marked as not to be kept in cache); *avg_us is the average launch duration
 * over the run, gaps between launches included. `sink` is 4 bytes of device memory that are (in practice) never
 * written. With more buffers than the last-level cache holds this is the rate at which a launch of that size can
 * stream HBM at all: the ceiling for a weight-streaming kernel of the same size. */
MTQ_API int mtq_read_kernel(const void *const *srcs, int n_srcs, size_t bytes, int repeat, int workgroups,
                            int in_flight, int nontemporal, void *sink, double *avg_us);

/* The wave-per-four-rows make of the headline GEMV (4-bit codes, groups of 64, bf16, rows of K = 4096 codes, N a multiple
 * of 16) with parts switched off: one wave per four weight rows, every load issued at once, no LDS, no barrier, the dot products
 * on the matrix cores (metaltile_amd/csrc/qmv_rows.hip, the kernel mtq_qmv runs at this shape). `sets` is n_sets x 5 device pointers (w, scales, biases, x,
 * out of one operand set, laid out as for mtq_qmv); `repeat` passes over the sets are enqueued back to back and
 * *avg_us (may be NULL) receives the average launch duration, gaps included. mode 0 computes the product (out is the
 * same as mtq_qmv's up to the order of the f32 sums), 1 leaves the arithmetic out (loads, the lane reduction and the
 * stores stay), 2 only loads the weights. With `stamps` (device memory, N / 4 x MTQ_ROWS_PROBE_STAMPS u64, or NULL)
 * one more launch on set 0 follows in the same chain, in front of n_sets - 1 plain ones, whose waves write readings of
 * the constant-rate counter: wave started, all loads issued, activations in operand order, first row done, all rows
 * done, results stored. */
#define MTQ_ROWS_PROBE_STAMPS 6
MTQ_API int mtq_probe_qmv_rows(const void *const *sets, int n_sets, uint32_t N, int mode, int repeat, uint64_t *stamps,
                               double *avg_us);

#ifdef __cplusplus
}
#endif
#endif /* MTQ_MEASURE_H */
