/* rof_bench.h -- benchmark and tuning interface of librof.so: timing helpers that bracket the aggregation with
 * HIP events on the launch stream, a plain copy kernel for calibrating profiler byte counters, and two process-wide
 * launch-tuning settings.  None of it has a counterpart in upstream and none of it is needed to use the library
 * (rof.h); bench.py and the tuning sweeps use it.  The two settings are plain globals read by every launch: set
 * them before launching from other threads, not while.
 */
#ifndef ROF_BENCH_H_
#define ROF_BENCH_H_

#include "rof.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Timing helper for benchmarks: runs rof_aggregate_epilogue (rof_aggregate when epilogue == NULL) `iters` times on `stream` between two HIP
 * events recorded on that same stream and returns the mean milliseconds per call. */
int rof_aggregate_timed(const rof_layout *layout, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                        int feat_dim, int normalized, const rof_epilogue *epilogue, void *workspace,
                        size_t workspace_bytes, void *stream, int iters, float *ms_per_call);

/* Per-launch timing for the roofline report: ms_launch[1] = mean duration of the destination-row
 * launch alone (HIP events on `stream` around it), ms_launch[0] = mean duration of the whole call minus
 * that, i.e. the partial-sum launch.  No upstream counterpart. */
int rof_aggregate_launch_times(const rof_layout *layout, const void *x, int x_dtype, int64_t ldx, void *out,
                               int64_t ldo, int feat_dim, int normalized, const rof_epilogue *epilogue,
                               void *workspace, size_t workspace_bytes, void *stream, int iters, float ms_launch[2]);

/* Plain device-to-device streaming copy (nbytes a multiple of 16, pointers 16-byte aligned).  Exists so
 * that a profiler's FETCH_SIZE / WRITE_SIZE counters can be calibrated against a transfer of known size.
 * No upstream counterpart. */
int rof_device_copy(void *dst, const void *src, size_t nbytes, void *stream);

/* Launch tuning: how many consecutive workgroups of the partial-sum launches / of the destination-row launch
 * stay on one XCD (each XCD has its own L2, so runs of neighbouring destination rows share gathered rows
 * there).  run_launch2 = 0 (the default) lets every layout use its own choice: one tile of destinations per
 * run when at least half of the neighbours lie within 8192 ids of their row (block-structured graphs), 4
 * workgroups otherwise.  Process-wide; no upstream counterpart. */
int rof_set_xcd_run(int run_launch1, int run_launch2);

/* Launch tuning: request `bytes` (0..65536) of unused LDS per workgroup, which caps how many workgroups
 * share a CU (160 KB LDS each) and with it the number of row gathers in flight.  Process-wide. */
int rof_set_lds_pad(int bytes);

#ifdef __cplusplus
}
#endif
#endif /* ROF_BENCH_H_ */
