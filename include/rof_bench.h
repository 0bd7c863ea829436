/* rof_bench.h -- benchmark and tuning interface of librof.so: timing helpers that bracket the aggregation with
 * HIP events on the launch stream, plain copy and read kernels for calibrating profiler byte counters, and the
 * launch-tuning settings of a layout.  None of it has a counterpart in upstream and none of it is needed to use the
 * library (rof.h); bench.py and the tuning sweeps use it.
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

/* Plain streaming read of nbytes (a multiple of 16, pointer 16-byte aligned) of device memory, `repeat` times over in
 * one launch; `sink` is one float of device memory that is practically never written.  Timed over a buffer far
 * larger than the caches it gives the read rate the memory system sustains on this device, the yardstick for the
 * gather launches' fetch rate; over a buffer of a few MB read many times, the rate of the L2s.
 * No upstream counterpart. */
int rof_device_read(const void *src, size_t nbytes, int repeat, float *sink, void *stream);

/* Nothing but row gathers, as a yardstick for the aggregation launches: every group of `lanes_per_row` lanes (4, 8,
 * 10, 12, 16, 20, 32 or 64; a row has 16 x lanes_per_row bytes) fetches 2 x iters pseudo-random rows of a table of `rows` rows
 * (a power of two; 16-byte aligned), two in flight.  *gathered_rows (may be NULL) receives the number of rows the
 * launch fetches.  Timed over a table that the L2s hold (1-2 MiB), that the Infinity Cache holds (tens of MiB) or
 * that only HBM holds (GiB), it gives the rates that gathers of that row size can reach on this device.
 * No upstream counterpart. */
int rof_device_gather(const void *table, uint32_t rows, int lanes_per_row, int iters, float *sink, void *stream,
                      uint64_t *gathered_rows);

/* Launch tuning of one layout.  Every field has a "library decides" value, which is what a new layout holds; the
 * settings belong to the layout (no process-wide state) and are read by every aggregation that uses it, so change
 * them only while no other thread launches with the same layout.  No upstream counterpart.
 *   xcd_run_partial / xcd_run_dst: how many consecutive workgroups of the partial-sum launches / of the
 *     destination-row launch stay on one XCD (each XCD has its own L2, so runs of neighbouring destination rows
 *     share gathered rows there).  0 = the library's choice: 1 for the partial-sum launches; for the destination
 *     rows one tile of destinations (256 workgroups at least) per run when 35 % of the neighbours or more lie
 *     within min(max(8192, the rows that fill 4 MB), n / 16) ids of their row (block-structured and banded graphs),
 *     4 workgroups otherwise.
 *   wave_cap: wavefronts per SIMD of the destination-row launch, 2..7; 0 = as many as fit; -1 = the library's
 *     choice from the size of the feature matrix, the row bytes and the row stride.
 *   deep: see below.
 *   lds_pad: bytes (0..65536) of unused LDS requested per workgroup in every launch, which caps how many
 *     workgroups share a CU and with it the number of row gathers in flight. */
typedef struct {
    int32_t xcd_run_partial;
    int32_t xcd_run_dst;
    int32_t wave_cap;
    int32_t lds_pad;
    int32_t deep;          /* row gathers in flight per lane group: -1 = the library's choice (more of them when the */
                           /* caches serve the whole fp32 feature matrix and the launch gathers under 8 GB), 0 = two, */
                           /* 1 = four (five at 10 lanes per row) wherever such an instantiation exists (fp32 rows,  */
                           /* 32-bit offsets)                                                                        */
    int32_t reserved[3];
} rof_launch_tuning;

int rof_layout_set_tuning(rof_layout *layout, const rof_launch_tuning *tuning);

/* Choose the launch tuning of a layout by timing instead of by the size rules: runs the aggregation on the caller's
 * operands (arguments as rof_aggregate_epilogue; `out` receives the same, correct result every time, since no setting
 * changes a bit) with the wavefront cap of the destination-row launch at 8 / 7 / 6, with two and four row gathers in
 * flight where both exist, and with XCD runs of 4 / 16 / 256 / one tile, one setting after the other, keeping each
 * winner (`rounds` timings of `iters` calls per candidate, the fastest counts; HIP events on `stream`, which the call
 * synchronises).  The winners are stored in the layout (and returned in *chosen when not NULL) and hold until
 * rof_layout_set_tuning changes them; they were measured for this width, stride and type, so calibrate the layout
 * with the operands it will be used with.  Costs about (9 candidates x rounds x iters) aggregations. */
int rof_layout_calibrate(rof_layout *layout, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                         int feat_dim, int normalized, const rof_epilogue *epilogue, void *workspace,
                         size_t workspace_bytes, void *stream, int rounds, int iters, rof_launch_tuning *chosen);
/* The settings as stored (the "library decides" values are returned as such). */
int rof_layout_get_tuning(const rof_layout *layout, rof_launch_tuning *tuning);

#ifdef __cplusplus
}
#endif
#endif /* ROF_BENCH_H_ */
