/* rof.h -- C ABI of the MI355X reuse-aware neighbour-aggregation library (librof.so).
 *
 * Every entry point is extern "C", takes plain pointers and sizes, returns 0 or a negative
 * rof_status, never throws and never exits the process.  State lives in the handles it returns;
 * the only process-wide state is the static device scratch of rof_aggregate_noalloc (one copy per
 * GPU).  Host-side functions are safe to call concurrently on
 * different handles; device-side functions enqueue on the hipStream_t they are given and do not
 * synchronise.
 *
 * Citations name the upstream interface each entry point replaces (paths relative to the
 * upstream tree).
 */
#ifndef ROF_H_
#define ROF_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    ROF_OK = 0,
    ROF_ERR_ARG = -1,      /* null pointer, negative size, inconsistent array lengths        */
    ROF_ERR_RANGE = -2,    /* an index points outside its array (checked on the host)        */
    ROF_ERR_ALLOC = -3,    /* host or device allocation failed                               */
    ROF_ERR_DEVICE = -4,   /* a HIP call failed; rof_last_device_error() has the HIP text    */
    ROF_ERR_STATE = -5,    /* handle not in the state the call needs (e.g. weights not set)  */
    ROF_ERR_UNSUPPORTED = -6,
    ROF_ERR_WORKSPACE = -7 /* caller's workspace is smaller than rof_layout_workspace_bytes  */
} rof_status;

const char *rof_strerror(int status);
const char *rof_last_device_error(void); /* thread-local text of the last HIP failure */
/* Version of this interface.  A caller compiled against another value of ROF_ABI_VERSION than rof_version() returns
 * must not pass structs or fixed-size arrays to the library: 2 grew rof_layout_opts from 32 to 48 bytes and the array
 * of rof_layout_stats from 16 to 20 counters; 3 added rof_layout_stats_n (which takes the caller's count, so later
 * counters no longer change a signature) and moved the launch tuning of rof_bench.h from process-wide settings into
 * the layout.  Structs keep reserved fields so that they can gain members without growing. */
#define ROF_ABI_VERSION 3
int rof_version(void);

/* ------------------------------------------------------------------------------------------
 * Host side 1: the reuse-plan builder.  Stays on the CPU (OpenMP); every array is bit-exact
 * with the upstream builder's output for the same input.
 *
 * Results come back in a "bag" of named uint32 arrays owned by the library.
 * ---------------------------------------------------------------------------------------- */
typedef struct rof_bag rof_bag;

/* Borrowed pointer to a named array (valid until rof_bag_free); returns its length or -1. */
int64_t rof_bag_get(const rof_bag *bag, const char *name, const uint32_t **data);
void rof_bag_free(rof_bag *bag);

/* replaces py_split_part -> split_part
 * (ROF/reuse_search_ext/src/reuse_search_ext.cc:82-103, reuse_search_ext.h:82-148).
 * bag: "part_ptr"[parts+1], "part2Node"[parts], "num_parts_per_node_acc"[n]. */
int rof_split_part(const uint32_t *indptr_dst, uint32_t n, int part_size, rof_bag **out);

/* replaces py_get_part_intersect -> get_part_intersect (reuse_search_ext.cc:108-142, h:152-228),
 * count half: "intersect_count"[parts].  The lists themselves are produced on demand by
 * rof_part_intersect_lists, because materialising all of them is quadratic in hub degree. */
int rof_part_intersect_count(const uint32_t *part_ptr, uint64_t num_parts, const uint32_t *indices_src, uint64_t e,
                             const uint32_t *indptr_src, const uint32_t *indices_dst, uint32_t n, int part_size,
                             int discard_remainder_part, rof_bag **out);

/* The intersection lists of the parts named in which[0..n_which):
 * bag: "ptr"[n_which+1], "data"[ptr[n_which]] (each list ascending). */
int rof_part_intersect_lists(const uint32_t *part_ptr, uint64_t num_parts, const uint32_t *indices_src, uint64_t e,
                             const uint32_t *indptr_src, const uint32_t *indices_dst, uint32_t n, int part_size,
                             int discard_remainder_part, const uint32_t *which, uint64_t n_which, rof_bag **out);

/* replaces py_greedy_max_reuse -> greedy_max_reuse (reuse_search_ext.cc:145-160, h:232-303).
 * bag: "index_ordered"[parts], "index_picked"[P]. */
int rof_greedy_max_reuse(const uint32_t *intersect_count, uint64_t num_parts, const uint32_t *part_ptr,
                         const uint32_t *indices_src, uint64_t e, rof_bag **out);

/* replaces py_reorganize_indices -> reorganize_indices (reuse_search_ext.cc:169-211, h:409-505) and
 * py_reorganize_indices_uniquely -> reorganize_indices_uniquely (cc:214-257, h:507-640).
 * picked_dst_ptr/picked_dst = the intersection lists of the picked parts, in pick order.
 * which: 1 = v1 arrays, 2 = v2 arrays, 3 = both.
 * bag v1: "new_indices_src"[e], "part_pointers_cache"[P+1], "column_index_cache", "part_cache_flagindex"[parts]
 * bag v2: "uniqpart_column_index", "uniqpart_pointers"[U+1], "part2Node_ptr"[U+1], "part2Node_col". */
int rof_reorganize(const uint32_t *part_ptr, uint64_t num_parts, const uint32_t *indices_src, uint64_t e,
                   const uint32_t *index_picked, uint64_t num_picked, const uint32_t *picked_dst_ptr,
                   const uint32_t *picked_dst, const uint32_t *indptr_dst, uint32_t n,
                   const uint32_t *num_parts_per_node_acc, int part_size, int which, rof_bag **out);

/* replaces py_inverse_csc_or_csr -> inverse_csc (reuse_search_ext.cc:51-78, h:18-78).
 * bag: "indptr"[n+1], "indices"[e] (rows ascending). */
int rof_transpose_csr(const uint32_t *indptr, const uint32_t *indices, uint32_t n, uint64_t e, rof_bag **out);

/* The whole upstream call sequence (ROF_evaluation/ROF_main.py:71-127) in one call.  Pass
 * indptr_src/indices_dst = NULL for a symmetric graph (ROF_main.py:62-64).
 * bag: every array above plus "picked_dst_ptr"/"picked_dst". */
int rof_plan_build(const uint32_t *indptr_dst, const uint32_t *indices_src, const uint32_t *indptr_src,
                   const uint32_t *indices_dst, uint32_t n, uint64_t e, int part_size, int discard_remainder_part,
                   rof_bag **out);

/* A different reuse search, off by default: the "dynamic greedy" sketched and left unfinished in the comment at
 * reuse_search_ext.h:305-321.  Candidates are the full parts with >= 2 destinations in their intersection list
 * (h:152-228; equal source tuples count once); the candidate with the longest current list is picked, and every
 * candidate that shares a source with it loses the picked part's destinations (ties: lower part index).  A source
 * may thus sit in many shared parts, never in two parts of one destination.  Pass indptr_src/indices_dst = NULL
 * for a symmetric graph.  The plan comes out in upstream's v2 format (h:537-636):
 * bag: "uniqpart_column_index", "uniqpart_pointers"[U+1], "part2Node_ptr"[U+1], "part2Node_col",
 *      "index_picked"[shared parts] (part indices in pick order), "shared_parts"[1], "candidates"[1]. */
int rof_plan_dynamic_greedy(const uint32_t *indptr_dst, const uint32_t *indices_src, const uint32_t *indptr_src,
                            const uint32_t *indices_dst, uint32_t n, uint64_t e, int part_size, rof_bag **out);

/* A different reuse search, off by default: "hub patterns".  No counterpart in upstream, whose comment block at
 * reuse_search_ext.h:305-406 sketches a stronger search than its one-part-per-source greedy and leaves it
 * unfinished.  The `hubs` most frequent sources are tied into blocks of `block` (2..16) by popularity rank;
 * for every destination row and block, the subset of the block's hubs among the row's in-neighbours is a
 * pattern; a (block, pattern) of >= 2 hubs shown by enough rows becomes a shared part whose consumers are
 * exactly those rows.  A source may thus take part in many shared parts, never in two of one row.
 * The plan comes out in upstream's v2 format (h:537-636) with part size = block:
 * bag: "uniqpart_column_index", "uniqpart_pointers"[U+1], "part2Node_ptr"[U+1], "part2Node_col",
 *      "hub_ids"[<= hubs] (by rank), "shared_parts"[1]. */
int rof_plan_hub_patterns(const uint32_t *indptr_dst, const uint32_t *indices_src, uint32_t n, uint64_t e,
                          uint32_t hubs, int block, rof_bag **out);

/* ------------------------------------------------------------------------------------------
 * Host side 2: the device layout.  A plan in any of the three upstream tensor formats is
 * re-laid out into (a) a CSR of reuse groups with their consumers and (b) a destination-centric
 * CSR of residual neighbours; from those the library derives its execution schedule
 * (degree-binned row tasks, split hub rows, virtual column ids for group partial sums) and
 * uploads it.  The layout owns its device memory (hipMalloc) until rof_layout_free.
 * ---------------------------------------------------------------------------------------- */
typedef struct rof_layout rof_layout;

typedef struct {
    int32_t min_consumers;   /* a group is materialised iff it has >= this many consumers; 0 = cost model; -1 = all */
    int32_t disable_reuse;   /* 1: expand every group back into its consumers' rows (the comparator)      */
    int32_t hub_split;       /* rows with more entries than this are gathered in segments one launch earlier;  */
                             /* 0 = by the rows a wavefront gathers at once (G = 64 / lanes_per_row) and the    */
                             /* row bytes: float32 rows 128 / 256 (matrix within / beyond 256 MB) at G = 1 and   */
                             /* >= 1024 bytes; otherwise up to G = 3 128 within and 1024 beyond 256 MB; 1024 at   */
                             /* G = 4; 640 from 5 on; bfloat16 rows 256 for G <= 2, 512 at 3, 1280 above; lower     */
                             /* (down to 128) on launches so small that a row of that length would outlast them,   */
                             /* and adjusted on dense graphs by what their rows look like (see layout.cpp).  With    */
                             /* 0 here and in `segment`, a small graph (fewer than 16 384 wavefronts                 */
                             /* of rows, at most 256 rows beyond 256 entries, none beyond 1536 per row that a        */
                             /* wavefront gathers at once) keeps its long rows whole: the destination-row launch then */
                             /* sums each with 4, 8 or 16 wavefronts of one workgroup; there is no earlier launch    */
    int32_t segment;         /* entries per segment; 0 = an eighth to a quarter of hub_split (see layout.cpp).  A row  */
                             /* so long that adding up its segments would outlast the launch gets longer ones.    */
    int32_t lanes_per_row;   /* lanes one gathered row occupies in the kernel that will use this layout:   */
                             /* smallest of 4,8,10,12,16,20,32,64 >= ceil(feat_dim / 4) (fp32) or / 8      */
                             /* (bf16); 0 = 16.  Steers the default hub_split and the sharing gate.        */
    int32_t entry_order;     /* feature rows inside one task are gathered 0: by source id, descending      */
                             /* (default; measured 2-3 % faster than plan order and 20 % faster than a      */
                             /* random order on MI355X), 1: in the order the plan lists them, 2: ascending   */
    int32_t tile_rows;       /* short rows are sorted by length inside tiles of this many destinations; 0 = 4096 */
    int32_t elem_bytes;      /* bytes per element of the rows that will be gathered: 4 (float32, also 0) or 2        */
                             /* (bfloat16, whose partial-sum rows are twice as wide as its gathered rows).  Steers   */
                             /* the default hub_split.                                                              */
    int32_t local_groups;    /* workgroup-local sharing (min_consumers = 0 only): short destinations that consume the */
                             /* same groups are placed in one workgroup, which sums those groups once into LDS;      */
                             /* 0 = on: a cluster must save 8 row gathers (on graphs whose rows gather from their own    */
                             /* neighbourhood also an eighth of its rows' gathers: it gives up the tile order), and all  */
                             /* clusters together 64 MB of gathers; k > 0 = every cluster that saves k; -1 = off      */
    int32_t share_scope;     /* which consumers read a shared group from the workspace: 0 = every consumer; 1 = only rows   */
                             /* long enough to be cut into segments (more than hub_split entries with every group           */
                             /* expanded): their partial-row reads happen in the swept launch, whose working set is small,   */
                             /* while every other consumer gets the group's sources folded back into its row.  The tests of  */
                             /* min_consumers / the cost model then count the consumers in scope only.                      */
    int32_t row_bytes;       /* bytes of one gathered row (feat_dim x element size) in the kernel that will use this layout; */
                             /* 0 = unknown (taken as 16 x lanes_per_row).  Steers the default hub_split and segment: at one  */
                             /* row per wavefront, rows of 1024 bytes or more are cut finer than narrower ones.                */
    int32_t reserved[1];
} rof_layout_opts;

/* v2 tensors: replaces the plan arguments of reuse_forward_v2 / reuse_backward_v2
 * (ROF/reuse_conv/reuse_conv.cpp:288-346; kernel contract reuse_conv_kernel.cu:852-954). */
int rof_layout_from_v2(const int32_t *uniqpart_column_index, const int32_t *uniqpart_pointers,
                       const int32_t *part2Node_ptr, const int32_t *part2Node_col, int64_t num_uniqparts,
                       int32_t num_nodes, int part_size, const rof_layout_opts *opts, rof_layout **out);

/* v1 tensors: replaces the plan arguments of reuse_forward_v1 / reuse_backward_v1
 * (reuse_conv.cpp:199-285; kernel contract reuse_conv_kernel.cu:396-601). */
int rof_layout_from_v1(const int32_t *column_index, const int32_t *part_pointers, const int32_t *part2Node,
                       int64_t num_parts, const int32_t *part_cache_flagindex, const int32_t *part_pointers_cache,
                       const int32_t *column_index_cache, int64_t cache_num, int32_t num_nodes, int part_size,
                       const rof_layout_opts *opts, rof_layout **out);

/* GNNA tensors (no reuse): replaces the plan arguments of GNNA_forward / GNNA_backward / SAG
 * (reuse_conv.cpp:132-196; kernel contract reuse_conv_kernel.cu:205-286, 123-196). */
int rof_layout_from_parts(const int32_t *column_index, const int32_t *part_pointers, const int32_t *part2Node,
                          int64_t num_parts, int32_t num_nodes, int part_size, const rof_layout_opts *opts,
                          rof_layout **out);

/* Canonical arrays of the layout (host copies, int32 viewed as uint32):
 *   "group_ptr"[G+1] "group_col"  "group_dst_ptr"[G+1] "group_dst"  "res_ptr"[N+1] "res_col"
 * "xcd_run"[1] and "long_row_cut"[2] (hub_split, segment) as chosen for this layout;
 * the schedule of the three launches ("g_*", "s_*", "b_*": task_ptr, task_nref, task_out, col; for the destination
 * rows also "b_task_nlds", "b_lg_ptr", "b_lg_task_ptr", "b_lg_col", "b_lg_task_first" and "b_shape" = long tasks, tasks of
 * the ordinary launch, clusters, LDS rows per cluster)
 * and the v2 tensors reconstructed from them ("uniqpart_column_index", "uniqpart_pointers",
 * "part2Node_ptr", "part2Node_col"), which equal the input of rof_layout_from_v2 bit for bit
 * whenever that input has the upstream builder's canonical shape. */
int rof_layout_export(const rof_layout *layout, rof_bag **out);

/* Counters: [0] nodes [1] original edges [2] groups [3] groups materialised in the workspace [4] gathered rows per
 * pass (E_u) [5] partial-row reads (R) [6] partial rows written (incl. hub segments) [7] hub segments
 * [8] phase-A tasks [9] phase-B tasks [10] device bytes held [11] part_size [12] long tasks of launch 1 [13] of launch 2
 * [14] canonical flag [15] rows gathered by launch 1 [16] workgroup-local groups (summed into LDS; a group counts once
 * per workgroup that sums it) [17] reads of them [18] workgroups that hold clustered destinations [19] LDS rows the
 * destination-row launch asks for per workgroup. */
int rof_layout_stats(const rof_layout *layout, int64_t stats[20]);
/* The first `count` of the counters the library knows (fewer: the rest is dropped; more: zero-filled): the twenty
 * above, then [20] the cut of long rows (hub_split) and [21] the segment length as chosen for this layout, [22] the
 * entries of the longest task of the destination-row launch, [23] the rows that the destination-row launch of a small
 * graph sums with several wavefronts of one workgroup each (0: long rows are cut into segments as [20] and [21] say). */
int rof_layout_stats_n(const rof_layout *layout, int64_t *stats, int count);

/* Copy the schedule to the current HIP device (idempotent). */
int rof_layout_upload(rof_layout *layout, void *stream);

/* Per-edge weights rsqrt(deg[src]) and per-row scales rsqrt(deg[dst]) from the float32 in-degree
 * vector the upstream kernels take (reuse_conv_kernel.cu:254,276,943-944).  degrees: device, [n]. */
int rof_layout_set_degrees(rof_layout *layout, const float *degrees_dev, void *stream);

size_t rof_layout_workspace_bytes(const rof_layout *layout, int feat_dim);

void rof_layout_free(rof_layout *layout);

/* ------------------------------------------------------------------------------------------
 * Device side: the aggregation itself (hand-written gfx950 kernels, wave64, no MFMA,
 * no global atomics).  Computes, for every node v,
 *     out[v,:] = s(v) * sum over v's neighbour entries u of w(u) * x[u,:]
 * with w = s = rsqrt(deg) when normalized (GCN: reuse_conv_kernel.cu:205-286, 836-954) and
 * w = s = 1 otherwise (sum aggregation: reuse_conv_kernel.cu:123-196), evaluated through the
 * layout's reuse groups.  x: [n, feat_dim] with row stride ldx (elements), out: float32
 * [n, feat_dim] with row stride ldo; every row of out is overwritten (no zero-fill needed).
 * x, out and a bias start on a boundary of their element type (ROF_ERR_ARG otherwise), the workspace on 16 bytes.
 * The same call serves the backward pass on d_output because upstream runs the un-transposed
 * plan there (reuse_conv_kernel.cu:1021-1041).
 * ---------------------------------------------------------------------------------------- */
enum { ROF_F32 = 0, ROF_BF16 = 1 };

int rof_aggregate(const rof_layout *layout, const void *x, int x_dtype, int64_t ldx, float *out, int64_t ldo,
                  int feat_dim, int normalized, void *workspace, size_t workspace_bytes, void *stream);

/* rof_aggregate with the rest of the layer fused into the store of each output row:
 *     out[v,:] = act( aggregate(v) + self_weight * x[v,:] + bias )
 * bias: device float32[feat_dim] or NULL (upstream adds it in a separate pass after the operator,
 *   reuse_conv.py:147-150);
 * relu != 0 clamps at zero (upstream's models apply F.relu to the layer output as one more pass:
 *   activation=F.relu, ROF_evaluation/ROF_main.py:181-200);
 * self_weight: the node's own row, e.g. 1 + eps of a GIN layer over the unnormalised sum of upstream's SAG
 *   kernel (reuse_conv_kernel.cu:123-196); 0 = none;
 * out_dtype ROF_F32 or ROF_BF16: the sum is always accumulated in fp32; with ROF_BF16 the finished row is
 *   rounded to nearest even and stored as bf16 (row stride ldo in elements), ready to be the bf16 input of the
 *   next layer's GEMM or aggregation without a conversion pass.
 * pad_columns != 0: the caller allows the library to treat the rows as round_up(feat_dim, 4) (8 for bf16
 *   features) columns wide: ldx and ldo are at least that, the extra columns of x are readable, `bias` (if any) has
 *   that many elements, and the extra columns of `out` receive the aggregate of the extra columns of x (whatever
 *   they hold: uninitialised padding of x may put non-finite values into the padding of out, never into columns
 *   0 .. feat_dim-1, which are the same either way).  Every piece a lane stores is then 16-byte aligned
 *   (2.4 M x 47 floats: 1.23 ms in rows of 48 against 1.25 ms packed).
 * Rows of nodes without in-edges become act(self_weight * x[v] + bias).  ep == NULL is rof_aggregate. */
typedef struct {
    const float *bias;
    int32_t relu;
    int32_t out_dtype;
    float self_weight;
    int32_t pad_columns;
    int32_t reserved[2];
} rof_epilogue;

int rof_aggregate_epilogue(const rof_layout *layout, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                           int feat_dim, int normalized, const rof_epilogue *epilogue, void *workspace,
                           size_t workspace_bytes, void *stream);

/* rof_aggregate_epilogue for callers that cannot allocate device memory or bring a workspace: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in upstream (whose
 * operators allocate their output and intermediates on every call, reuse_conv_kernel.cu:302-303).  The partial-sum rows live in a static device array of
 * ROF_NOALLOC_WORKSPACE_BYTES inside the library, one copy per GPU, held until the process ends; the call itself
 * allocates and frees nothing.  Its address on a device is looked up once, by rof_layout_upload or by the first
 * call on that device (so make that first call outside a graph capture).
 * Returns ROF_ERR_WORKSPACE (rof_last_device_error() names the limit) when
 * rof_layout_workspace_bytes(layout, feat_dim) exceeds ROF_NOALLOC_WORKSPACE_BYTES: use rof_aggregate_epilogue
 * with a workspace of your own then.  All calls on one GPU share the array: calls that overlap in time on one
 * GPU (different streams or threads) race and must be serialised by the caller.  Nothing in the array has to be
 * cleared between calls, because every partial row is written before it is read within one call.
 * x, out, epilogue (may be NULL) and the result are exactly those of rof_aggregate_epilogue. */
#define ROF_NOALLOC_WORKSPACE_BYTES ((size_t)64 << 20)
int rof_aggregate_noalloc(const rof_layout *layout, const void *x, int x_dtype, int64_t ldx, void *out, int64_t ldo,
                          int feat_dim, int normalized, const rof_epilogue *epilogue, void *stream);

/* Column sums of a row-major device matrix: out[c] = sum_r x[r, c], x float32 or bfloat16 [n, f] with row
 * stride ldx (elements), out float32[f].  This is the bias gradient of a layer (upstream leaves it to autograd's
 * reduction of `out + self.bias`, reuse_conv.py:147-150); summed in fp32 in a fixed order (bitwise repeatable).
 * workspace: rof_column_sums_workspace_bytes(n, f) bytes of device memory. */
size_t rof_column_sums_workspace_bytes(int64_t n, int f);
int rof_column_sums(const void *x, int x_dtype, int64_t ldx, int64_t n, int f, float *out, void *workspace,
                    size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ROF_H_ */
