// Internal types shared by the host-side sources of librof.so.  Not installed.
#ifndef ROF_INTERNAL_H_
#define ROF_INTERNAL_H_

#include <cstdint>
#include <map>
#include <string>
#include <vector>

struct rof_bag {
    std::map<std::string, std::vector<uint32_t>> arr;
};

// One launch worth of work: tasks in execution order.  Task t gathers the rows named by
// col[task_ptr[t] .. task_ptr[t+1]) -- the first task_nref[t] of them are partial-sum rows
// (ids >= the node count, pointing into the workspace), the rest are feature rows -- and writes
// their weighted sum to output row task_out[t].  Tasks [0, n_wave) are long and get a whole
// wavefront each; the remaining ones are short and share a wavefront.
//
// Destination-row phase only: workgroup-local reuse groups.  The tasks [n_regular, n_tasks) at the end of the list
// are *clustered*: destinations that share reuse groups, brought together by the schedule builder and run by a
// launch of their own, one workgroup per cluster.  Cluster i has the tasks lg_task_first[i] .. lg_task_first[i+1]
// (any number of short tasks, worked through in rounds).  Its workgroup first sums the cluster's local groups
// lg_ptr[i] .. lg_ptr[i+1] into LDS rows 0, 1, ... (local group j gathers lg_col[lg_task_ptr[j] ..
// lg_task_ptr[j+1])), and the tasks then take those partial sums from LDS: the first task_nlds[t] entries of such
// a task are LDS row numbers (before the task_nref[t] partial-sum rows and the feature rows).
struct rof_phase_host {
    std::vector<int32_t> task_ptr, task_nref, task_out, col;
    int32_t n_wave = 0;
    int32_t n_tasks = 0;
    std::vector<int32_t> task_nlds;                  // empty: no task reads LDS rows
    std::vector<int32_t> lg_ptr, lg_task_ptr, lg_col, lg_task_first;
    int32_t n_regular = 0;                           // tasks of the ordinary launch (= n_tasks without clusters)
    int32_t lg_blocks = 0;                           // clusters
    int32_t lg_max_rows = 0;                         // most LDS rows any cluster needs
};

struct rof_phase_dev {
    int32_t *task_ptr = nullptr, *task_nref = nullptr, *task_out = nullptr, *col = nullptr;
    float *w = nullptr;       // per entry: rsqrt(deg[col]) for feature rows, 1 for partial rows
    float *scale = nullptr;   // per task: rsqrt(deg[task_out]) (destination rows only)
    int32_t n_wave = 0, n_tasks = 0;
    int64_t n_entries = 0;
    // workgroup-local groups (destination rows only); task_nref then carries task_nlds in its top 8 bits
    int32_t *lg_ptr = nullptr, *lg_task_ptr = nullptr, *lg_col = nullptr, *lg_task_first = nullptr;
    float *lg_w = nullptr;
    int64_t lg_entries = 0;
    int32_t n_regular = 0, lg_blocks = 0, lg_max_rows = 0;
};

struct rof_layout {
    int32_t n = 0;
    int32_t part_size = 0;
    int64_t e_orig = 0;
    bool canonical = false;   // group/residual arrays reproduce the upstream v2 tensors exactly
    // canonical arrays: CSR of reuse groups (+ their consumers) and destination-centric residual CSR
    std::vector<int32_t> group_ptr, group_col, group_dst_ptr, group_dst, res_ptr, res_col;
    // schedule
    rof_phase_host g, s, b;   // g: shared groups; s: segments of long rows (may read g's rows); b: destination rows
    int32_t hub_split = 0, segment = 0;
    int32_t xcd_run = 4;      // consecutive workgroups of the destination-row launch kept on one XCD
    int32_t coop_tasks = 0;   // small launches: the first this many destination tasks are summed by several wavefronts each,
    int32_t coop16 = 0, coop8 = 0;   // the first coop16 of them by 16 (a whole workgroup), the next coop8 by 8, the rest by 4
    // launch tuning of the benchmark interface (rof_layout_set_tuning): 0 / -1 = the library's own choice
    int32_t tune_xcd_run_partial = 0, tune_xcd_run_dst = 0, tune_wave_cap = -1, tune_lds_pad = 0, tune_deep = -1;
    bool local_sources = false;   // 35 % of the gathered rows lie within min(max(8192, rows of 4 MB), n / 16) ids of their destination
    int64_t n_slots = 0;      // rows of the partial-sum workspace
    int64_t n_materialised = 0, n_segments = 0, gathered_rows = 0, partial_reads = 0, gathered_before_rows = 0;
    int64_t n_local_groups = 0, lds_reads = 0;   // workgroup-local groups (summed into LDS) and the reads of them
    // device copies
    rof_phase_dev dg, ds, db;
    bool uploaded = false, weights_set = false;
    int device = -1;
    int32_t lds_per_cu = 0;   // LDS bytes of one CU of that device (0: not queried; the gfx950 figure is used)
    int64_t device_bytes = 0;
};

void rof_set_device_error(const char *what, const char *text);

#endif
