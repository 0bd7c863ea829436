// Host side of the device layout: turns a plan in any of the three upstream tensor formats into
//   (1) the canonical arrays -- a CSR of reuse groups with their consumers, and a destination-centric
//       CSR of residual neighbours -- from which the upstream v2 tensors can be rebuilt bit for bit;
//   (2) the execution schedule for the gfx950 kernels: every destination row becomes one task whose
//       entries are either feature-row ids or "virtual" ids >= N naming a partial-sum row; groups that
//       are worth sharing become tasks of a first launch and segments of very long rows tasks of a second
//       launch, both filling partial-sum rows that the last launch (one task per destination) reads.
//       Tasks are ordered long-to-short, short ones tile by tile, so that the lanes of a wavefront that
//       share one launch slot do the same amount of work; inside a task the gathered rows are listed by
//       descending id, which keeps consecutive gathers close in memory.
#include <algorithm>
#include <functional>
#include <memory>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <new>
#include <numeric>
#include <vector>
#include <omp.h>

#include "rof.h"
#include "rof_internal.h"

namespace {

typedef std::vector<int32_t> ivec;

// Tasks up to this many entries share a wavefront (one lane group each); longer ones get a wavefront of their
// own.  Measured on MI355X at 5 rows per wavefront: 64 and 128 are 1 % faster than 32 and 256 is slower; at one
// row per wavefront 64 equals 32 and 128 is 10 % slower.  A launch too small to fill the machine twice is bound
// by its longest task instead and keeps the lower cut (16 384 rows: 18 us against 26).
const int32_t kShortRow = 64, kShortRowSmall = 32;
const int64_t kWavesToFill = 2 * 8192;   // two rounds of 256 CUs x 32 wavefronts
// Rows that several wavefronts of one workgroup sum on small launches: more entries than kCoopRow, at most kCoopMaxRows
// of them (measured with the 16 wavefronts of a workgroup for every row, kCoopWaves in agg_rows.h: 2^14 nodes x 32 floats, 106 rows beyond 256 entries
// 6.4 us, 468 beyond 128 entries 9.4, two launches with segments 10.7; 2^16 nodes, 697 rows beyond 256 entries: 26.4 us
// against 22.5 with segments), the longest of at most kCoopChain entries per lane group (2486 entries at two rows per
// wavefront, 78 per lane group: 15.7 us against 18.9).
const int32_t kCoopRow = 256, kCoopWaves = 16, kCoopChain = 96, kCoopMaxRows = 256;
// Wavefronts per such row: 16 (a whole workgroup) beyond kCoopRow16 entries, 8 beyond kCoopRow8, 4 below (2^15 nodes,
// 121 long rows, 16 / 32 / 47 floats: 8.2 / 9.1 / 11.2 us with 16 wavefronts for every row, 7.4 / 8.5 / 11.0 with the
// steps at 1024 and 512 entries, 6.5 / 7.9 / 10.1 at 2048 and 1024; 2^14 nodes: 6.5 / 6.2 / 6.2 at 32 floats).
const int32_t kCoopRow16 = 2048, kCoopRow8 = 1024;
// Long rows.  Rows longer than a cut are gathered in segments that fill partial rows one launch earlier, and
// the segment tasks of all rows run in the order of the highest source id they gather (entries inside a task are
// listed by descending id): every wavefront in flight then works in the same narrow band of the feature matrix
// and the launch sweeps the matrix once from top to bottom, so a row gathered for one destination is still in
// L2 when the next destinations need it.  The effect is large -- rotating each row's list by a random offset,
// which keeps every task monotone but puts the tasks out of phase, costs 25 % on the 2.4 M-node workload -- and
// it is why the cut is low.  Every segment writes and re-reads one partial row (fp32, so twice a gathered row when
// those are bf16), which is what stops finer cuts.  The table below is measured (MI355X, R-MAT graphs of 2^18 to
// 2.4 M nodes and average degrees 8 to 48, cut / segment from 64 / 16 to 8192 / 2048; G = rows a wavefront gathers
// per instruction), the figures are the cost of the neighbouring choices against the one taken:
//   fp32, G = 1, rows of 1024 bytes or more: 128 / 32 when the caches can hold the matrix (2^18 nodes x 256 floats:
//     256 / 64 +7 %, 1024 / 256 +15 %), else 256 / 32 (128 / 32 0 ... +7 %, 512 / 128 +7 ... +8 %);
//   fp32, G = 1, narrower rows (160 floats): 1024 / 128 on matrices beyond the caches (128 / 32 +2 ... +34 %,
//     512 / 64 -2 ... +4 %, 2048 / 512 +4 ... +13 %), 128 / 32 on smaller ones (1024 / 128 +11 %);
//   fp32, G = 2 ... 3 (100 floats): 1024 / 128 beyond the caches (128 / 32 +2 ... +26 %, 256 / 64 +1 ... +5 %),
//     128 / 32 on smaller matrices (1024 / 128 +3 %);
//   fp32, G = 4 (64 floats): 1024 / 128 (384 / 96 0 ... +6 %, 128 / 32 +1 ... +19 %);
//   fp32, G >= 5: 640 / 160 (1024 / 256 -2 ... +2 %, 256 / 64 +4 ... +7 %, 5457 +7 % on the 2.4 M-node workload);
//   fp32, G >= 4, fewer rows than fill the machine twice: 256 / 128 (G = 4: 128 / 64), and any cut steps down where
//     the longest task under it would outlast the launch (see default_cut);
//   bf16, G <= 2 (256 columns): 256 / 48 (2^22 nodes: -18 % against 8192; segments of 32 / 40 / 48 / 56 / 64 / 96 /
//     128 entries 8.53 / 8.49 / 8.46 / 8.57 / 8.57 / 8.92 / 9.17 ms), 256 / 128 when the caches can hold the matrix,
//     128 / 32 on launches that cannot fill the machine twice; G = 3: 512 / 128; G >= 4 (128 columns):
//     1280 / 320 (640 / 160 -1 ... +4 %, 2560 / 640 0 ... +4 %).
// No rule of sizes gets every graph right (the same width wants 128 / 32 on one graph and 1024 / 128 on another),
// which is what the timed choice between candidate layouts is for (LayoutFamily(autotune=True)).
// (Giving long rows a whole workgroup instead -- four wavefronts combined through LDS -- was measured as well:
// no faster than segments on any workload, so it is not built in.)
const int64_t kCachedMatrixBytes = 256 << 20;   // the Infinity Cache
const int64_t kL2Bytes = 4 << 20;               // of one XCD
// The longest task of a launch is one chain of dependent gathers, measured at (10 + 0.14 x row bytes) ns an entry
// while the caches serve them; a launch lasts about 15 us + 60 us per GB it gathers.  Entries a chain may have if it
// is not to outlast 3/4 of the launch:
int64_t chain_limit(int64_t edges, int64_t row_bytes) {
    const int64_t launch_ns = 15000 + edges * row_bytes * 60 / 1000000;
    const int64_t entry_ns = 10 + row_bytes * 14 / 100;
    return 3 * launch_ns / (4 * entry_ns);
}
void default_cut(int32_t groups, int32_t elem_bytes, int64_t row_bytes, int64_t matrix_bytes, int64_t rows, int64_t edges,
                 int32_t &cut, int32_t &segment) {
    const bool cached = matrix_bytes <= kCachedMatrixBytes;
    if (elem_bytes == 2 && groups <= 2) {
        // segments of 48 entries are the optimum of the 2^22-node workload; matrices that the caches hold want
        // fewer, longer segments (2^16 ... 2^18 nodes x 256 columns: 256 / 128 is 3 ... 23 % faster than 256 / 48),
        // and the smallest launches the short chains of 128 / 32
        cut = rows / groups < kWavesToFill ? 128 : 256;
        segment = rows / groups < kWavesToFill ? 32 : cached ? 128 : 48;
    } else if (elem_bytes == 2) {
        cut = groups == 3 ? 512 : 1280;
        segment = cut / 4;
    } else if (groups == 1 && row_bytes >= 1024) {
        cut = cached ? 128 : 256;
        segment = 32;
    } else if (groups <= 3) {
        cut = cached ? 128 : 1024;
        segment = cached ? 32 : 128;
    } else if (rows / groups < kWavesToFill) {
        // a destination-row launch that cannot fill the machine twice lasts as long as its longest task: a lower cut
        // shortens that chain of dependent gathers (2^14 nodes x 32 floats: 13.2 us at 640 / 160, 11.0 at 256 / 128,
        // 11.6 at 128 / 64, 14.3 at 1024 / 256; 2^15 nodes x 64 floats: 25.4 us at 256 / 128, 20.5 at 128 / 64)
        cut = groups == 4 ? 128 : 256;
        segment = groups == 4 ? 64 : 128;
    } else if (groups == 4) {
        cut = 1024;
        segment = 128;
    } else {
        cut = 640;
        segment = 160;
    }
    // Where a chain of `cut` entries would outlast the launch (chain_limit), the launch waits for its longest rows
    // (2^17 nodes, average degree 8, 64 floats: 46.6 us at 1024 / 128, 30.3 at 384 / 96; 2^16 nodes, degree 15: 45.8
    // against 25.7), so the cut steps down.
    const int64_t limit = chain_limit(edges, row_bytes);
    static const int32_t kLadder[][2] = {{1024, 128}, {640, 160}, {384, 96}, {256, 128}};
    for (const auto &step : kLadder) {
        if (cut <= limit || cut <= 256) break;
        if (step[0] < cut) {
            cut = step[0];
            segment = step[1];
        }
    }
}
// Sharing groups costs one more launch (~4-6 us on MI355X), and on heavy-tailed graphs what it saves is cheap:
// the sources of a popular group are themselves popular rows that sit in L2, while the partial rows that
// replace them are read a few dozen times each.  Measured gain of the destination-row launch against the net
// saving (row gathers saved - partial-row reads added), as a fraction of all gathers and in bytes:
//   R-MAT, upstream plans: 1.1 % / 128 MB -> -0.7 .. +0.4 %;  2.4 % / 283 MB -> -1.5 %;  1.2 % / 845 MB -> 0.0 %
//   R-MAT, hub-pattern plans: 3.3 % -> -0.9 %;  6.2 % -> -4.5 %
//   planted reuse: 81 % / 1.9 GB -> +45 .. +100 %;  small graph, 4 MB -> -6 us of 18
// A small saving is a saving on hub rows; only a plan that removes a sizeable part of all gathers is worth its
// partial rows.  Plans below either figure are executed with every group folded back into its consumers.
const int64_t kMinSavedBytes = 256000000;
const int64_t kMinSavedShare = 10;   // net saving >= 1/10 of all gathers
const int32_t kTileRows = 4096;      // short tasks are length-sorted inside tiles of this many rows
// A workgroup of clustered destinations is kept when its local groups save at least this many row gathers: below
// that the two barriers and the serial start of the workgroup cost more than the gathers it avoids.
const int64_t kMinClusterSaving = 8;

bool ptr_ok(const int32_t *p, int64_t n, int64_t *total) {
    if (!p || p[0] != 0) return false;
    for (int64_t i = 0; i < n; ++i)
        if (p[i] > p[i + 1]) return false;
    *total = p[n];
    return true;
}

bool ids_ok(const int32_t *a, int64_t len, int64_t bound) {
    bool ok = true;
#pragma omp parallel for schedule(static) reduction(&& : ok)
    for (int64_t i = 0; i < len; ++i)
        if (a[i] < 0 || a[i] >= bound) ok = false;
    return ok;
}

// Is the multi-consumer-first / node-ascending / part_size-chunked shape of the upstream v2 emitter
// (reuse_search_ext.h:537-636) present?  Only then does the export reproduce the input exactly.
bool v2_is_canonical(const int32_t *uptr, const int32_t *dptr, const int32_t *dcol, int64_t U, int ps, int64_t G) {
    int64_t w = G;
    while (w < U) {
        int32_t node = dcol[dptr[w]];
        if (w > G && dcol[dptr[w - 1]] >= node) return false;   // nodes strictly ascending across runs
        int64_t run = w;
        while (run < U && dcol[dptr[run]] == node) ++run;
        for (int64_t q = w; q < run; ++q) {
            int32_t len = uptr[q + 1] - uptr[q];
            if (len < 1 || len > ps || (q + 1 < run && len != ps)) return false;
        }
        w = run;
    }
    return true;
}

struct TaskList {   // tasks in natural order, before sorting
    ivec ptr{0}, nref, out, col, nlds;
    void begin_task(int32_t out_row) { out.push_back(out_row); }
    void end_task(int32_t refs, int32_t lds_rows = 0) {
        nref.push_back(refs);
        nlds.push_back(lds_rows);
        ptr.push_back((int32_t)col.size());
    }
};

// Short tasks placed by the schedule builder rather than by the tile order: whole workgroups of destinations that
// share reuse groups (see build_clusters), with the groups each workgroup sums into LDS.
struct Clusters {
    ivec tasks;                       // destination tasks of the cluster section, cluster by cluster
    ivec task_first{0};               // per cluster: its range in `tasks`
    ivec lg_ptr{0}, lg_task_ptr{0}, lg_col;   // per workgroup: its local groups; per local group: its sources
    int32_t max_rows = 0;
    // destination -> (group, LDS row) pairs served from LDS
    ivec of_node;                     // index into ptr, or -1
    ivec ptr{0}, group, row;
};

// Cut between long tasks (a wavefront each) and short ones (a lane group each) for a launch of these task lengths.
int32_t short_cut(const int64_t T, const int64_t over, int32_t groups) {
    return over + (T - over + groups - 1) / groups >= kWavesToFill ? kShortRow : kShortRowSmall;
}

// Long tasks first (descending), then the short tasks tile by tile, each tile descending, and last the tasks of
// `placed` in their given order (the clustered short tasks, may be null; they run in a launch of their own, one lane
// group each whatever their length, so the cut between long and short tasks is taken from the other tasks alone).
// `groups`: short tasks that share a wavefront.  With `band` (one key per task: the highest source id it gathers)
// both kinds are ordered by descending key instead.
void order_tasks(const ivec &ptr, int64_t tile_rows, int32_t groups, const ivec *band, const ivec *placed,
                 ivec &order, int32_t &n_wave) {
    int64_t T = (int64_t)ptr.size() - 1;
    order.clear();
    order.reserve(T);
    std::vector<char> taken;
    if (placed && !placed->empty()) {
        taken.assign(T, 0);
        for (int32_t t : *placed) taken[t] = 1;
    }
    auto free_task = [&taken](int64_t t) { return taken.empty() || !taken[t]; };
    int64_t over = 0, mine = 0;
    for (int64_t t = 0; t < T; ++t)
        if (free_task(t)) {
            ++mine;
            over += ptr[t + 1] - ptr[t] > kShortRow;
        }
    const int32_t cut = short_cut(mine, over, groups);
    ivec longs;
    for (int64_t t = 0; t < T; ++t)
        if (free_task(t) && ptr[t + 1] - ptr[t] > cut) longs.push_back((int32_t)t);
    if (band && cut == kShortRow) {   // a launch too small to fill the machine keeps the longest-first order
        ivec shorts;
        for (int64_t t = 0; t < T; ++t)
            if (free_task(t) && ptr[t + 1] - ptr[t] <= cut) shorts.push_back((int32_t)t);
        auto higher = [band](int32_t x, int32_t y) { return (*band)[x] > (*band)[y]; };
        std::stable_sort(longs.begin(), longs.end(), higher);
        std::stable_sort(shorts.begin(), shorts.end(), higher);
        n_wave = (int32_t)longs.size();
        order = longs;
        order.insert(order.end(), shorts.begin(), shorts.end());
        if (placed) order.insert(order.end(), placed->begin(), placed->end());
        return;
    }
    std::stable_sort(longs.begin(), longs.end(),
                     [&ptr](int32_t x, int32_t y) { return ptr[x + 1] - ptr[x] > ptr[y + 1] - ptr[y]; });
    n_wave = (int32_t)longs.size();
    order = longs;
    std::vector<ivec> bucket(cut + 1);
    for (int64_t t0 = 0; t0 < T; t0 += tile_rows) {
        int64_t t1 = std::min(T, t0 + tile_rows);
        for (auto &b : bucket) b.clear();
        for (int64_t t = t0; t < t1; ++t) {
            int32_t len = ptr[t + 1] - ptr[t];
            if (len <= cut && free_task(t)) bucket[len].push_back((int32_t)t);
        }
        for (int32_t len = cut; len >= 0; --len) order.insert(order.end(), bucket[len].begin(), bucket[len].end());
    }
    if (placed) order.insert(order.end(), placed->begin(), placed->end());
}

void finalize_phase(const TaskList &tl, int64_t tile_rows, int32_t groups, bool by_band, rof_phase_host &ph,
                    const Clusters *cl = nullptr) {
    int64_t T = (int64_t)tl.out.size();
    ivec order, band;
    if (by_band) {
        band.resize(T);
        for (int64_t t = 0; t < T; ++t) {
            const int32_t first = tl.ptr[t] + tl.nref[t];   // feature rows follow the partial-row references
            band[t] = first < tl.ptr[t + 1] ? tl.col[first] : -1;
        }
    }
    order_tasks(tl.ptr, tile_rows, groups, by_band ? &band : nullptr, cl ? &cl->tasks : nullptr, order, ph.n_wave);
    ph.n_tasks = (int32_t)T;
    ph.n_regular = ph.n_tasks;
    if (cl && !cl->tasks.empty()) {
        ph.n_regular = ph.n_tasks - (int32_t)cl->tasks.size();
        ph.lg_blocks = (int32_t)cl->lg_ptr.size() - 1;
        ph.lg_task_first = cl->task_first;
        for (int32_t &f : ph.lg_task_first) f += ph.n_regular;   // positions in the ordered task list
        ph.lg_ptr = cl->lg_ptr;
        ph.lg_task_ptr = cl->lg_task_ptr;
        ph.lg_col = cl->lg_col;
        ph.lg_max_rows = cl->max_rows;
        ph.task_nlds.resize(T);
    }
    ph.task_ptr.assign(T + 1, 0);
    ph.task_nref.resize(T);
    ph.task_out.resize(T);
    for (int64_t i = 0; i < T; ++i) {
        int32_t t = order[i];
        ph.task_ptr[i + 1] = ph.task_ptr[i] + (tl.ptr[t + 1] - tl.ptr[t]);
        ph.task_nref[i] = tl.nref[t];
        ph.task_out[i] = tl.out[t];
        if (!ph.task_nlds.empty()) ph.task_nlds[i] = tl.nlds[t];
    }
    ph.col.resize(tl.col.size());
#pragma omp parallel for schedule(dynamic, 4096)
    for (int64_t i = 0; i < T; ++i) {
        int32_t t = order[i];
        int32_t len = tl.ptr[t + 1] - tl.ptr[t];
        if (len) memcpy(ph.col.data() + ph.task_ptr[i], tl.col.data() + tl.ptr[t], (size_t)len * sizeof(int32_t));
    }
}

// Workgroup-local reuse.  A reuse group whose consumers sit in one workgroup is summed once by that workgroup into
// LDS and read from there by each consumer: no partial row travels through memory and no launch is added (upstream
// keeps the partial sum of a part in shared memory too and fans it out with atomics, reuse_conv_kernel.cu:876-952;
// here the consumers come to the partial sum instead).  The schedule builder is free to order destination tasks, so
// it brings consumers together: the short destinations (one lane group each) that consume a group with at least two
// such consumers are sorted by the first such group they consume and cut into clusters of up to kClusterTasks
// (preferably where the group changes); one workgroup works through a cluster's tasks in rounds.  In every cluster
// the groups that at least two of its destinations consume become local groups, most saving first, as far as the
// LDS rows go.  Clusters that save fewer than `min_saving` row gathers are dissolved (their destinations return to
// the tile order).  full_len[v]: entries of destination v with every group expanded.
const int32_t kClusterTasks = 64;
// One workgroup works through a cluster alone, 4 * `groups` tasks at a time, so a cluster is also limited by its
// work: at most this many entries per lane group.  (Clusters of 64 rows of up to 64 entries each at one row per
// wavefront took longer than the whole launch of all other rows.)
const int32_t kClusterDepth = 96;
// The clusters run as a launch of their own (~8 us with its tail on MI355X): they are kept only if together they
// save at least this many bytes of row gathers.
const int64_t kMinLocalSavedBytes = 64000000;

void build_clusters(const rof_layout *L, const ivec &ng_ptr, const ivec &ng, const ivec &full_len, int32_t cut,
                    int32_t groups, int32_t max_rows, int64_t min_saving, bool relative_gate, Clusters &cl) {
    const int32_t n = L->n;
    const int64_t G = (int64_t)L->group_ptr.size() - 1;
    cl.of_node.assign(n, -1);
    if (G == 0) return;
    auto glen = [&](int32_t g) { return L->group_ptr[g + 1] - L->group_ptr[g]; };
    // groups with at least two short consumers
    ivec short_consumers(G, 0);
    for (int32_t v = 0; v < n; ++v)
        if (full_len[v] <= cut)
            for (int32_t j = ng_ptr[v]; j < ng_ptr[v + 1]; ++j) short_consumers[ng[j]]++;
    struct Cand { int32_t key, len, v; };
    std::vector<Cand> cand;
    for (int32_t v = 0; v < n; ++v) {
        if (full_len[v] > cut) continue;
        for (int32_t j = ng_ptr[v]; j < ng_ptr[v + 1]; ++j)
            if (short_consumers[ng[j]] >= 2 && glen(ng[j]) >= 2) {
                cand.push_back({ng[j], full_len[v], v});   // ng lists a node's groups in ascending order
                break;
            }
    }
    if ((int64_t)cand.size() < 2) return;
    std::sort(cand.begin(), cand.end(), [](const Cand &a, const Cand &b) {
        return a.key != b.key ? a.key < b.key : a.len != b.len ? a.len > b.len : a.v < b.v;
    });
    ivec count(G, 0), touched, pick;
    ivec row_of(G, -1);
    size_t b0 = 0;
    while (b0 < cand.size()) {
        // whole runs of destinations with the same first group while they fit -- by tasks, and by the LDS rows
        // their shared groups need; a run that does not fit is split only if the cluster would otherwise stay
        // less than half full
        size_t b1 = b0;
        int32_t shared = 0;   // groups that at least two destinations of the cluster consume
        int64_t work = 0;     // entries of the cluster's rows
        const int64_t max_work = (int64_t)4 * groups * kClusterDepth;
        touched.clear();
        auto add = [&](size_t i0, size_t i1) {
            for (size_t i = i0; i < i1; ++i)
                for (int32_t j = ng_ptr[cand[i].v]; j < ng_ptr[cand[i].v + 1]; ++j) {
                    const int32_t c = count[ng[j]]++;
                    if (c == 0) touched.push_back(ng[j]);
                    shared += c == 1 && glen(ng[j]) >= 2;
                }
        };
        auto remove = [&](size_t i0, size_t i1) {
            for (size_t i = i0; i < i1; ++i)
                for (int32_t j = ng_ptr[cand[i].v]; j < ng_ptr[cand[i].v + 1]; ++j)
                    shared -= --count[ng[j]] == 1 && glen(ng[j]) >= 2;
        };
        while (b1 < cand.size() && b1 - b0 < (size_t)kClusterTasks) {
            size_t run = b1;
            while (run < cand.size() && cand[run].key == cand[b1].key) ++run;
            if (run - b0 > (size_t)kClusterTasks) {
                if (b1 - b0 >= (size_t)kClusterTasks / 2) break;
                run = b0 + kClusterTasks;
            }
            int64_t run_work = 0;
            for (size_t i = b1; i < run; ++i) {
                run_work += cand[i].len;
                if (work + run_work > max_work && i > b0 + 1) {   // the part of the run that still fits (two rows at least)
                    run_work -= cand[i].len;
                    run = i;
                    break;
                }
            }
            if (run == b1) break;
            work += run_work;
            add(b1, run);
            if (shared > max_rows && b1 > b0) {   // this run's groups no longer fit into the LDS rows
                remove(b1, run);
                work -= run_work;
                break;
            }
            b1 = run;
            if (work >= max_work) break;
        }
        pick.clear();
        for (int32_t g : touched)
            if (count[g] >= 2 && glen(g) >= 2) pick.push_back(g);
        std::sort(pick.begin(), pick.end(), [&](int32_t a, int32_t b) {
            const int64_t sa = (int64_t)(count[a] - 1) * glen(a), sb = (int64_t)(count[b] - 1) * glen(b);
            return sa != sb ? sa > sb : a < b;
        });
        if ((int32_t)pick.size() > max_rows) pick.resize(max_rows);
        int64_t saving = 0;
        for (int32_t g : pick) saving += (int64_t)(count[g] - 1) * glen(g) - count[g] / 4;   // four LDS reads ~ one gather
        // A cluster gives up its rows' place in the tile order (and with it the locality of neighbouring rows on one
        // XCD) and is worked through by one workgroup: by default it is kept only if it removes at least an eighth
        // of its rows' gathers (block-structured graph, part size 2: clusters saving 3 % made the layer 1.7x slower).
        if (!pick.empty() && saving >= min_saving && (!relative_gate || saving * 8 >= work)) {
            for (size_t r = 0; r < pick.size(); ++r) {
                row_of[pick[r]] = (int32_t)r;
                cl.lg_col.insert(cl.lg_col.end(), L->group_col.begin() + L->group_ptr[pick[r]],
                                 L->group_col.begin() + L->group_ptr[pick[r] + 1]);
                cl.lg_task_ptr.push_back((int32_t)cl.lg_col.size());
            }
            cl.lg_ptr.push_back((int32_t)cl.lg_task_ptr.size() - 1);
            cl.max_rows = std::max(cl.max_rows, (int32_t)pick.size());
            // inside the cluster: by what is left of each row, longest first, so that the lane groups that share
            // a wavefront finish together
            std::vector<std::pair<int32_t, int32_t>> rest;   // (remaining entries, destination)
            for (size_t i = b0; i < b1; ++i) {
                const int32_t v = cand[i].v;
                int32_t len = full_len[v];
                cl.of_node[v] = (int32_t)cl.ptr.size() - 1;
                for (int32_t j = ng_ptr[v]; j < ng_ptr[v + 1]; ++j)
                    if (row_of[ng[j]] >= 0) {
                        cl.group.push_back(ng[j]);
                        cl.row.push_back(row_of[ng[j]]);
                        len -= glen(ng[j]) - 1;
                    }
                cl.ptr.push_back((int32_t)cl.group.size());
                rest.push_back({len, v});
            }
            std::sort(rest.begin(), rest.end(), [](const std::pair<int32_t, int32_t> &a, const std::pair<int32_t, int32_t> &b) {
                return a.first != b.first ? a.first > b.first : a.second < b.second;
            });
            for (auto &p : rest) cl.tasks.push_back(p.second);
            cl.task_first.push_back((int32_t)cl.tasks.size());
            for (int32_t g : pick) row_of[g] = -1;
        }
        for (int32_t g : touched) count[g] = 0;
        b0 = b1;
    }
}

int build_schedule(rof_layout *L, const rof_layout_opts *o) {
    const int32_t n = L->n;
    const int64_t G = (int64_t)L->group_ptr.size() - 1;
    int32_t lpr = (o && o->lanes_per_row > 0) ? o->lanes_per_row : 16;
    if (lpr > 64) lpr = 64;
    const int32_t groups = std::max(1, 64 / lpr);
    const int64_t total = (int64_t)L->res_col.size() + (int64_t)L->group_dst.size();
    const int32_t elem_bytes = (o && o->elem_bytes == 2) ? 2 : 4;
    const int64_t row_bytes = (o && o->row_bytes > 0) ? o->row_bytes : (int64_t)lpr * 16;
    int32_t rule_cut = 0, rule_segment = 0;
    default_cut(groups, elem_bytes, row_bytes, (int64_t)n * row_bytes, n, L->e_orig > 0 ? L->e_orig : total, rule_cut,
                rule_segment);
    // entries of every destination with every group expanded
    ivec len_all((size_t)n);
    {
        std::vector<int64_t> len((size_t)n);
        for (int32_t v = 0; v < n; ++v) len[v] = L->res_ptr[v + 1] - L->res_ptr[v];
        for (int64_t g = 0; g < G; ++g)
            for (int32_t j = L->group_dst_ptr[g]; j < L->group_dst_ptr[g + 1]; ++j)
                len[L->group_dst[j]] += L->group_ptr[g + 1] - L->group_ptr[g];
        for (int32_t v = 0; v < n; ++v) len_all[v] = (int32_t)std::min<int64_t>(len[v], INT32_MAX);
    }
    // Dense graphs: two thirds of all edges in rows of more than 128 entries.  What suits them depends on whether a
    // set of sources that one L2 can hold is popular -- the share of all gathers that goes to the 4 MB / row bytes
    // most gathered rows.
    //  * Popular sources (45 % and more; measured 47-64 %) stay in L2 by themselves, and what the segments cost counts:
    //    the fine cut of the wide rows (128 / 32 up to three rows per wavefront on a matrix that the caches hold) was
    //    measured at average degree 14, where it balances a few hub rows; where the segments are the launch, 32 entries
    //    are too few for a task that costs a wavefront, a partial row written and read, and three dependent loads
    //    before its first gather (R-MAT 2^18 nodes, average degree 83, 160 floats: 1.15 ms at 128 / 32, 0.89 at 128 /
    //    64, 0.86 at 128 / 128, 0.79 at 512 / 128, 0.75 at 1024 / 128; 2^16 nodes, degree 341: 0.87 / 0.72 at 512 /
    //    128; 512 / 128 is at or within 6 % of the best of seven choices on the nine such graphs measured at 72, 100
    //    and 160 floats; rows of 1 KB: 256 / 64 within 4 % of the best on four graphs, 1024 / 128 up to 14 % behind
    //    and 128 / 32 up to 22 %).
    //  * No popular sources (uniform degrees of 600: 3-12 %; R-MAT a = .5 on 233 000 nodes, average degree 435: 30-40
    //    %): a row gathered as one task ranges over the whole matrix and misses, while the segments of a row of `len`
    //    entries each gather from a band of segment / len of it, which the swept launch keeps in L2.  So the wide
    //    rows keep their fine cut (uniform degrees, 160 floats: 2.95 ms at 128 / 32, 5.08 at 128 / 128; the R-MAT
    //    graph, 128 floats: 2.84 at 128 / 32, 3.17 at 512 / 128), and from four rows per wavefront, where half of the
    //    rows are that long, the cut comes down to 256 / 64 so that the rows are cut at all (uniform degrees of 600 sit just under 640: 24 floats 1.35 ms at
    //    640 / 160, 0.61 at 256 / 64; 47 floats 2.13 / 0.85; 128 bf16 at 1280 / 320 2.15 / 1.16; the R-MAT graph at 64
    //    floats 1.54 at 1024 / 128, 1.40 at 256 / 64).  Only on a matrix of several L2s and a launch that fills the
    //    machine; sparse graphs lose 4-5 % with the lower cut and do not meet the condition.
    const bool fine_wide = elem_bytes == 4 && groups <= 3 && rule_cut == 128 && rule_segment == 32;
    const bool coarse_narrow = groups >= 4 && rule_cut > 256 && (int64_t)n * row_bytes >= 2 * kL2Bytes &&
                               n / groups >= kWavesToFill;
    if (fine_wide || coarse_narrow) {
        int64_t beyond = 0, all = 0, long_rows = 0;
        for (int32_t v = 0; v < n; ++v) {
            all += len_all[v];
            if (len_all[v] > 128) {
                beyond += len_all[v];
                ++long_rows;
            }
        }
        if (beyond * 3 >= all * 2) {
            // how often every row is gathered (every group expanded), then the k most gathered
            int64_t hot = 0;
            const int64_t k = std::min<int64_t>(n, kL2Bytes / std::max<int64_t>(1, row_bytes));
            ivec sorted((size_t)n, 0);
            for (int32_t c : L->res_col) sorted[c]++;
            for (int64_t g = 0; g < G; ++g) {
                const int32_t uses = L->group_dst_ptr[g + 1] - L->group_dst_ptr[g];
                for (int32_t j = L->group_ptr[g]; j < L->group_ptr[g + 1]; ++j) sorted[L->group_col[j]] += uses;
            }
            if (k > 0 && k < n) std::nth_element(sorted.begin(), sorted.begin() + (k - 1), sorted.end(), std::greater<int32_t>());
            for (int64_t i = 0; i < k; ++i) hot += sorted[i];
            const bool popular = hot * 20 >= all * 9;
            if (fine_wide && popular) {
                const bool wide = groups == 1 && row_bytes >= 1024;
                rule_cut = wide ? 256 : 512;
                rule_segment = wide ? 64 : 128;
            } else if (coarse_narrow && !popular && long_rows * 2 >= n) {
                // (only where the typical row is that long: on heavy-tailed graphs, whose median row has a few entries,
                // a lower cut costs 4-7 %)
                rule_cut = 256;
                rule_segment = 64;
            }
        }
    }
    const int32_t hub_split = (o && o->hub_split > 0) ? o->hub_split : rule_cut;
    // (a caller's cut with the library's segment: the rule's share of the rule's cut)
    const int32_t segment = (o && o->segment > 0) ? o->segment
                                                  : std::max<int32_t>(16, (int64_t)hub_split * rule_segment / rule_cut);
    L->hub_split = hub_split;
    L->segment = segment;
    // Small launches (the library's own cut): no row is cut.  The destination-row launch runs workgroups of
    // 16 wavefronts and gives every row of more than kCoopRow entries 4, 8 or 16 of them, which each sum their share
    // of it and combine in LDS: the chain of dependent gathers of a segment without the second launch that
    // segments need (2^14 nodes x 32 floats: two launches of 5-6 us each).  Only while the longest row leaves a lane
    // group at most kCoopChain entries; a longer one is better off spread over the machine in segments.
    bool coop = false;
    if (!(o && (o->hub_split > 0 || o->segment > 0 || o->share_scope == 1)) && n / groups < kWavesToFill) {
        int32_t longest = 0;
        int64_t long_rows = 0;
        for (int32_t v = 0; v < n; ++v) {
            longest = std::max(longest, len_all[v]);
            long_rows += len_all[v] > kCoopRow;
        }
        coop = long_rows > 0 && long_rows <= kCoopMaxRows && longest <= (int64_t)kCoopWaves * groups * kCoopChain;
    }
    const int32_t cut_rows = coop ? INT32_MAX : hub_split;   // rows beyond this are cut into segments
    // Partial rows are cold when the row that adds them up reads them (written one launch earlier, each read once): an
    // entry of that chain costs about twice the cached figure -- and never less than a memory latency (700 ns) shared by
    // the two reads that each of the wavefront's `groups` lane groups keeps in flight, which is what counts at wide
    // rows (bipartite graph, 160 floats, one row of 821 000 entries: 4550 segments made the destination-row launch 1.69
    // ms, 1.6 of it that row's task at 350 ns a segment; 1.19 ms with half as many).
    int64_t max_segments;
    {
        const int64_t edges = L->e_orig > 0 ? L->e_orig : total;
        const int64_t launch_ns = 15000 + edges * row_bytes * 60 / 1000000;
        const int64_t ref_ns = std::max<int64_t>(2 * (10 + row_bytes * 14 / 100), 700 / (2 * groups));
        max_segments = std::max<int64_t>(64, 3 * launch_ns / (4 * ref_ns));
    }
    if (o && (o->share_scope < 0 || o->share_scope > 1)) return ROF_ERR_ARG;
    const bool disable = o && o->disable_reuse;
    const int32_t min_consumers = o ? o->min_consumers : 0;
    const int32_t entry_order = o ? o->entry_order : 0;
    const int64_t tile_rows = (o && o->tile_rows > 0) ? o->tile_rows : kTileRows;

    // node -> groups it consumes (ascending group index)
    ivec ng_ptr((size_t)n + 1, 0), ng;
    for (int64_t j = 0; j < (int64_t)L->group_dst.size(); ++j) ng_ptr[L->group_dst[j] + 1]++;
    for (int32_t v = 0; v < n; ++v) ng_ptr[v + 1] += ng_ptr[v];
    ng.resize(ng_ptr[n]);
    {
        ivec at(ng_ptr.begin(), ng_ptr.end() - 1);
        for (int64_t g = 0; g < G; ++g)
            for (int32_t j = L->group_dst_ptr[g]; j < L->group_dst_ptr[g + 1]; ++j) ng[at[L->group_dst[j]]++] = (int32_t)g;
    }

    // "nearby" = within two tiles of ids, and within a sixteenth of the graph: on a graph of a few tiles every source
    // is within two tiles, which says nothing about locality (R-MAT, 2^14 ... 2^15 nodes: taken for local, whole
    // tiles per XCD run cost 12 ... 25 % against runs of 4; a block model of sixteen 4096-node blocks still gains
    // 23 % from them)
    // (and as far as the rows go that one L2 holds: 16 partners within 32 768 ids on 2^21 nodes at 24 floats, where 4
    // MB are 43 690 rows, run 43 % faster with whole tiles per XCD run than with runs of 4; at 72 floats 9 %)
    const int32_t near_ids = (int32_t)std::max<int64_t>(
        1, std::min<int64_t>(std::max<int64_t>(2 * kTileRows, kL2Bytes / std::max<int64_t>(1, row_bytes)), n / 16));
    // Do the rows gather from their own neighbourhood (35 % of the sources nearby, every group expanded: R-MAT graphs
    // of 2^14 ... 2.4 M nodes measure 6-26 %, a band of 32 768 ids at 288-byte rows 44 %, block models 80-93 %)?
    // Then neighbouring rows share sources through the L2 of the XCD that their tile runs on, and a row that a
    // cluster takes out of the tile order loses that.
    auto sources_are_local = [&]() {
        int64_t near = 0, all = (int64_t)L->res_col.size();
        for (int32_t v = 0; v < n; ++v)
            for (int32_t j = L->res_ptr[v]; j < L->res_ptr[v + 1]; ++j) near += std::abs(L->res_col[j] - v) < near_ids;
        for (int64_t g = 0; g < G; ++g)
            for (int32_t d = L->group_dst_ptr[g]; d < L->group_dst_ptr[g + 1]; ++d)
                for (int32_t j = L->group_ptr[g]; j < L->group_ptr[g + 1]; ++j, ++all)
                    near += std::abs(L->group_col[j] - L->group_dst[d]) < near_ids;
        return all > 0 && near * 20 >= all * 7;
    };

    // Workgroup-local sharing first (cost-model mode only): consumers that the schedule can bring together in one
    // workgroup take the group's sum from LDS; what is decided below for the partial-sum workspace then concerns
    // the remaining consumers only.
    Clusters cl;
    cl.of_node.assign(n, -1);
    const int32_t local_groups = o ? o->local_groups : 0;
    const int32_t share_scope = o ? o->share_scope : 0;
    ivec served(G, 0);   // consumers of each group that read it from LDS
    ivec full_len;       // entries of every destination with every group expanded (only needed where groups exist)
    int64_t over = 0;    // destinations whose task, as cut by hub_split, is a long one
    if (G > 0) {
        full_len.swap(len_all);
        for (int32_t v = 0; v < n; ++v) {
            const int64_t len = full_len[v];
            const int64_t task_len = len > cut_rows ? (len + segment - 1) / segment : len;
            over += task_len > kShortRow;
        }
    }
    // share_scope 1: only rows that will be cut into segments read shared groups from the workspace
    auto in_scope = [&](int32_t v) { return share_scope != 1 || full_len[v] > cut_rows; };
    if (!disable && min_consumers == 0 && local_groups >= 0 && G > 0) {
        // sharing only shortens rows, so a row that is short now stays short, and rows above the segment cut are
        // no candidates
        const int32_t cut = short_cut(n, over, groups);
        // LDS rows per workgroup: 16 KB at the width this layout is built for, at most 31 rows: the widest row any
        // launch can ask for is that of bf16 features at 64 lanes, (64 * 8 + 4) * 4 = 2064 bytes, and 31 of those
        // still fit the 64 KB a workgroup may request (32 would not)
        const int32_t row_bytes = lpr * 16 * ((o && o->elem_bytes == 2) ? 2 : 1);
        const int32_t max_rows = std::max(4, std::min(31, (16 << 10) / row_bytes));
        // (the relative gate protects the tile order, which only graphs with local sources profit from: on graphs
        // without it every cluster that saves kMinClusterSaving gathers pays -- planted sets of 3 anchors x 64 members
        // + 24 random neighbours, 16 % of the gathers removable: 1.056 ms with reuse disabled, 1.082 with the clusters
        // that pass the relative gate, 0.960 with all of them)
        build_clusters(L, ng_ptr, ng, full_len, std::min(cut, cut_rows), groups, max_rows, local_groups > 0 ? local_groups : kMinClusterSaving,
                       local_groups == 0 && sources_are_local(), cl);
        for (int32_t v = 0; v < n; ++v)
            if (cl.of_node[v] >= 0)
                for (int32_t j = cl.ptr[cl.of_node[v]]; j < cl.ptr[cl.of_node[v] + 1]; ++j) served[cl.group[j]]++;
        // what the clusters save: every consumer's copy of a local group's sources but the one the cluster gathers
        int64_t local_saved = -(int64_t)cl.lg_col.size();
        for (int64_t g = 0; g < G; ++g) local_saved += (int64_t)served[g] * (L->group_ptr[g + 1] - L->group_ptr[g]);
        if (local_groups == 0 && local_saved * lpr * 16 < kMinLocalSavedBytes) {   // not worth a launch of their own
            cl = Clusters();
            cl.of_node.assign(n, -1);
            std::fill(served.begin(), served.end(), 0);
        }
    }

    // Which groups are computed once and shared through the workspace.  A group is worth a partial-sum row when the
    // row gathers it saves exceed the partial-row reads plus the one write it adds.
    auto worth = [&](int64_t cnt, int64_t len) {
        if (disable) return false;
        if (min_consumers < 0) return true;   // every group, even one nobody consumes (v1 cache rows)
        if (len <= 0 || cnt <= 0) return false;
        if (min_consumers > 0) return cnt >= min_consumers;
        return (cnt - 1) * len > cnt + 1;
    };
    // consumers of each group that would read it from the workspace
    ivec scoped(G, 0);
    for (int64_t g = 0; g < G; ++g) {
        if (share_scope != 1) {
            scoped[g] = L->group_dst_ptr[g + 1] - L->group_dst_ptr[g] - served[g];
            continue;
        }
        for (int32_t j = L->group_dst_ptr[g]; j < L->group_dst_ptr[g + 1]; ++j) scoped[g] += in_scope(L->group_dst[j]);
    }
    // a plan whose sharing would not repay its extra launch is executed with every group folded back
    int64_t saved = 0;
    for (int64_t g = 0; g < G; ++g) {
        int64_t cnt = scoped[g], len = L->group_ptr[g + 1] - L->group_ptr[g];
        if (worth(cnt, len)) saved += (cnt - 1) * len - cnt;
    }
    const bool too_small = min_consumers == 0 && (saved * lpr * 16 < kMinSavedBytes ||   // a lane holds 16 bytes of a row
                                                  saved * kMinSavedShare < total);
    std::vector<int32_t> slot_of(G, -1);
    int64_t slots = 0;
    TaskList tg, ts, tb;
    for (int64_t g = 0; g < G; ++g) {
        if (too_small) break;
        if (!worth(scoped[g], L->group_ptr[g + 1] - L->group_ptr[g])) continue;
        slot_of[g] = (int32_t)slots++;
        tg.begin_task(slot_of[g]);
        tg.col.insert(tg.col.end(), L->group_col.begin() + L->group_ptr[g], L->group_col.begin() + L->group_ptr[g + 1]);
        tg.end_task(0);
    }
    L->n_materialised = slots;

    tb.ptr.reserve((size_t)n + 1);
    tb.nref.reserve(n);
    tb.out.reserve(n);
    tb.col.reserve(L->res_col.size() + L->group_dst.size());
    int64_t gathered = (int64_t)tg.col.size() + (int64_t)cl.lg_col.size(), reads = 0, segments = 0, nearby = 0, lds_reads = 0;

    ivec row;   // one destination's entries: LDS rows first, then references, then feature rows
    ivec local_row(G, -1);
    for (int32_t v = 0; v < n; ++v) {
        row.clear();
        int32_t refs = 0, nlds = 0;
        if (cl.of_node[v] >= 0)
            for (int32_t j = cl.ptr[cl.of_node[v]]; j < cl.ptr[cl.of_node[v] + 1]; ++j) {
                local_row[cl.group[j]] = cl.row[j];
                row.push_back(cl.row[j]);
                ++nlds;
            }
        const bool reads_workspace = ng_ptr[v + 1] > ng_ptr[v] && in_scope(v);
        for (int32_t j = ng_ptr[v]; j < ng_ptr[v + 1]; ++j)
            if (local_row[ng[j]] < 0 && slot_of[ng[j]] >= 0 && reads_workspace) {
                row.push_back(n + slot_of[ng[j]]);
                ++refs;
            }
        for (int32_t j = ng_ptr[v]; j < ng_ptr[v + 1]; ++j) {
            int32_t g = ng[j];
            if (local_row[g] < 0 && (slot_of[g] < 0 || !reads_workspace))
                row.insert(row.end(), L->group_col.begin() + L->group_ptr[g], L->group_col.begin() + L->group_ptr[g + 1]);
        }
        if (nlds)
            for (int32_t j = cl.ptr[cl.of_node[v]]; j < cl.ptr[cl.of_node[v] + 1]; ++j) local_row[cl.group[j]] = -1;
        row.insert(row.end(), L->res_col.begin() + L->res_ptr[v], L->res_col.begin() + L->res_ptr[v + 1]);
        // The order of the summands is free.  Walking the feature matrix monotonically keeps consecutive
        // gathers of a task close in memory (same pages, neighbouring lines); measured on MI355X against the
        // plan's own order: descending ids 2-3 % faster, ascending 1 % faster, a random order 20 % slower.
        if (entry_order == 0) std::sort(row.begin() + nlds + refs, row.end(), std::greater<int32_t>());
        else if (entry_order == 2) std::sort(row.begin() + nlds + refs, row.end());
        const int64_t len = (int64_t)row.size();
        for (int64_t j = nlds + refs; j < len; ++j) nearby += std::abs(row[j] - v) < near_ids;
        gathered += len - refs - nlds;
        reads += refs;
        lds_reads += nlds;
        tb.begin_task(v);
        if (len > cut_rows) {
            // A long row is cut into segments; each becomes a partial-sum task of the middle launch
            // (after the groups it may reference, before the rows), and the row itself just adds them up.
            // (Rows served from LDS are short: nlds is 0 here.)
            // (a row so long that its segments' partial rows would themselves be the longest chain of the launch
            // gets longer segments: 2^20 nodes with two rows of 2^20 entries at 64 floats, 8192 segments of 128:
            // 0.82 ms, of which the two rows' own tasks last 0.78; 2048 segments of 512: 0.40 ms)
            const int64_t seg_len = std::max<int64_t>(segment, (len + max_segments - 1) / max_segments);
            int32_t nseg = 0;
            for (int64_t s0 = 0; s0 < len; s0 += seg_len) {
                int64_t s1 = std::min<int64_t>(len, s0 + seg_len);
                int32_t slot = (int32_t)slots++;
                ts.begin_task(slot);
                ts.col.insert(ts.col.end(), row.begin() + s0, row.begin() + s1);
                ts.end_task((int32_t)std::max<int64_t>(0, std::min<int64_t>(refs, s1) - s0));
                tb.col.push_back(n + slot);
                ++nseg;
            }
            segments += nseg;
            reads += nseg;
            tb.end_task(nseg);
        } else {
            tb.col.insert(tb.col.end(), row.begin(), row.end());
            tb.end_task(refs, nlds);
        }
    }
    if (slots + (int64_t)n >= INT32_MAX || tb.col.size() >= (size_t)INT32_MAX) return ROF_ERR_UNSUPPORTED;
    // Runs of workgroups per XCD in the destination-row launch.  When rows gather from their own neighbourhood
    // a run covers one whole tile of destinations (a workgroup packs 4 x `groups` short rows), so that the tile's
    // sources are fetched into one L2 only: measured on a block-structured graph of 4096-node blocks, 256
    // workgroups (= one tile at 4 rows per wavefront) are 11 % faster than 64 and 16 % faster than 16.  On
    // graphs without that locality short runs balance the XCDs better (R-MAT, 2.4 M nodes: runs of 4 were 0-2 %
    // faster than 16 at every width from 16 to 100 floats on two devices and equal on a third, 1 and 2 are 0.9 %
    // slower than 4, 64 is 1-6 % slower; smaller graphs measure alike from 2 to 16).
    // (at least 256 workgroups: at five rows per wavefront and more a tile is fewer, and runs of 256 measure the same
    // on block models and 6 % faster on a graph whose sources lie in a band around the row)
    const int64_t tile_run = std::max<int64_t>(256, std::min<int64_t>(1024, tile_rows / (4 * groups)));
    L->local_sources = gathered > 0 && nearby * 20 >= gathered * 7;
    L->xcd_run = L->local_sources ? (int32_t)tile_run : 4;
    L->n_slots = slots;
    L->n_segments = segments;
    L->gathered_rows = gathered;
    L->partial_reads = reads;
    finalize_phase(tg, 1 << 30, groups, false, L->g);
    finalize_phase(ts, 1 << 30, groups, entry_order == 0, L->s);   // the sweep needs the descending lists
    finalize_phase(tb, tile_rows, groups, false, L->b, &cl);
    L->coop_tasks = L->coop16 = L->coop8 = 0;
    if (coop)   // the long tasks come first, longest first
        while (L->coop_tasks < L->b.n_wave && L->b.task_ptr[L->coop_tasks + 1] - L->b.task_ptr[L->coop_tasks] > kCoopRow) {
            const int32_t len = L->b.task_ptr[L->coop_tasks + 1] - L->b.task_ptr[L->coop_tasks];
            L->coop16 += len > kCoopRow16;
            L->coop8 += len > kCoopRow8 && len <= kCoopRow16;
            ++L->coop_tasks;
        }
    L->n_local_groups = (int64_t)cl.lg_task_ptr.size() - 1;
    L->lds_reads = lds_reads;
    L->gathered_before_rows = (int64_t)tg.col.size();
    for (size_t t = 0; t < ts.out.size(); ++t) L->gathered_before_rows += (ts.ptr[t + 1] - ts.ptr[t]) - ts.nref[t];
    return ROF_OK;
}

std::unique_ptr<rof_layout> new_layout(int32_t n, int ps) {
    std::unique_ptr<rof_layout> L(new (std::nothrow) rof_layout);
    if (!L) return nullptr;
    L->n = n;
    L->part_size = ps;
    return L;
}

// Build the canonical arrays from "unique parts": part w has sources src[sptr[w]..sptr[w+1]) and
// consumers dcol[dptr[w]..dptr[w+1]).
void canonical_from_unique(rof_layout *L, const int32_t *src, const int32_t *sptr, const int32_t *dptr,
                           const int32_t *dcol, int64_t U) {
    const int32_t n = L->n;
    L->group_ptr.assign(1, 0);
    L->group_dst_ptr.assign(1, 0);
    L->res_ptr.assign((size_t)n + 1, 0);
    int64_t e = 0;
    for (int64_t w = 0; w < U; ++w) {
        int32_t cnt = dptr[w + 1] - dptr[w], len = sptr[w + 1] - sptr[w];
        e += (int64_t)cnt * len;
        if (cnt >= 2) {
            L->group_col.insert(L->group_col.end(), src + sptr[w], src + sptr[w + 1]);
            L->group_ptr.push_back((int32_t)L->group_col.size());
            L->group_dst.insert(L->group_dst.end(), dcol + dptr[w], dcol + dptr[w + 1]);
            L->group_dst_ptr.push_back((int32_t)L->group_dst.size());
        } else if (cnt == 1) {
            L->res_ptr[dcol[dptr[w]] + 1] += len;
        }
    }
    L->e_orig = e;
    for (int32_t v = 0; v < n; ++v) L->res_ptr[v + 1] += L->res_ptr[v];
    L->res_col.resize(L->res_ptr[n]);
    ivec at(L->res_ptr.begin(), L->res_ptr.end() - 1);
    for (int64_t w = 0; w < U; ++w) {
        if (dptr[w + 1] - dptr[w] != 1) continue;
        int32_t v = dcol[dptr[w]], len = sptr[w + 1] - sptr[w];
        if (len) memcpy(L->res_col.data() + at[v], src + sptr[w], (size_t)len * sizeof(int32_t));
        at[v] += len;
    }
}

// Takes ownership: the layout is released on every path that does not hand it to the caller, including
// an allocation failure thrown while the schedule is built.
int finish(std::unique_ptr<rof_layout> L, const rof_layout_opts *opts, rof_layout **out) {
    int st = build_schedule(L.get(), opts);
    if (st) return st;
    *out = L.release();
    return ROF_OK;
}

}  // namespace

extern "C" {

int rof_layout_from_v2(const int32_t *ucol, const int32_t *uptr, const int32_t *dptr, const int32_t *dcol,
                       int64_t U, int32_t n, int part_size, const rof_layout_opts *opts, rof_layout **out) {
    if (!out || !uptr || !dptr || U < 0 || n < 0 || part_size < 1) return ROF_ERR_ARG;
    int64_t ne = 0, nd = 0;
    if (!ptr_ok(uptr, U, &ne) || !ptr_ok(dptr, U, &nd)) return ROF_ERR_RANGE;
    if ((ne && !ucol) || (nd && !dcol)) return ROF_ERR_ARG;
    if (!ids_ok(ucol, ne, n) || !ids_ok(dcol, nd, n)) return ROF_ERR_RANGE;
    try {
        std::unique_ptr<rof_layout> L = new_layout(n, part_size);
        if (!L) return ROF_ERR_ALLOC;
        canonical_from_unique(L.get(), ucol, uptr, dptr, dcol, U);
        int64_t G = (int64_t)L->group_ptr.size() - 1;
        bool groups_first = true;
        for (int64_t w = 0; w < U && groups_first; ++w) {
            int32_t cnt = dptr[w + 1] - dptr[w];
            if ((w < G) != (cnt >= 2) || cnt == 0) groups_first = false;
        }
        L->canonical = groups_first && v2_is_canonical(uptr, dptr, dcol, U, part_size, G);
        return finish(std::move(L), opts, out);
    } catch (const std::bad_alloc &) {
        return ROF_ERR_ALLOC;
    }
}

int rof_layout_from_v1(const int32_t *col, const int32_t *pptr, const int32_t *p2n, int64_t parts, const int32_t *flag,
                       const int32_t *cptr, const int32_t *ccol, int64_t cache_num, int32_t n, int part_size,
                       const rof_layout_opts *opts, rof_layout **out) {
    if (!out || !pptr || !cptr || parts < 0 || cache_num < 0 || n < 0 || part_size < 1) return ROF_ERR_ARG;
    if (parts && (!p2n || !flag)) return ROF_ERR_ARG;
    int64_t ne = 0, nc = 0;
    if (!ptr_ok(pptr, parts, &ne) || !ptr_ok(cptr, cache_num, &nc)) return ROF_ERR_RANGE;
    if ((ne && !col) || (nc && !ccol)) return ROF_ERR_ARG;
    if (!ids_ok(col, ne, n) || !ids_ok(ccol, nc, n) || !ids_ok(p2n, parts, n)) return ROF_ERR_RANGE;
    if (!ids_ok(flag, parts, cache_num + 1)) return ROF_ERR_RANGE;
    try {
        std::unique_ptr<rof_layout> L = new_layout(n, part_size);
        if (!L) return ROF_ERR_ALLOC;
        // groups = cache rows (reuse_conv_kernel.cu:431-440); consumers = nodes of the flagged parts
        // (cu:523-531), which come in ascending node order because part2Node is non-decreasing
        L->group_ptr.assign(cptr, cptr + cache_num + 1);
        L->group_col.assign(ccol, ccol + nc);
        L->group_dst_ptr.assign((size_t)cache_num + 1, 0);
        L->res_ptr.assign((size_t)n + 1, 0);
        int64_t e = 0;
        for (int64_t p = 0; p < parts; ++p) {
            if (flag[p] > 0) {
                L->group_dst_ptr[flag[p]]++;
                e += cptr[flag[p]] - cptr[flag[p] - 1];
            } else {
                L->res_ptr[p2n[p] + 1] += pptr[p + 1] - pptr[p];
                e += pptr[p + 1] - pptr[p];
            }
        }
        L->e_orig = e;
        for (int64_t g = 0; g < cache_num; ++g) L->group_dst_ptr[g + 1] += L->group_dst_ptr[g];
        for (int32_t v = 0; v < n; ++v) L->res_ptr[v + 1] += L->res_ptr[v];
        L->group_dst.resize(L->group_dst_ptr[cache_num]);
        L->res_col.resize(L->res_ptr[n]);
        ivec gat(L->group_dst_ptr.begin(), L->group_dst_ptr.end() - 1), rat(L->res_ptr.begin(), L->res_ptr.end() - 1);
        for (int64_t p = 0; p < parts; ++p) {
            if (flag[p] > 0) {
                L->group_dst[gat[flag[p] - 1]++] = p2n[p];
            } else {
                int32_t len = pptr[p + 1] - pptr[p];
                if (len) memcpy(L->res_col.data() + rat[p2n[p]], col + pptr[p], (size_t)len * sizeof(int32_t));
                rat[p2n[p]] += len;
            }
        }
        bool ok = true;   // canonical iff every cache row has >= 2 consumers
        for (int64_t g = 0; g < cache_num; ++g)
            if (L->group_dst_ptr[g + 1] - L->group_dst_ptr[g] < 2) ok = false;
        L->canonical = ok;
        return finish(std::move(L), opts, out);
    } catch (const std::bad_alloc &) {
        return ROF_ERR_ALLOC;
    }
}

int rof_layout_from_parts(const int32_t *col, const int32_t *pptr, const int32_t *p2n, int64_t parts, int32_t n,
                          int part_size, const rof_layout_opts *opts, rof_layout **out) {
    if (!out || !pptr || parts < 0 || n < 0 || part_size < 1 || (parts && !p2n)) return ROF_ERR_ARG;
    int64_t ne = 0;
    if (!ptr_ok(pptr, parts, &ne)) return ROF_ERR_RANGE;
    if (ne && !col) return ROF_ERR_ARG;
    if (!ids_ok(col, ne, n) || !ids_ok(p2n, parts, n)) return ROF_ERR_RANGE;
    try {
        std::unique_ptr<rof_layout> L = new_layout(n, part_size);
        if (!L) return ROF_ERR_ALLOC;
        L->group_ptr.assign(1, 0);
        L->group_dst_ptr.assign(1, 0);
        L->res_ptr.assign((size_t)n + 1, 0);
        for (int64_t p = 0; p < parts; ++p) L->res_ptr[p2n[p] + 1] += pptr[p + 1] - pptr[p];
        for (int32_t v = 0; v < n; ++v) L->res_ptr[v + 1] += L->res_ptr[v];
        L->res_col.resize(L->res_ptr[n]);
        ivec at(L->res_ptr.begin(), L->res_ptr.end() - 1);
        for (int64_t p = 0; p < parts; ++p) {
            int32_t len = pptr[p + 1] - pptr[p];
            if (len) memcpy(L->res_col.data() + at[p2n[p]], col + pptr[p], (size_t)len * sizeof(int32_t));
            at[p2n[p]] += len;
        }
        L->e_orig = ne;
        L->canonical = true;
        return finish(std::move(L), opts, out);
    } catch (const std::bad_alloc &) {
        return ROF_ERR_ALLOC;
    }
}

int rof_layout_export(const rof_layout *L, rof_bag **out) {
    if (!L || !out) return ROF_ERR_ARG;
    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        auto put = [bag](const char *name, const ivec &v) {
            auto &d = bag->arr[name];
            d.resize(v.size());
            if (!v.empty()) memcpy(d.data(), v.data(), v.size() * sizeof(int32_t));
        };
        put("group_ptr", L->group_ptr);
        put("group_col", L->group_col);
        put("group_dst_ptr", L->group_dst_ptr);
        put("group_dst", L->group_dst);
        put("res_ptr", L->res_ptr);
        put("res_col", L->res_col);
        bag->arr["canonical"].assign(1, L->canonical ? 1u : 0u);
        bag->arr["xcd_run"].assign(1, (uint32_t)L->xcd_run);
        bag->arr["long_row_cut"] = {(uint32_t)L->hub_split, (uint32_t)L->segment};   // as chosen for this layout
        // v2 tensors: groups first, then every node's residual list re-chunked by part_size
        // (reuse_search_ext.h:537-636)
        const int ps = L->part_size;
        int64_t G = (int64_t)L->group_ptr.size() - 1;
        auto &ucol = bag->arr["uniqpart_column_index"], &uptr = bag->arr["uniqpart_pointers"];
        auto &dptr = bag->arr["part2Node_ptr"], &dcol = bag->arr["part2Node_col"];
        ucol.assign(L->group_col.begin(), L->group_col.end());
        ucol.insert(ucol.end(), L->res_col.begin(), L->res_col.end());
        uptr.assign(L->group_ptr.begin(), L->group_ptr.end());
        dptr.assign(L->group_dst_ptr.begin(), L->group_dst_ptr.end());
        dcol.assign(L->group_dst.begin(), L->group_dst.end());
        uint32_t base = (uint32_t)L->group_col.size();
        for (int32_t v = 0; v < L->n; ++v) {
            int32_t beg = L->res_ptr[v], end = L->res_ptr[v + 1];
            for (int32_t q = beg; q < end; q += ps) {
                uptr.push_back(base + (uint32_t)std::min(q + ps, end));
                dcol.push_back((uint32_t)v);
                dptr.push_back((uint32_t)dcol.size());
            }
        }
        (void)G;
        // schedule, for inspection and host-side tests
        put("g_task_ptr", L->g.task_ptr);
        put("g_task_nref", L->g.task_nref);
        put("g_task_out", L->g.task_out);
        put("g_col", L->g.col);
        put("s_task_ptr", L->s.task_ptr);
        put("s_task_nref", L->s.task_nref);
        put("s_task_out", L->s.task_out);
        put("s_col", L->s.col);
        put("b_task_ptr", L->b.task_ptr);
        put("b_task_nref", L->b.task_nref);
        put("b_task_out", L->b.task_out);
        put("b_col", L->b.col);
        put("b_task_nlds", L->b.task_nlds);
        put("b_lg_ptr", L->b.lg_ptr);
        put("b_lg_task_ptr", L->b.lg_task_ptr);
        put("b_lg_col", L->b.lg_col);
        put("b_lg_task_first", L->b.lg_task_first);
        bag->arr["b_shape"] = {(uint32_t)L->b.n_wave, (uint32_t)L->b.n_regular, (uint32_t)L->b.lg_blocks,
                               (uint32_t)L->b.lg_max_rows};
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

int rof_layout_stats_n(const rof_layout *L, int64_t *stats, int count) {
    if (!L || !stats || count < 0) return ROF_ERR_ARG;
    int64_t s[24];
    int rc = rof_layout_stats(L, s);
    if (rc) return rc;
    s[20] = L->hub_split;
    s[21] = L->segment;
    s[22] = 0;   // longest task of the destination-row launch
    for (int32_t t = 0; t < L->b.n_tasks; ++t) s[22] = std::max<int64_t>(s[22], L->b.task_ptr[t + 1] - L->b.task_ptr[t]);
    s[23] = L->coop_tasks;
    for (int i = 0; i < count; ++i) stats[i] = i < 24 ? s[i] : 0;
    return ROF_OK;
}

int rof_layout_stats(const rof_layout *L, int64_t s[20]) {
    if (!L || !s) return ROF_ERR_ARG;
    memset(s, 0, 20 * sizeof(int64_t));
    s[0] = L->n;
    s[1] = L->e_orig;
    s[2] = (int64_t)L->group_ptr.size() - 1;
    s[3] = L->n_materialised;
    s[4] = L->gathered_rows;
    s[5] = L->partial_reads;
    s[6] = L->n_slots;
    s[7] = L->n_segments;
    s[8] = L->g.n_tasks + L->s.n_tasks;
    s[9] = L->b.n_tasks;
    s[10] = L->device_bytes;
    s[11] = L->part_size;
    s[12] = L->g.n_wave + L->s.n_wave;
    s[13] = L->b.n_wave;
    s[14] = L->canonical ? 1 : 0;
    s[15] = L->gathered_before_rows;
    s[16] = L->n_local_groups;
    s[17] = L->lds_reads;
    s[18] = L->b.lg_blocks;
    s[19] = L->b.lg_blocks > 0 ? L->b.lg_max_rows : 0;
    return ROF_OK;
}

}  // extern "C"
