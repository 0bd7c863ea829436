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
// Long rows.  Rows longer than a cut are gathered in segments that fill partial rows one launch earlier, and
// the segment tasks of all rows run in the order of the highest source id they gather (entries inside a task are
// listed by descending id): every wavefront in flight then works in the same narrow band of the feature matrix
// and the launch sweeps the matrix once from top to bottom, so a row gathered for one destination is still in
// L2 when the next destinations need it.  The effect is large -- rotating each row's list by a random offset,
// which keeps every task monotone but puts the tasks out of phase, costs 25 % on the 2.4 M-node workload -- and
// it is why the cut is low: measured optima with G rows per wavefront are cut / segment = 96-128 / 32 at G = 1
// (-12 % against a cut of 1024), 256 / 64 at G = 2 (-18 % against 8192), 640-1024 / 160 at G = 5 (-7 % against
// 5457).  Every segment writes and re-reads one partial row (fp32, so twice a gathered row when those are bf16),
// which is what stops finer cuts: at G = 2 the best cut is 128 / 32 for fp32 rows (-10 % against 256 / 64) and
// 256 / 64 for bf16 rows; at G = 4 256-512; at G = 8 and 16 640-1024 (256 is 10-30 % slower there).
// (Giving long rows a whole workgroup instead -- four wavefronts combined through LDS -- was measured as well:
// no faster than segments on any workload, so it is not built in.)
int32_t default_cut(int32_t groups, int32_t elem_bytes) {
    const int32_t cut = groups <= 2 ? 128 : groups == 3 ? 256 : groups == 4 ? 384 : 640;
    return std::min(640, elem_bytes == 2 ? 2 * cut : cut);
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
    ivec ptr{0}, nref, out, col;
    void begin_task(int32_t out_row) { out.push_back(out_row); }
    void end_task(int32_t refs) {
        nref.push_back(refs);
        ptr.push_back((int32_t)col.size());
    }
};

// Long tasks first (descending), then short tasks tile by tile, each tile descending.  `groups`: short tasks
// that share a wavefront.  With `band` (one key per task: the highest source id it gathers) both kinds are
// ordered by descending key instead.
void order_tasks(const ivec &ptr, int64_t tile_rows, int32_t groups, const ivec *band, ivec &order, int32_t &n_wave) {
    int64_t T = (int64_t)ptr.size() - 1;
    order.clear();
    order.reserve(T);
    int64_t over = 0;
    for (int64_t t = 0; t < T; ++t) over += ptr[t + 1] - ptr[t] > kShortRow;
    const int32_t cut = over + (T - over + groups - 1) / groups >= kWavesToFill ? kShortRow : kShortRowSmall;
    ivec longs;
    for (int64_t t = 0; t < T; ++t)
        if (ptr[t + 1] - ptr[t] > cut) longs.push_back((int32_t)t);
    if (band && cut == kShortRow) {   // a launch too small to fill the machine keeps the longest-first order
        ivec shorts;
        for (int64_t t = 0; t < T; ++t)
            if (ptr[t + 1] - ptr[t] <= cut) shorts.push_back((int32_t)t);
        auto higher = [band](int32_t x, int32_t y) { return (*band)[x] > (*band)[y]; };
        std::stable_sort(longs.begin(), longs.end(), higher);
        std::stable_sort(shorts.begin(), shorts.end(), higher);
        n_wave = (int32_t)longs.size();
        order = longs;
        order.insert(order.end(), shorts.begin(), shorts.end());
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
            if (len <= cut) bucket[len].push_back((int32_t)t);
        }
        for (int32_t len = cut; len >= 0; --len) order.insert(order.end(), bucket[len].begin(), bucket[len].end());
    }
}

void finalize_phase(const TaskList &tl, int64_t tile_rows, int32_t groups, bool by_band, rof_phase_host &ph) {
    int64_t T = (int64_t)tl.out.size();
    ivec order, band;
    if (by_band) {
        band.resize(T);
        for (int64_t t = 0; t < T; ++t) {
            const int32_t first = tl.ptr[t] + tl.nref[t];   // feature rows follow the partial-row references
            band[t] = first < tl.ptr[t + 1] ? tl.col[first] : -1;
        }
    }
    order_tasks(tl.ptr, tile_rows, groups, by_band ? &band : nullptr, order, ph.n_wave);
    ph.n_tasks = (int32_t)T;
    ph.task_ptr.assign(T + 1, 0);
    ph.task_nref.resize(T);
    ph.task_out.resize(T);
    for (int64_t i = 0; i < T; ++i) {
        int32_t t = order[i];
        ph.task_ptr[i + 1] = ph.task_ptr[i] + (tl.ptr[t + 1] - tl.ptr[t]);
        ph.task_nref[i] = tl.nref[t];
        ph.task_out[i] = tl.out[t];
    }
    ph.col.resize(tl.col.size());
#pragma omp parallel for schedule(dynamic, 4096)
    for (int64_t i = 0; i < T; ++i) {
        int32_t t = order[i];
        int32_t len = tl.ptr[t + 1] - tl.ptr[t];
        if (len) memcpy(ph.col.data() + ph.task_ptr[i], tl.col.data() + tl.ptr[t], (size_t)len * sizeof(int32_t));
    }
}

int build_schedule(rof_layout *L, const rof_layout_opts *o) {
    const int32_t n = L->n;
    const int64_t G = (int64_t)L->group_ptr.size() - 1;
    int32_t lpr = (o && o->lanes_per_row > 0) ? o->lanes_per_row : 16;
    if (lpr > 64) lpr = 64;
    const int32_t groups = std::max(1, 64 / lpr);
    const int64_t total = (int64_t)L->res_col.size() + (int64_t)L->group_dst.size();
    const int32_t hub_split = (o && o->hub_split > 0) ? o->hub_split : default_cut(groups, o ? o->elem_bytes : 4);
    const int32_t segment = (o && o->segment > 0) ? o->segment : std::max(16, hub_split / 4);
    L->hub_split = hub_split;
    L->segment = segment;
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

    // Which groups are computed once and shared.  A group is worth a partial-sum row when the row
    // gathers it saves exceed the partial-row reads plus the one write it adds.
    auto worth = [&](int64_t cnt, int64_t len) {
        if (disable) return false;
        if (min_consumers < 0) return true;   // every group, even one nobody consumes (v1 cache rows)
        if (len <= 0 || cnt <= 0) return false;
        if (min_consumers > 0) return cnt >= min_consumers;
        return (cnt - 1) * len > cnt + 1;
    };
    // a plan whose sharing would not repay its extra launch is executed with every group folded back
    int64_t saved = 0;
    for (int64_t g = 0; g < G; ++g) {
        int64_t cnt = L->group_dst_ptr[g + 1] - L->group_dst_ptr[g], len = L->group_ptr[g + 1] - L->group_ptr[g];
        if (worth(cnt, len)) saved += (cnt - 1) * len - cnt;
    }
    const bool too_small = min_consumers == 0 && (saved * lpr * 16 < kMinSavedBytes ||   // a lane holds 16 bytes of a row
                                                  saved * kMinSavedShare < total);
    std::vector<int32_t> slot_of(G, -1);
    int64_t slots = 0;
    TaskList tg, ts, tb;
    for (int64_t g = 0; g < G; ++g) {
        if (too_small) break;
        if (!worth(L->group_dst_ptr[g + 1] - L->group_dst_ptr[g], L->group_ptr[g + 1] - L->group_ptr[g])) continue;
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
    int64_t gathered = (int64_t)tg.col.size(), reads = 0, segments = 0, nearby = 0;
    ivec row;   // one destination's entries: references first, then feature rows
    for (int32_t v = 0; v < n; ++v) {
        row.clear();
        int32_t refs = 0;
        for (int32_t j = ng_ptr[v]; j < ng_ptr[v + 1]; ++j)
            if (slot_of[ng[j]] >= 0) {
                row.push_back(n + slot_of[ng[j]]);
                ++refs;
            }
        for (int32_t j = ng_ptr[v]; j < ng_ptr[v + 1]; ++j) {
            int32_t g = ng[j];
            if (slot_of[g] < 0)
                row.insert(row.end(), L->group_col.begin() + L->group_ptr[g], L->group_col.begin() + L->group_ptr[g + 1]);
        }
        row.insert(row.end(), L->res_col.begin() + L->res_ptr[v], L->res_col.begin() + L->res_ptr[v + 1]);
        // The order of the summands is free.  Walking the feature matrix monotonically keeps consecutive
        // gathers of a task close in memory (same pages, neighbouring lines); measured on MI355X against the
        // plan's own order: descending ids 2-3 % faster, ascending 1 % faster, a random order 20 % slower.
        if (entry_order == 0) std::sort(row.begin() + refs, row.end(), std::greater<int32_t>());
        else if (entry_order == 2) std::sort(row.begin() + refs, row.end());
        const int64_t len = (int64_t)row.size();
        for (int64_t j = refs; j < len; ++j) nearby += std::abs(row[j] - v) < 2 * kTileRows;
        gathered += len - refs;
        reads += refs;
        tb.begin_task(v);
        if (len > hub_split) {
            // A long row is cut into segments; each becomes a partial-sum task of the middle launch
            // (after the groups it may reference, before the rows), and the row itself just adds them up.
            int32_t nseg = 0;
            for (int64_t s0 = 0; s0 < len; s0 += segment) {
                int64_t s1 = std::min<int64_t>(len, s0 + segment);
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
            tb.end_task(refs);
        }
    }
    if (slots + (int64_t)n >= INT32_MAX || tb.col.size() >= (size_t)INT32_MAX) return ROF_ERR_UNSUPPORTED;
    // Runs of workgroups per XCD in the destination-row launch.  When rows gather from their own neighbourhood
    // a run covers one whole tile of destinations (a workgroup packs 4 x `groups` short rows), so that the tile's
    // sources are fetched into one L2 only: measured on a block-structured graph of 4096-node blocks, 256
    // workgroups (= one tile at 4 rows per wavefront) are 11 % faster than 64 and 16 % faster than 16.  On
    // graphs without that locality short runs balance the XCDs better (R-MAT: 16 is 2-6 % faster than 64, and
    // 1..16 measure alike).
    const int64_t tile_run = std::max<int64_t>(16, std::min<int64_t>(1024, tile_rows / (4 * groups)));
    L->xcd_run = (gathered > 0 && nearby * 2 >= gathered) ? (int32_t)tile_run : 16;
    L->n_slots = slots;
    L->n_segments = segments;
    L->gathered_rows = gathered;
    L->partial_reads = reads;
    finalize_phase(tg, 1 << 30, groups, false, L->g);
    finalize_phase(ts, 1 << 30, groups, entry_order == 0, L->s);   // the sweep needs the descending lists
    finalize_phase(tb, tile_rows, groups, false, L->b);
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
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

int rof_layout_stats(const rof_layout *L, int64_t s[16]) {
    if (!L || !s) return ROF_ERR_ARG;
    memset(s, 0, 16 * sizeof(int64_t));
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
    return ROF_OK;
}

}  // extern "C"
