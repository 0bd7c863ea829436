// CPU reuse-plan builder (OpenMP).  Produces, bit for bit, the arrays of the upstream builder
// (ROF/reuse_search_ext/src/reuse_search_ext.h) but is organised for graphs with tens of millions
// of edges and heavy-tailed degrees:
//   * intersections are driven by the shortest source list and gallop through the longer ones;
//     chunks whose sources are all hubs are de-duplicated first, so each distinct hub tuple is
//     intersected once;
//   * only the counts are kept for all chunks; the lists are built for picked chunks only;
//   * the row permutation is done per destination row, rows in parallel, with a position table
//     for long rows instead of a linear search per moved element.
// The one place where the output depends on library behaviour is the order of equal counts left
// by std::sort (h:260-264); the same call on the same element type is made here.
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstring>
#include <map>
#include <numeric>
#include <string>
#include <vector>
#include <omp.h>

#include "rof.h"
#include "rof_internal.h"

namespace {

typedef uint32_t u32;
typedef uint64_t u64;
typedef std::vector<u32> vec;

// ---------------------------------------------------------------------------------------------
// out-neighbour lists, guaranteed ascending and duplicate-free (std::set semantics of h:194,204)
struct OutLists {
    const u32 *ptr;
    const u32 *idx;
    vec own_ptr, own_idx;   // used only when the caller's rows were not already sorted-unique
};

void prepare_out_lists(const u32 *indptr_src, const u32 *indices_dst, u32 n, OutLists &g) {
    bool sorted = true;
#pragma omp parallel for schedule(static) reduction(&& : sorted)
    for (int64_t v = 0; v < (int64_t)n; ++v) {
        for (u32 k = indptr_src[v] + 1; k < indptr_src[v + 1]; ++k)
            if (indices_dst[k - 1] >= indices_dst[k]) sorted = false;
    }
    if (sorted) {
        g.ptr = indptr_src;
        g.idx = indices_dst;
        return;
    }
    std::vector<vec> rows(n);
#pragma omp parallel for schedule(dynamic, 1024)
    for (int64_t v = 0; v < (int64_t)n; ++v) {
        vec &r = rows[v];
        r.assign(indices_dst + indptr_src[v], indices_dst + indptr_src[v + 1]);
        std::sort(r.begin(), r.end());
        r.erase(std::unique(r.begin(), r.end()), r.end());
    }
    g.own_ptr.assign(n + 1, 0);
    for (u32 v = 0; v < n; ++v) g.own_ptr[v + 1] = g.own_ptr[v] + (u32)rows[v].size();
    g.own_idx.resize(g.own_ptr[n]);
#pragma omp parallel for schedule(dynamic, 1024)
    for (int64_t v = 0; v < (int64_t)n; ++v)
        if (!rows[v].empty()) memcpy(g.own_idx.data() + g.own_ptr[v], rows[v].data(), rows[v].size() * sizeof(u32));
    g.ptr = g.own_ptr.data();
    g.idx = g.own_idx.data();
}

// first element >= key in the ascending range [lo, hi), probing exponentially from lo
inline const u32 *gallop(const u32 *lo, const u32 *hi, u32 key) {
    if (lo == hi || *lo >= key) return lo;
    size_t step = 1;
    const u32 *p = lo;
    while (p + step < hi && p[step] < key) {
        p += step;
        step <<= 1;
    }
    const u32 *stop = (p + step < hi) ? p + step + 1 : hi;
    return std::lower_bound(p + 1, stop, key);
}

// Intersection of the out-lists of srcs[0..k).  Returns the size; fills `res` (ascending) if asked.
// `a`, `b` are scratch.
size_t intersect_sources(const OutLists &g, const u32 *srcs, int k, vec *res, vec &a, vec &b) {
    if (k <= 0) {
        if (res) res->clear();
        return 0;
    }
    // order the sources by list length, shortest first (the set being intersected is order-free)
    u32 order_small[16];
    vec order_big;
    u32 *order = order_small;
    if (k > 16) {
        order_big.resize(k);
        order = order_big.data();
    }
    for (int i = 0; i < k; ++i) order[i] = srcs[i];
    std::sort(order, order + k, [&g](u32 x, u32 y) {
        u32 dx = g.ptr[x + 1] - g.ptr[x], dy = g.ptr[y + 1] - g.ptr[y];
        return dx < dy || (dx == dy && x < y);
    });
    const u32 *cur = g.idx + g.ptr[order[0]];
    size_t cur_n = g.ptr[order[0] + 1] - g.ptr[order[0]];
    vec *dst = &a, *spare = &b;
    for (int i = 1; i < k && cur_n; ++i) {
        if (order[i] == order[i - 1]) continue;
        const u32 *lo = g.idx + g.ptr[order[i]];
        const u32 *hi = g.idx + g.ptr[order[i] + 1];
        dst->clear();
        for (size_t j = 0; j < cur_n; ++j) {
            lo = gallop(lo, hi, cur[j]);
            if (lo == hi) break;
            if (*lo == cur[j]) dst->push_back(cur[j]);
        }
        cur = dst->data();
        cur_n = dst->size();
        std::swap(dst, spare);
    }
    if (res) res->assign(cur, cur + cur_n);
    return cur_n;
}

inline bool part_is_skipped(u32 beg, u32 end, int ps, bool discard) {
    return end <= beg || (discard && (int)(end - beg) != ps);   // h:177-181
}

// Chunks whose cheapest source has at least this many out-neighbours are de-duplicated by source
// tuple before intersecting.
const u32 kHubTuple = 256;

void intersect_counts(const u32 *part_ptr, u64 parts, const u32 *indices_src, const OutLists &g, int ps, bool discard,
                      vec &cnt) {
    cnt.assign(parts, 0);
    std::vector<u32> heavy;   // chunk ids postponed for de-duplication
    {
        std::vector<std::vector<u32>> heavy_t(omp_get_max_threads());
#pragma omp parallel
        {
            vec a, b;
            std::vector<u32> &mine = heavy_t[omp_get_thread_num()];
#pragma omp for schedule(dynamic, 4096)
            for (int64_t p = 0; p < (int64_t)parts; ++p) {
                u32 beg = part_ptr[p], end = part_ptr[p + 1];
                if (part_is_skipped(beg, end, ps, discard)) continue;
                u32 mind = UINT32_MAX;
                for (u32 k = beg; k < end; ++k) {
                    u32 s = indices_src[k];
                    mind = std::min(mind, g.ptr[s + 1] - g.ptr[s]);
                }
                if (mind >= kHubTuple && end - beg > 1) {
                    mine.push_back((u32)p);
                    continue;
                }
                cnt[p] = (u32)intersect_sources(g, indices_src + beg, (int)(end - beg), nullptr, a, b);
            }
        }
        for (auto &v : heavy_t) heavy.insert(heavy.end(), v.begin(), v.end());
    }
    if (heavy.empty()) return;
    auto tuple_less = [&](u32 p, u32 q) {
        u32 lp = part_ptr[p + 1] - part_ptr[p], lq = part_ptr[q + 1] - part_ptr[q];
        if (lp != lq) return lp < lq;
        int c = memcmp(indices_src + part_ptr[p], indices_src + part_ptr[q], lp * sizeof(u32));
        return c < 0 || (c == 0 && p < q);
    };
    auto tuple_equal = [&](u32 p, u32 q) {
        u32 lp = part_ptr[p + 1] - part_ptr[p], lq = part_ptr[q + 1] - part_ptr[q];
        return lp == lq && memcmp(indices_src + part_ptr[p], indices_src + part_ptr[q], lp * sizeof(u32)) == 0;
    };
    std::sort(heavy.begin(), heavy.end(), tuple_less);
    std::vector<u32> heads;   // positions in `heavy` where a new tuple starts
    for (size_t i = 0; i < heavy.size(); ++i)
        if (i == 0 || !tuple_equal(heavy[i - 1], heavy[i])) heads.push_back((u32)i);
    heads.push_back((u32)heavy.size());
#pragma omp parallel
    {
        vec a, b;
#pragma omp for schedule(dynamic, 16)
        for (int64_t h = 0; h < (int64_t)heads.size() - 1; ++h) {
            u32 p = heavy[heads[h]];
            u32 c = (u32)intersect_sources(g, indices_src + part_ptr[p], (int)(part_ptr[p + 1] - part_ptr[p]), nullptr,
                                           a, b);
            for (u32 i = heads[h]; i < heads[h + 1]; ++i) cnt[heavy[i]] = c;
        }
    }
}

void intersect_lists(const u32 *part_ptr, const u32 *indices_src, const OutLists &g, int ps, bool discard,
                     const u32 *which, u64 n_which, vec &out_ptr, vec &out_data) {
    std::vector<vec> lists(n_which);
#pragma omp parallel
    {
        vec a, b;
#pragma omp for schedule(dynamic, 64)
        for (int64_t i = 0; i < (int64_t)n_which; ++i) {
            u32 p = which[i];
            u32 beg = part_ptr[p], end = part_ptr[p + 1];
            if (part_is_skipped(beg, end, ps, discard)) continue;
            intersect_sources(g, indices_src + beg, (int)(end - beg), &lists[i], a, b);
        }
    }
    out_ptr.assign(n_which + 1, 0);
    for (u64 i = 0; i < n_which; ++i) out_ptr[i + 1] = out_ptr[i] + (u32)lists[i].size();
    out_data.resize(out_ptr[n_which]);
#pragma omp parallel for schedule(dynamic, 256)
    for (int64_t i = 0; i < (int64_t)n_which; ++i)
        if (!lists[i].empty()) memcpy(out_data.data() + out_ptr[i], lists[i].data(), lists[i].size() * sizeof(u32));
}

// ---------------------------------------------------------------------------------------------
void split_part(const u32 *indptr, u32 n, int ps, vec &part_ptr, vec &part2node, vec &acc) {
    acc.assign(n, 0);
    u64 total = 0;
    for (u32 v = 0; v < n; ++v) {   // inclusive prefix (h:99-111)
        u32 span = indptr[v + 1] - indptr[v];
        total += (span + ps - 1) / ps;
        acc[v] = (u32)total;
    }
    part_ptr.assign(total + 1, 0);
    part2node.assign(total, 0);
#pragma omp parallel for schedule(static)
    for (int64_t v = 0; v < (int64_t)n; ++v) {
        u32 beg = indptr[v], end = indptr[v + 1];
        u32 np = (end - beg + ps - 1) / ps;
        u32 base = acc[v] - np;
        for (u32 j = 0; j < np; ++j) {
            part2node[base + j] = (u32)v;
            part_ptr[base + j + 1] = (j == np - 1) ? end : beg + (j + 1) * ps;   // h:139-146
        }
    }
}

void greedy_max_reuse(const u32 *cnt, u64 parts, const u32 *part_ptr, const u32 *indices_src, u64 e, vec &ordered,
                      vec &picked) {
    ordered.resize(parts);
    std::iota(ordered.begin(), ordered.end(), 0u);
    // Must stay this exact call: the tie order of std::sort is part of the plan (h:260-264).
    std::sort(ordered.begin(), ordered.end(), [cnt](size_t i1, size_t i2) { return cnt[i1] > cnt[i2]; });
    picked.clear();
    u32 max_src = 0;
    for (u64 k = 0; k < e; ++k) max_src = std::max(max_src, indices_src[k]);
    std::vector<uint8_t> used((size_t)max_src + 1, 0);
    for (u64 i = 0; i < parts; ++i) {
        u32 p = ordered[i];
        if (cnt[p] < 2) break;   // pick_threshold (h:235,272)
        bool clash = false;
        for (u32 k = part_ptr[p]; k < part_ptr[p + 1]; ++k)
            if (used[indices_src[k]]) {
                clash = true;
                break;
            }
        if (clash) continue;
        picked.push_back(p);
        for (u32 k = part_ptr[p]; k < part_ptr[p + 1]; ++k) used[indices_src[k]] = 1;
    }
}

// value -> position table for one long row (open addressing); falls back to scanning when the row
// holds a value twice, because upstream moves the first match (h:467).
struct RowIndex {
    vec key, pos;
    u32 mask = 0;
    bool ok = false;
    void build(const u32 *row, u32 len) {
        u32 cap = 16;
        while (cap < 2 * len) cap <<= 1;
        key.assign(cap, UINT32_MAX);
        pos.assign(cap, 0);
        mask = cap - 1;
        ok = true;
        for (u32 i = 0; i < len; ++i) {
            u32 h = (row[i] * 2654435761u) & mask;
            while (key[h] != UINT32_MAX) {
                if (key[h] == row[i]) {
                    ok = false;
                    return;
                }
                h = (h + 1) & mask;
            }
            key[h] = row[i];
            pos[h] = i;
        }
    }
    u32 *find(u32 v) {
        u32 h = (v * 2654435761u) & mask;
        while (key[h] != UINT32_MAX) {
            if (key[h] == v) return &pos[h];
            h = (h + 1) & mask;
        }
        return nullptr;
    }
};

const u32 kScanRow = 96;   // rows up to this length are searched linearly

// Shared row permutation of both reorganisers (h:450-498, 553-599).  consumed[v] = number of picked
// chunks node v takes; uses[v] lists them in pick order.
void permute_rows(const u32 *part_ptr, const u32 *indices_src, u64 e, const u32 *picked, u64 P, const u32 *gptr,
                  const u32 *gdst, const u32 *indptr_dst, u32 n, vec &rows, vec &use_ptr, vec &use_pick,
                  vec &moved) {
    rows.assign(indices_src, indices_src + e);
    moved.assign((size_t)n, 0);
    use_ptr.assign((size_t)n + 1, 0);
    for (u64 i = 0; i < P; ++i)
        for (u32 j = gptr[i]; j < gptr[i + 1]; ++j) use_ptr[gdst[j] + 1]++;
    for (u32 v = 0; v < n; ++v) use_ptr[v + 1] += use_ptr[v];
    use_pick.resize(use_ptr[n]);
    {
        vec at(use_ptr.begin(), use_ptr.end() - 1);
        for (u64 i = 0; i < P; ++i)   // pick order ascending => each node's list ascending
            for (u32 j = gptr[i]; j < gptr[i + 1]; ++j) use_pick[at[gdst[j]]++] = (u32)i;
    }
#pragma omp parallel
    {
        RowIndex table;
#pragma omp for schedule(dynamic, 512)
        for (int64_t v = 0; v < (int64_t)n; ++v) {
            u32 ub = use_ptr[v], ue = use_ptr[v + 1];
            if (ub == ue) continue;
            u32 *row = rows.data() + indptr_dst[v];
            u32 len = indptr_dst[v + 1] - indptr_dst[v];
            bool indexed = false;
            if (len > kScanRow) {
                table.build(row, len);
                indexed = table.ok;
            }
            u32 at = 0;
            for (u32 t = ub; t < ue; ++t) {
                u32 p = picked[use_pick[t]];
                for (u32 k = part_ptr[p]; k < part_ptr[p + 1]; ++k) {
                    u32 want = indices_src[k];
                    u32 q = len;
                    if (indexed) {
                        u32 *slot = table.find(want);
                        if (slot && *slot >= at) {
                            q = *slot;
                            u32 moved = row[at];
                            if (q != at) {
                                *table.find(moved) = q;
                                *slot = at;
                            }
                        }
                    } else {
                        for (q = at; q < len && row[q] != want; ++q) {}
                    }
                    if (q < len) {
                        std::swap(row[q], row[at]);
                        ++at;
                    }
                }
            }
            moved[v] = at;
        }
    }
}

int reorganize(const u32 *part_ptr, u64 parts, const u32 *indices_src, u64 e, const u32 *picked, u64 P,
               const u32 *gptr, const u32 *gdst, const u32 *indptr_dst, u32 n, const u32 *acc, int ps, int which,
               rof_bag *bag) {
    vec rows, use_ptr, use_pick, moved;
    permute_rows(part_ptr, indices_src, e, picked, P, gptr, gdst, indptr_dst, n, rows, use_ptr, use_pick, moved);
    if (which & 1) {
        vec &flag = bag->arr["part_cache_flagindex"];
        flag.assign(parts, 0);
        // cursor of node v starts at acc[v-1], and at 0 for v = 0 (h:430,495: the last prefix entry is
        // zeroed and indexed with (v-1+n)%n)
#pragma omp parallel for schedule(dynamic, 2048)
        for (int64_t v = 0; v < (int64_t)n; ++v) {
            u32 first = v == 0 ? 0 : acc[v - 1];
            for (u32 t = use_ptr[v]; t < use_ptr[v + 1]; ++t) {
                u64 slot = (u64)first + (t - use_ptr[v]);
                if (slot < parts) flag[slot] = use_pick[t] + 1;
            }
        }
        vec &cptr = bag->arr["part_pointers_cache"], &ccol = bag->arr["column_index_cache"];
        cptr.assign(P + 1, 0);
        for (u64 i = 0; i < P; ++i) cptr[i + 1] = cptr[i] + (part_ptr[picked[i] + 1] - part_ptr[picked[i]]);
        ccol.resize(cptr[P]);
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < (int64_t)P; ++i)
            memcpy(ccol.data() + cptr[i], indices_src + part_ptr[picked[i]], (cptr[i + 1] - cptr[i]) * sizeof(u32));
        if (which & 2) bag->arr["new_indices_src"] = rows;
        else bag->arr["new_indices_src"].swap(rows);
    }
    if (which & 2) {
        const vec &R = (which & 1) ? bag->arr["new_indices_src"] : rows;
        // the leftover of node v starts after the entries that were moved to the front (h:592)
        vec left_beg((size_t)n);
#pragma omp parallel for schedule(static)
        for (int64_t v = 0; v < (int64_t)n; ++v) left_beg[v] = indptr_dst[v] + moved[v];
        std::vector<u64> res_parts((size_t)n + 1, 0), res_cols((size_t)n + 1, 0);
        for (u32 v = 0; v < n; ++v) {
            u32 left = indptr_dst[v + 1] - left_beg[v];
            res_parts[v + 1] = res_parts[v] + (left + ps - 1) / ps;
            res_cols[v + 1] = res_cols[v] + left;
        }
        u64 picked_cols = 0, picked_dsts = gptr[P];
        for (u64 i = 0; i < P; ++i) picked_cols += part_ptr[picked[i] + 1] - part_ptr[picked[i]];
        u64 U = P + res_parts[n];
        vec &ucol = bag->arr["uniqpart_column_index"], &uptr = bag->arr["uniqpart_pointers"];
        vec &dptr = bag->arr["part2Node_ptr"], &dcol = bag->arr["part2Node_col"];
        ucol.resize(picked_cols + res_cols[n]);
        uptr.resize(U + 1);
        dptr.resize(U + 1);
        dcol.resize(picked_dsts + res_parts[n]);
        uptr[0] = 0;
        dptr[0] = 0;
        u32 c = 0;
        for (u64 i = 0; i < P; ++i) {   // h:548-551, 601-604
            u32 p = picked[i], len = part_ptr[p + 1] - part_ptr[p];
            memcpy(ucol.data() + c, indices_src + part_ptr[p], len * sizeof(u32));
            c += len;
            uptr[i + 1] = c;
            dptr[i + 1] = gptr[i + 1];
        }
        if (picked_dsts) memcpy(dcol.data(), gdst, picked_dsts * sizeof(u32));
#pragma omp parallel for schedule(dynamic, 2048)
        for (int64_t v = 0; v < (int64_t)n; ++v) {   // h:607-636
            u32 beg = left_beg[v], end = indptr_dst[v + 1];
            if (beg == end) continue;
            u64 cbase = picked_cols + res_cols[v];
            memcpy(ucol.data() + cbase, R.data() + beg, (end - beg) * sizeof(u32));
            u64 pbase = P + res_parts[v];
            u32 np = (u32)(res_parts[v + 1] - res_parts[v]);
            for (u32 j = 0; j < np; ++j) {
                u32 stop = std::min<u32>((j + 1) * ps, end - beg);
                uptr[pbase + j + 1] = (u32)(cbase + stop);
                dcol[picked_dsts + res_parts[v] + j] = (u32)v;
                dptr[pbase + j + 1] = (u32)(picked_dsts + res_parts[v] + j + 1);
            }
        }
    }
    return ROF_OK;
}

bool csr_ok(const u32 *ptr, u64 n, u64 e) {
    if (!ptr || ptr[0] != 0 || ptr[n] != e) return false;
    for (u64 v = 0; v < n; ++v)
        if (ptr[v] > ptr[v + 1]) return false;
    return true;
}

bool ids_ok(const u32 *idx, u64 e, u64 bound) {
    bool ok = true;
#pragma omp parallel for schedule(static) reduction(&& : ok)
    for (int64_t k = 0; k < (int64_t)e; ++k)
        if (idx[k] >= bound) ok = false;
    return ok;
}

}  // namespace

// =============================================================================================
extern "C" {

int64_t rof_bag_get(const rof_bag *bag, const char *name, const uint32_t **data) {
    if (!bag || !name) return -1;
    auto it = bag->arr.find(name);
    if (it == bag->arr.end()) return -1;
    if (data) *data = it->second.data();
    return (int64_t)it->second.size();
}

void rof_bag_free(rof_bag *bag) { delete bag; }

int rof_split_part(const uint32_t *indptr_dst, uint32_t n, int part_size, rof_bag **out) {
    if (!indptr_dst || !out || part_size < 1) return ROF_ERR_ARG;
    if (!csr_ok(indptr_dst, n, indptr_dst[n])) return ROF_ERR_RANGE;
    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        split_part(indptr_dst, n, part_size, bag->arr["part_ptr"], bag->arr["part2Node"],
                   bag->arr["num_parts_per_node_acc"]);
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

static int check_intersect_args(const uint32_t *part_ptr, uint64_t num_parts, const uint32_t *indices_src, uint64_t e,
                                const uint32_t *indptr_src, const uint32_t *indices_dst, uint32_t n, int part_size) {
    if (!part_ptr || !indptr_src || part_size < 1) return ROF_ERR_ARG;
    if (e && (!indices_src || !indices_dst)) return ROF_ERR_ARG;
    if (!csr_ok(part_ptr, num_parts, e)) return ROF_ERR_RANGE;
    if (!csr_ok(indptr_src, n, indptr_src[n])) return ROF_ERR_RANGE;
    if (!ids_ok(indices_src, e, n)) return ROF_ERR_RANGE;
    if (!ids_ok(indices_dst, indptr_src[n], (uint64_t)UINT32_MAX)) return ROF_ERR_RANGE;
    return ROF_OK;
}

int rof_part_intersect_count(const uint32_t *part_ptr, uint64_t num_parts, const uint32_t *indices_src, uint64_t e,
                             const uint32_t *indptr_src, const uint32_t *indices_dst, uint32_t n, int part_size,
                             int discard_remainder_part, rof_bag **out) {
    if (!out) return ROF_ERR_ARG;
    int st = check_intersect_args(part_ptr, num_parts, indices_src, e, indptr_src, indices_dst, n, part_size);
    if (st) return st;
    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        OutLists g;
        prepare_out_lists(indptr_src, indices_dst, n, g);
        intersect_counts(part_ptr, num_parts, indices_src, g, part_size, discard_remainder_part != 0,
                         bag->arr["intersect_count"]);
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

int rof_part_intersect_lists(const uint32_t *part_ptr, uint64_t num_parts, const uint32_t *indices_src, uint64_t e,
                             const uint32_t *indptr_src, const uint32_t *indices_dst, uint32_t n, int part_size,
                             int discard_remainder_part, const uint32_t *which, uint64_t n_which, rof_bag **out) {
    if (!out || (n_which && !which)) return ROF_ERR_ARG;
    int st = check_intersect_args(part_ptr, num_parts, indices_src, e, indptr_src, indices_dst, n, part_size);
    if (st) return st;
    if (!ids_ok(which, n_which, num_parts)) return ROF_ERR_RANGE;
    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        OutLists g;
        prepare_out_lists(indptr_src, indices_dst, n, g);
        intersect_lists(part_ptr, indices_src, g, part_size, discard_remainder_part != 0, which, n_which,
                        bag->arr["ptr"], bag->arr["data"]);
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

int rof_greedy_max_reuse(const uint32_t *intersect_count, uint64_t num_parts, const uint32_t *part_ptr,
                         const uint32_t *indices_src, uint64_t e, rof_bag **out) {
    if (!out || !part_ptr || (num_parts && !intersect_count) || (e && !indices_src)) return ROF_ERR_ARG;
    if (!csr_ok(part_ptr, num_parts, e)) return ROF_ERR_RANGE;
    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        greedy_max_reuse(intersect_count, num_parts, part_ptr, indices_src, e, bag->arr["index_ordered"],
                         bag->arr["index_picked"]);
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

int rof_reorganize(const uint32_t *part_ptr, uint64_t num_parts, const uint32_t *indices_src, uint64_t e,
                   const uint32_t *index_picked, uint64_t num_picked, const uint32_t *picked_dst_ptr,
                   const uint32_t *picked_dst, const uint32_t *indptr_dst, uint32_t n,
                   const uint32_t *num_parts_per_node_acc, int part_size, int which, rof_bag **out) {
    if (!out || !part_ptr || !indptr_dst || !picked_dst_ptr || part_size < 1 || !(which & 3)) return ROF_ERR_ARG;
    if ((e && !indices_src) || (num_picked && !index_picked) || (n && !num_parts_per_node_acc)) return ROF_ERR_ARG;
    if (!csr_ok(part_ptr, num_parts, e) || !csr_ok(indptr_dst, n, e)) return ROF_ERR_RANGE;
    if (!csr_ok(picked_dst_ptr, num_picked, picked_dst_ptr[num_picked])) return ROF_ERR_RANGE;
    if (picked_dst_ptr[num_picked] && !picked_dst) return ROF_ERR_ARG;
    if (!ids_ok(index_picked, num_picked, num_parts) || !ids_ok(picked_dst, picked_dst_ptr[num_picked], n))
        return ROF_ERR_RANGE;
    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        reorganize(part_ptr, num_parts, indices_src, e, index_picked, num_picked, picked_dst_ptr, picked_dst,
                   indptr_dst, n, num_parts_per_node_acc, part_size, which, bag);
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

int rof_transpose_csr(const uint32_t *indptr, const uint32_t *indices, uint32_t n, uint64_t e, rof_bag **out) {
    if (!out || !indptr || (e && !indices)) return ROF_ERR_ARG;
    if (!csr_ok(indptr, n, e) || !ids_ok(indices, e, n)) return ROF_ERR_RANGE;
    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        vec &op = bag->arr["indptr"], &ox = bag->arr["indices"];
        op.assign((size_t)n + 1, 0);
        ox.resize(e);
        for (u64 k = 0; k < e; ++k) op[indices[k] + 1]++;
        for (u32 v = 0; v < n; ++v) op[v + 1] += op[v];
        vec at(op.begin(), op.end() - 1);
        for (u32 v = 0; v < n; ++v)   // ascending v => every output row ascending (h:53-57)
            for (u32 k = indptr[v]; k < indptr[v + 1]; ++k) ox[at[indices[k]]++] = v;
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

int rof_plan_build(const uint32_t *indptr_dst, const uint32_t *indices_src, const uint32_t *indptr_src,
                   const uint32_t *indices_dst, uint32_t n, uint64_t e, int part_size, int discard_remainder_part,
                   rof_bag **out) {
    if (!out || !indptr_dst || (e && !indices_src) || part_size < 1) return ROF_ERR_ARG;
    if ((indptr_src == nullptr) != (indices_dst == nullptr) && e) return ROF_ERR_ARG;
    if (!indptr_src) {
        indptr_src = indptr_dst;
        indices_dst = indices_src;
    }
    if (!csr_ok(indptr_dst, n, e) || !csr_ok(indptr_src, n, e)) return ROF_ERR_RANGE;
    if (!ids_ok(indices_src, e, n) || !ids_ok(indices_dst, e, n)) return ROF_ERR_RANGE;
    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        auto &A = bag->arr;
        bool discard = discard_remainder_part != 0;
        split_part(indptr_dst, n, part_size, A["part_ptr"], A["part2Node"], A["num_parts_per_node_acc"]);
        const vec &pp = A["part_ptr"];
        u64 parts = pp.size() - 1;
        OutLists g;
        prepare_out_lists(indptr_src, indices_dst, n, g);
        intersect_counts(pp.data(), parts, indices_src, g, part_size, discard, A["intersect_count"]);
        greedy_max_reuse(A["intersect_count"].data(), parts, pp.data(), indices_src, e, A["index_ordered"],
                         A["index_picked"]);
        const vec &picked = A["index_picked"];
        intersect_lists(pp.data(), indices_src, g, part_size, discard, picked.data(), picked.size(),
                        A["picked_dst_ptr"], A["picked_dst"]);
        reorganize(pp.data(), parts, indices_src, e, picked.data(), picked.size(), A["picked_dst_ptr"].data(),
                   A["picked_dst"].data(), indptr_dst, n, A["num_parts_per_node_acc"].data(), part_size, 3, bag);
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}

}  // extern "C"
