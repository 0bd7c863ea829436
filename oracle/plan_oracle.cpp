// TEST INFRASTRUCTURE -- not part of the shipped library.
//
// CPU oracle for the reuse-plan builder: a deliberately plain, single-threaded restatement of
// the upstream algorithm (ROF/reuse_search_ext/src/reuse_search_ext.h).  It favours obviousness
// over speed: sorted-vector merges, linear searches, one pass per step.  The shipped builder
// (artifact_amd/csrc/plan_builder.cpp) must reproduce every array below bit for bit.
//
// Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this file's
// library.  Pinning: tests/test_oracle_plan.py checks it against the committed golden plans
// (produced by the upstream builder itself), against oracle/_ref where that is built, and
// against the structural invariants of a valid plan.
//
// Steps and the upstream lines each follows:
//   chunk_rows        reuse_search_ext.h:82-148   (split_part)
//   common_dsts       reuse_search_ext.h:152-228  (get_part_intersect)
//   greedy_pick       reuse_search_ext.h:232-303  (greedy_max_reuse)
//   permute_rows      reuse_search_ext.h:437-504 / 537-605 (shared swap loop of both reorganisers)
//   emit_v1           reuse_search_ext.h:409-505  (reorganize_indices)
//   emit_v2           reuse_search_ext.h:507-640  (reorganize_indices_uniquely)
//   transpose_csr     reuse_search_ext.h:18-78    (inverse_csc)
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <map>
#include <string>
#include <vector>

typedef uint32_t u32;
typedef std::vector<u32> vec;

struct orc_plan {
    std::map<std::string, vec> arr;
};

// reuse_search_ext.h:96-147: every row is cut into ceil(deg/ps) chunks, the last one short.
// acc is the inclusive prefix sum of chunk counts per node (h:104-111).
static void chunk_rows(const vec &indptr, int ps, vec &part_ptr, vec &part2node, vec &acc) {
    size_t n = indptr.size() - 1;
    part_ptr.assign(1, 0);
    part2node.clear();
    acc.assign(n, 0);
    u32 running = 0;
    for (size_t v = 0; v < n; ++v) {
        u32 beg = indptr[v], end = indptr[v + 1];
        for (u32 p = beg; p < end; p += ps) {
            part_ptr.push_back(std::min<u32>(p + ps, end));
            part2node.push_back((u32)v);
            ++running;
        }
        acc[v] = running;
    }
}

// reuse_search_ext.h:170-224: the nodes that every source of the chunk points to, ascending.
// Remainder chunks yield the empty list when `discard` is set (h:177-181).
static void common_dsts(const vec &part_ptr, const vec &indices_src, const vec &indptr_src,
                        const vec &indices_dst, int ps, bool discard, vec &out_ptr, vec &out_data) {
    size_t parts = part_ptr.size() - 1;
    out_ptr.assign(1, 0);
    out_data.clear();
    vec cur, nxt, lst;
    for (size_t p = 0; p < parts; ++p) {
        u32 beg = part_ptr[p], end = part_ptr[p + 1];
        if (!(discard && (int)(end - beg) != ps) && end > beg) {
            u32 s0 = indices_src[beg];
            cur.assign(indices_dst.begin() + indptr_src[s0], indices_dst.begin() + indptr_src[s0 + 1]);
            std::sort(cur.begin(), cur.end());
            cur.erase(std::unique(cur.begin(), cur.end()), cur.end());   // std::set semantics, h:194
            for (u32 k = beg + 1; k < end; ++k) {
                u32 s = indices_src[k];
                lst.assign(indices_dst.begin() + indptr_src[s], indices_dst.begin() + indptr_src[s + 1]);
                std::sort(lst.begin(), lst.end());
                nxt.clear();
                std::set_intersection(lst.begin(), lst.end(), cur.begin(), cur.end(), std::back_inserter(nxt));
                nxt.erase(std::unique(nxt.begin(), nxt.end()), nxt.end());
                cur.swap(nxt);
            }
            out_data.insert(out_data.end(), cur.begin(), cur.end());
        }
        out_ptr.push_back((u32)out_data.size());
    }
}

// reuse_search_ext.h:245-302.  The order of equal counts is whatever std::sort leaves
// (h:260-264); the same call on the same element type reproduces it.
static void greedy_pick(const vec &cnt, const vec &part_ptr, const vec &indices_src, vec &ordered, vec &picked) {
    ordered.resize(cnt.size());
    for (size_t i = 0; i < ordered.size(); ++i) ordered[i] = (u32)i;
    std::sort(ordered.begin(), ordered.end(), [&cnt](size_t a, size_t b) { return cnt[a] > cnt[b]; });
    picked.clear();
    std::vector<u32> used;   // kept sorted
    for (size_t i = 0; i < ordered.size(); ++i) {
        u32 p = ordered[i];
        if (cnt[p] < 2) break;                                   // pick_threshold, h:235,272
        bool clash = false;
        for (u32 k = part_ptr[p]; k < part_ptr[p + 1] && !clash; ++k)
            clash = std::binary_search(used.begin(), used.end(), indices_src[k]);
        if (clash) continue;
        picked.push_back(p);
        for (u32 k = part_ptr[p]; k < part_ptr[p + 1]; ++k) {
            u32 s = indices_src[k];
            auto it = std::lower_bound(used.begin(), used.end(), s);
            if (it == used.end() || *it != s) used.insert(it, s);   // set insert ignores repeats, h:296
        }
    }
}

// Swap loop shared by both reorganisers (h:450-498 and 553-599): for the i-th picked chunk and
// each node d that contains it, bring the chunk's sources (in the chunk's original order) to the
// front of what is left of d's row by first-match search and swap.  `slot[d]` counts how many
// picked chunks d has consumed; v1 records i+1 at the node's next chunk slot (h:495-496).
static void permute_rows(const vec &part_ptr, const vec &orig, const vec &ipp, const vec &ipd, const vec &picked,
                         const vec &indptr_dst, const vec &acc_in, vec &rows, vec &cur_pos, vec *flags) {
    rows = orig;
    cur_pos.assign(indptr_dst.begin(), indptr_dst.end());
    size_t n = indptr_dst.size() - 1;
    vec acc = acc_in;
    if (!acc.empty()) acc.back() = 0;                              // h:430 / 530
    for (size_t i = 0; i < picked.size(); ++i) {
        u32 p = picked[i], pb = part_ptr[p], pe = part_ptr[p + 1];
        for (u32 j = ipp[p]; j < ipp[p + 1]; ++j) {
            u32 d = ipd[j];
            u32 at = cur_pos[d], row_end = indptr_dst[d + 1];
            for (u32 k = pb; k < pe; ++k) {
                u32 q = at;
                while (q < row_end && rows[q] != orig[k]) ++q;
                if (q < row_end) { std::swap(rows[q], rows[at]); ++at; }
            }
            cur_pos[d] = at;
            size_t prev = (d + n - 1) % n;
            // with discard off a remainder chunk can be picked and this slot can run past the array
            // (upstream writes out of bounds there: undefined); the oracle drops such writes
            if (flags && acc[prev] < flags->size()) (*flags)[acc[prev]] = (u32)i + 1;
            acc[prev] += 1;
        }
    }
}

extern "C" {

orc_plan *orc_plan_build(const u32 *indptr_dst, const u32 *indices_src, const u32 *indptr_src,
                         const u32 *indices_dst, u32 n, u32 e, int ps, int discard) {
    orc_plan *pl = new orc_plan;
    auto &A = pl->arr;
    vec ipd(indptr_dst, indptr_dst + n + 1), isrc(indices_src, indices_src + e);
    vec ips(indptr_src, indptr_src + n + 1), idst(indices_dst, indices_dst + e);

    chunk_rows(ipd, ps, A["part_ptr"], A["part2Node"], A["num_parts_per_node_acc"]);
    common_dsts(A["part_ptr"], isrc, ips, idst, ps, discard != 0, A["intersect_ptr"], A["intersect_data"]);
    vec &ipp = A["intersect_ptr"];
    vec &cnt = A["intersect_count"];
    cnt.resize(ipp.size() - 1);
    for (size_t p = 0; p + 1 < ipp.size(); ++p) cnt[p] = ipp[p + 1] - ipp[p];
    greedy_pick(cnt, A["part_ptr"], isrc, A["index_ordered"], A["index_picked"]);
    const vec &picked = A["index_picked"];
    const vec &pp = A["part_ptr"];

    // ---- v1 (h:409-505): permuted rows + cache CSR + per-chunk flag
    vec cur_pos;
    A["part_cache_flagindex"].assign(pp.size() - 1, 0);
    permute_rows(pp, isrc, ipp, A["intersect_data"], picked, ipd, A["num_parts_per_node_acc"],
                 A["new_indices_src"], cur_pos, &A["part_cache_flagindex"]);
    vec &cptr = A["part_pointers_cache"], &ccol = A["column_index_cache"];
    cptr.assign(1, 0);
    for (u32 p : picked) {
        ccol.insert(ccol.end(), isrc.begin() + pp[p], isrc.begin() + pp[p + 1]);   // h:501-503
        cptr.push_back((u32)ccol.size());
    }

    // ---- v2 (h:507-640): picked chunks first, then each node's leftover neighbours re-chunked
    vec rows2, cur2;
    permute_rows(pp, isrc, ipp, A["intersect_data"], picked, ipd, A["num_parts_per_node_acc"], rows2, cur2, nullptr);
    vec &ucol = A["uniqpart_column_index"], &uptr = A["uniqpart_pointers"];
    vec &dptr = A["part2Node_ptr"], &dcol = A["part2Node_col"];
    uptr.assign(1, 0);
    dptr.assign(1, 0);
    for (u32 p : picked) {
        dcol.insert(dcol.end(), A["intersect_data"].begin() + ipp[p], A["intersect_data"].begin() + ipp[p + 1]);
        dptr.push_back((u32)dcol.size());                                            // h:550-551
        ucol.insert(ucol.end(), isrc.begin() + pp[p], isrc.begin() + pp[p + 1]);
        uptr.push_back((u32)ucol.size());                                            // h:602-604
    }
    for (u32 v = 0; v < n; ++v) {                                                    // h:607-636
        u32 beg = cur2[v], end = ipd[v + 1];
        for (u32 q = beg; q < end; q += ps) {
            u32 stop = std::min<u32>(q + ps, end);
            ucol.insert(ucol.end(), rows2.begin() + q, rows2.begin() + stop);
            uptr.push_back((u32)ucol.size());
            dcol.push_back(v);
            dptr.push_back((u32)dcol.size());
        }
    }
    return pl;
}

// Returns the element count and, if `out` is non-null, copies the array.
int64_t orc_plan_array(const orc_plan *pl, const char *name, u32 *out) {
    auto it = pl->arr.find(name);
    if (it == pl->arr.end()) return -1;
    if (out && !it->second.empty()) memcpy(out, it->second.data(), it->second.size() * sizeof(u32));
    return (int64_t)it->second.size();
}

void orc_plan_free(orc_plan *pl) { delete pl; }

// reuse_search_ext.h:18-78: CSR transpose with ascending rows.
void orc_transpose_csr(const u32 *indptr, const u32 *indices, u32 n, u32 e, u32 *out_ptr, u32 *out_idx) {
    std::vector<u32> deg(n + 1, 0);
    for (u32 k = 0; k < e; ++k) deg[indices[k] + 1]++;
    out_ptr[0] = 0;
    for (u32 v = 0; v < n; ++v) out_ptr[v + 1] = out_ptr[v] + deg[v + 1];
    std::vector<u32> at(out_ptr, out_ptr + n);
    for (u32 v = 0; v < n; ++v)
        for (u32 k = indptr[v]; k < indptr[v + 1]; ++k) out_idx[at[indices[k]]++] = v;   // v ascending => rows sorted
}

}  // extern "C"
