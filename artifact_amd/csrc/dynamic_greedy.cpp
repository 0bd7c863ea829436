// Alternative reuse search: the "dynamic greedy" that upstream sketches in the comment block of
// reuse_search_ext.h:305-321 and leaves unfinished (the function under it, h:322-406, is a copy of the static
// greedy).  Off by default; upstream's bit-exact plan (plan_builder.cpp) stays the default.
//
// Upstream's static greedy (h:232-303) walks the parts by descending size of their intersection lists and takes
// a part only if none of its sources is used by an earlier pick, so a source ends up in at most one shared part
// of the whole graph.  The sketch relaxes that to what correctness needs -- no destination may consume two
// shared parts that overlap in a source:
//   1. candidates are the full parts whose intersection list I_p (destinations that have all of p's sources
//      among their in-neighbours, h:152-228) holds at least two destinations; parts with equal sources are
//      one candidate (the first such part);
//   2. a max-heap orders the candidates by the current size of I_p (ties: lower part index first);
//   3. the top candidate c is picked with its current I_c, and every other candidate cc that shares a source
//      with c loses c's destinations: I_cc <- I_cc \ I_c; candidates that fall under two destinations die;
//   4. until the heap is empty.
// By step 3 two picked parts that share a source never share a destination, so every destination can drop the
// sources of all the parts it consumes from its own list.  The plan is emitted in upstream's v2 format
// (h:537-636: shared parts in pick order, then every node's remaining in-neighbours in chunks of part_size), so
// the device layout and the operator API run it unchanged.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <new>
#include <queue>
#include <utility>
#include <vector>
#include <omp.h>

#include "rof.h"
#include "rof_internal.h"

namespace {

typedef uint32_t u32;
typedef uint64_t u64;
typedef std::vector<u32> vec;

struct Bag {   // frees a bag obtained from another entry point of this library
    rof_bag *b = nullptr;
    ~Bag() { rof_bag_free(b); }
    const u32 *get(const char *name, int64_t *len = nullptr) const {
        const u32 *p = nullptr;
        int64_t l = rof_bag_get(b, name, &p);
        if (len) *len = l;
        return p;
    }
};

struct Entry {   // heap entry: size of the candidate's list when it was pushed
    u32 size, cand;
    bool operator<(const Entry &o) const { return size != o.size ? size < o.size : cand > o.cand; }
};

}  // namespace

extern "C" int rof_plan_dynamic_greedy(const uint32_t *indptr_dst, const uint32_t *indices_src,
                                       const uint32_t *indptr_src, const uint32_t *indices_dst, uint32_t n, uint64_t e,
                                       int part_size, rof_bag **out) {
    if (!out || !indptr_dst || (e && !indices_src) || part_size < 2 || (!indptr_src) != (!indices_dst)) return ROF_ERR_ARG;
    if (!indptr_src) {   // symmetric graph: the in-neighbour lists are the out-neighbour lists
        indptr_src = indptr_dst;
        indices_dst = indices_src;
    }
    const int ps = part_size;
    int rc;
    Bag split, counts, lists;
    if ((rc = rof_split_part(indptr_dst, n, ps, &split.b))) return rc;
    int64_t np1 = 0;
    const u32 *part_ptr = split.get("part_ptr", &np1);
    const u64 parts = (u64)np1 - 1;
    if ((rc = rof_part_intersect_count(part_ptr, parts, indices_src, e, indptr_src, indices_dst, n, ps, 1, &counts.b)))
        return rc;   // validates both CSRs
    const u32 *cnt = counts.get("intersect_count");

    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        // 1. candidates: full parts with at least two destinations, one per distinct source tuple
        vec cand;
        for (u64 p = 0; p < parts; ++p)
            if (cnt[p] >= 2) cand.push_back((u32)p);
        auto srcs = [&](u32 p) { return indices_src + part_ptr[p]; };
        std::sort(cand.begin(), cand.end(), [&](u32 a, u32 b) {
            int c = std::memcmp(srcs(a), srcs(b), (size_t)ps * sizeof(u32));   // equality is all that matters here
            return c != 0 ? c < 0 : a < b;
        });
        cand.erase(std::unique(cand.begin(), cand.end(),
                               [&](u32 a, u32 b) { return std::memcmp(srcs(a), srcs(b), (size_t)ps * sizeof(u32)) == 0; }),
                   cand.end());
        std::sort(cand.begin(), cand.end());   // candidate number = rank of its part index
        const u32 C = (u32)cand.size();

        // their intersection lists, each ascending; lists shrink in place (live[c] = current length)
        if ((rc = rof_part_intersect_lists(part_ptr, parts, indices_src, e, indptr_src, indices_dst, n, ps, 1,
                                           cand.data(), C, &lists.b))) {
            delete bag;
            return rc;
        }
        int64_t ldata_len = 0;
        const u32 *lptr0 = lists.get("ptr"), *ldata0 = lists.get("data", &ldata_len);
        const vec lptr(lptr0, lptr0 + (size_t)C + 1);
        vec ldata(ldata0, ldata0 + (ldata_len > 0 ? ldata_len : 0));
        rof_bag_free(lists.b);   // the copies above are what is worked on
        lists.b = nullptr;
        vec live(C);
        for (u32 c = 0; c < C; ++c) live[c] = lptr[c + 1] - lptr[c];
        // 64-bit signature of each list (one hashed bit per destination): two lists whose signatures do not
        // meet have no destination in common, which settles more than half of the comparisons without reading a list
        auto bit_of = [](u32 d) { return (u64)1 << ((d * 0x9E3779B1u) >> 26); };
        std::vector<u64> sig(C, 0);
#pragma omp parallel for schedule(dynamic, 4096)
        for (u32 c = 0; c < C; ++c) {
            u64 m = 0;
            for (u32 j = lptr[c]; j < lptr[c + 1]; ++j) m |= bit_of(ldata[j]);
            sig[c] = m;
        }

        // source -> candidates that contain it
        vec by_src_ptr((size_t)n + 1, 0), by_src((size_t)C * ps);
        for (u32 c = 0; c < C; ++c)
            for (int k = 0; k < ps; ++k) by_src_ptr[srcs(cand[c])[k] + 1]++;
        for (u32 s = 0; s < n; ++s) by_src_ptr[s + 1] += by_src_ptr[s];
        // Each entry of a source's list carries a copy of the candidate's signature, so that walking a list reads
        // memory in order and goes to the candidate itself only when the signatures meet.  Lists only shrink, so a
        // copy that is out of date still covers the current list; it is refreshed when the candidate is visited.
        std::vector<u64> by_sig((size_t)C * ps);
        {
            vec at(by_src_ptr.begin(), by_src_ptr.end() - 1);
            for (u32 c = 0; c < C; ++c)
                for (int k = 0; k < ps; ++k) {
                    const u32 j = at[srcs(cand[c])[k]]++;
                    by_src[j] = c;
                    by_sig[j] = sig[c];
                }
        }
        vec by_src_end(by_src_ptr.begin() + 1, by_src_ptr.end());   // current end of each source's list

        // 2.-4. the greedy itself; stale heap entries are refreshed when they surface
        std::priority_queue<Entry> heap;
        for (u32 c = 0; c < C; ++c) heap.push(Entry{live[c], c});
        std::vector<uint8_t> done(C, 0);   // picked or dead
        vec picked;                        // candidate numbers in pick order
        while (!heap.empty()) {
            const Entry top = heap.top();
            heap.pop();
            const u32 c = top.cand;
            if (done[c]) continue;
            if (top.size != live[c]) {     // shrank since it was pushed
                if (live[c] >= 2) heap.push(Entry{live[c], c});
                else done[c] = 1;
                continue;
            }
            done[c] = 1;
            picked.push_back(c);
            const u32 *ic = ldata.data() + lptr[c];
            const u32 nc = live[c];
            const u64 sig_c = sig[c];
            for (int k = 0; k < ps; ++k) {
                const u32 s = srcs(cand[c])[k];
                u32 keep = by_src_ptr[s];   // the list of s is compacted as it is walked: finished candidates leave
                for (u32 j = by_src_ptr[s]; j < by_src_end[s]; ++j) {
                    const u32 cc = by_src[j];
                    if (done[cc]) continue;
                    const u64 seen = by_sig[j];
                    by_src[keep] = cc;
                    by_sig[keep] = seen;
                    ++keep;
                    if (!(seen & sig_c)) continue;          // no destination in common
                    by_sig[keep - 1] = sig[cc];
                    if (!(sig[cc] & sig_c)) continue;
                    u32 *icc = ldata.data() + lptr[cc];
                    const u32 ncc = live[cc];
                    if (ic[nc - 1] < icc[0] || icc[ncc - 1] < ic[0]) continue;   // the id ranges do not meet
                    u32 w = 0;                 // icc \ ic, both ascending
                    if ((u64)ncc * 16 < nc) {   // a short list against a long one: look each element up
                        for (u32 a = 0; a < ncc; ++a)
                            if (!std::binary_search(ic, ic + nc, icc[a])) icc[w++] = icc[a];
                    } else {
                        u32 a = 0, b = 0;
                        while (a < ncc) {
                            while (b < nc && ic[b] < icc[a]) ++b;
                            if (b < nc && ic[b] == icc[a]) ++a;
                            else icc[w++] = icc[a++];
                        }
                    }
                    if (w != ncc) {
                        u64 m = 0;
                        for (u32 a = 0; a < w; ++a) m |= bit_of(icc[a]);
                        sig[cc] = by_sig[keep - 1] = m;
                        live[cc] = w;
                        if (w < 2) {
                            done[cc] = 1;
                            --keep;            // it was the last one kept
                        }
                    }
                }
                by_src_end[s] = keep;
            }
        }
        const u64 G = picked.size();

        // emit: shared parts in pick order ...
        vec &ucol = bag->arr["uniqpart_column_index"], &uptr = bag->arr["uniqpart_pointers"];
        vec &dptr = bag->arr["part2Node_ptr"], &dcol = bag->arr["part2Node_col"];
        vec &index_picked = bag->arr["index_picked"];
        uptr.push_back(0);
        dptr.push_back(0);
        for (u32 c : picked) {
            index_picked.push_back(cand[c]);
            ucol.insert(ucol.end(), srcs(cand[c]), srcs(cand[c]) + ps);
            uptr.push_back((u32)ucol.size());
            dcol.insert(dcol.end(), ldata.begin() + lptr[c], ldata.begin() + lptr[c] + live[c]);
            dptr.push_back((u32)dcol.size());
        }
        // ... then what is left of every row: node -> shared parts it consumes
        vec ng_ptr((size_t)n + 1, 0), ng(dcol.size());
        for (u32 d : dcol) ng_ptr[d + 1]++;
        for (u32 v = 0; v < n; ++v) ng_ptr[v + 1] += ng_ptr[v];
        {
            vec at(ng_ptr.begin(), ng_ptr.end() - 1);
            for (u64 g = 0; g < G; ++g)
                for (u32 j = dptr[g]; j < dptr[g + 1]; ++j) ng[at[dcol[j]]++] = (u32)g;
        }
        vec left(n);
        for (u32 v = 0; v < n; ++v) {
            const u64 deg = indptr_dst[v + 1] - indptr_dst[v], through = (u64)(ng_ptr[v + 1] - ng_ptr[v]) * (u64)ps;
            if (through > deg) {   // the out-neighbour lists are not the transpose of the in-neighbour lists
                delete bag;
                return ROF_ERR_RANGE;
            }
            left[v] = (u32)(deg - through);
        }
        std::vector<u64> chunk_at((size_t)n + 1, 0), col_at((size_t)n + 1, 0);
        for (u32 v = 0; v < n; ++v) {
            chunk_at[v + 1] = chunk_at[v] + (left[v] + ps - 1) / ps;
            col_at[v + 1] = col_at[v] + left[v];
        }
        const u64 U = G + chunk_at[n], ncol0 = ucol.size(), nd0 = dcol.size();
        if (U + 1 > (u64)INT32_MAX || ncol0 + col_at[n] > (u64)INT32_MAX) {
            delete bag;
            return ROF_ERR_UNSUPPORTED;
        }
        ucol.resize(ncol0 + col_at[n]);
        uptr.resize(U + 1);
        dptr.resize(U + 1);
        dcol.resize(nd0 + chunk_at[n]);
        bool consistent = true;
#pragma omp parallel reduction(&& : consistent)
        {
            vec covered((size_t)n, 0);   // covered[s] == v + 1: source s of row v comes through a shared part
#pragma omp for schedule(dynamic, 1024)
            for (u32 v = 0; v < n; ++v) {
                for (u32 j = ng_ptr[v]; j < ng_ptr[v + 1]; ++j)
                    for (u32 q = uptr[ng[j]]; q < uptr[ng[j] + 1]; ++q) {
                        if (covered[ucol[q]] == v + 1) consistent = false;   // two parts of one row share a source
                        covered[ucol[q]] = v + 1;
                    }
                u64 at = ncol0 + col_at[v];
                const u64 stop_at = at + left[v];
                for (u32 j = indptr_dst[v]; j < indptr_dst[v + 1]; ++j) {
                    const u32 s = indices_src[j];
                    if (covered[s] == v + 1) {
                        covered[s] = 0;        // a repeated occurrence is an ordinary neighbour again
                        continue;
                    }
                    if (at < stop_at) ucol[at] = s;
                    ++at;
                }
                if (at != stop_at) consistent = false;   // a shared part named a source the row does not have
                const u64 chunks = chunk_at[v + 1] - chunk_at[v];
                for (u64 c = 0; c < chunks; ++c) {
                    const u64 w = G + chunk_at[v] + c;
                    const u64 stop = std::min<u64>((c + 1) * (u64)ps, left[v]);
                    uptr[w + 1] = (u32)(ncol0 + col_at[v] + stop);
                    dptr[w + 1] = (u32)(nd0 + chunk_at[v] + c + 1);
                    dcol[nd0 + chunk_at[v] + c] = v;
                }
            }
        }
        if (!consistent) {   // cannot happen for valid CSRs that are each other's transpose
            delete bag;
            return ROF_ERR_RANGE;
        }
        bag->arr["shared_parts"] = vec{(u32)G};
        bag->arr["candidates"] = vec{C};
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}
