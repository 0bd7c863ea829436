// Alternative reuse search: "hub patterns".  Not the upstream algorithm -- upstream's builder stays the
// default and bit-exact (plan_builder.cpp); this one answers the open item upstream leaves in
// reuse_search_ext.h:305-406 (a search that finds more reuse than the one-part-per-source greedy) with a
// scheme that fits heavy-tailed graphs and runs in O(E) plus one sort.
//
// Upstream picks parts whose source sets are pairwise disjoint over the whole graph (h:266-296), so a hub
// source can take part in one shared group only, while it co-occurs with many other hubs in many rows.  Here:
//   1. rank the sources by the number of rows they appear in; the first `hubs` are hubs; consecutive ranks
//      are tied into blocks of `block` hubs (similar popularity, hence similar co-occurrence);
//   2. per destination row and block, the subset of the block's hubs among the row's neighbours is a bit
//      pattern; every (block, pattern) with at least two hubs is a candidate group whose consumers are the
//      rows showing exactly that pattern -- groups of one block never overlap inside a row, so a row may
//      consume one group per block;
//   3. a candidate is kept when it repays itself: (consumers - 1) * hubs_in_pattern > consumers + 1 (row
//      gathers saved against the partial-row reads and the one write it adds);
//   4. the result is emitted in upstream's own v2 format (h:537-636: shared parts first, then every node's
//      remaining neighbours in chunks), with part size = `block`, so everything downstream -- the device
//      layout, ROF.reuse_forward_v2, even upstream's kernel -- runs it unchanged.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <new>
#include <parallel/algorithm>
#include <utility>
#include <vector>
#include <omp.h>

#include "rof.h"
#include "rof_internal.h"

namespace {

typedef uint32_t u32;
typedef uint64_t u64;
typedef std::vector<u32> vec;

struct Seen {   // (block << 16 | pattern, row)
    u64 key;
    u32 row;
    bool operator<(const Seen &o) const { return key != o.key ? key < o.key : row < o.row; }
};

inline u64 make_key(u32 blk, u32 pattern) { return ((u64)blk << 16) | pattern; }

// Calls f(block, pattern) for every block of which row [beg, end) holds at least two hubs.  A source that
// occurs twice in a row counts once (the second occurrence stays an ordinary neighbour).
template <typename F>
inline void row_patterns(const u32 *src, u64 beg, u64 end, const int32_t *rank, int block, std::vector<uint16_t> &mask,
                         vec &touched, F f) {
    for (u64 j = beg; j < end; ++j) {
        const int32_t r = rank[src[j]];
        if (r < 0) continue;
        const u32 blk = (u32)r / (u32)block, bit = 1u << ((u32)r % (u32)block);
        if (!mask[blk]) touched.push_back(blk);
        mask[blk] |= (uint16_t)bit;
    }
    for (u32 blk : touched) {
        const u32 m = mask[blk];
        mask[blk] = 0;
        if (m & (m - 1)) f(blk, m);
    }
    touched.clear();
}

}  // namespace

extern "C" int rof_plan_hub_patterns(const uint32_t *indptr_dst, const uint32_t *indices_src, uint32_t n, uint64_t e,
                                     uint32_t hubs, int block, rof_bag **out) {
    if (!out || !indptr_dst || (e && !indices_src) || block < 2 || block > 16 || hubs < 2) return ROF_ERR_ARG;
    if (indptr_dst[0] != 0 || indptr_dst[n] != e) return ROF_ERR_RANGE;
    for (u32 v = 0; v < n; ++v)
        if (indptr_dst[v] > indptr_dst[v + 1]) return ROF_ERR_RANGE;
    bool ok = true;
#pragma omp parallel for schedule(static) reduction(&& : ok)
    for (u64 j = 0; j < e; ++j)
        if (indices_src[j] >= n) ok = false;
    if (!ok) return ROF_ERR_RANGE;

    rof_bag *bag = new (std::nothrow) rof_bag;
    if (!bag) return ROF_ERR_ALLOC;
    try {
        // 1. hubs: the sources that appear in the most rows (ties: smaller id first)
        vec occ(n, 0);
#pragma omp parallel for schedule(static)
        for (u64 j = 0; j < e; ++j) {
#pragma omp atomic
            occ[indices_src[j]]++;
        }
        vec cand;
        for (u32 s = 0; s < n; ++s)
            if (occ[s] >= 2) cand.push_back(s);
        auto more = [&occ](u32 a, u32 b) { return occ[a] != occ[b] ? occ[a] > occ[b] : a < b; };
        if (cand.size() > hubs) {
            std::nth_element(cand.begin(), cand.begin() + hubs, cand.end(), more);
            cand.resize(hubs);
        }
        std::sort(cand.begin(), cand.end(), more);
        const u32 H = (u32)cand.size();
        const u32 nb = (H + block - 1) / block;
        std::vector<int32_t> rank(n, -1);
        for (u32 i = 0; i < H; ++i) rank[cand[i]] = (int32_t)i;

        // 2. every (block, pattern, row) with at least two hubs
        const int T = omp_get_max_threads();
        std::vector<std::vector<Seen>> local(T);
#pragma omp parallel
        {
            std::vector<uint16_t> mask(nb, 0);
            vec touched;
            std::vector<Seen> &mine = local[omp_get_thread_num()];
#pragma omp for schedule(dynamic, 1024)
            for (u32 v = 0; v < n; ++v)
                row_patterns(indices_src, indptr_dst[v], indptr_dst[v + 1], rank.data(), block, mask, touched,
                             [&](u32 blk, u32 m) { mine.push_back(Seen{make_key(blk, m), v}); });
        }
        std::vector<Seen> seen;
        {
            size_t total = 0;
            for (auto &l : local) total += l.size();
            seen.reserve(total);
            for (auto &l : local) {
                seen.insert(seen.end(), l.begin(), l.end());
                std::vector<Seen>().swap(l);
            }
        }
        __gnu_parallel::sort(seen.begin(), seen.end());

        // 3. candidates that repay themselves become shared parts, in (block, pattern) order
        std::vector<u64> shared_key;          // ascending
        std::vector<u64> shared_beg;          // start of the run in `seen`
        vec &ucol = bag->arr["uniqpart_column_index"], &uptr = bag->arr["uniqpart_pointers"];
        vec &dptr = bag->arr["part2Node_ptr"], &dcol = bag->arr["part2Node_col"];
        uptr.push_back(0);
        dptr.push_back(0);
        for (size_t i = 0; i < seen.size();) {
            size_t j = i;
            while (j < seen.size() && seen[j].key == seen[i].key) ++j;
            const u64 cnt = j - i, len = (u64)__builtin_popcount((u32)(seen[i].key & 0xffff));
            if ((cnt - 1) * len > cnt + 1) {
                shared_key.push_back(seen[i].key);
                shared_beg.push_back(i);
                const u32 blk = (u32)(seen[i].key >> 16), m = (u32)(seen[i].key & 0xffff);
                vec members;
                for (int b = 0; b < block; ++b)
                    if (m >> b & 1) members.push_back(cand[(size_t)blk * block + b]);
                std::sort(members.begin(), members.end());
                ucol.insert(ucol.end(), members.begin(), members.end());
                uptr.push_back((u32)ucol.size());
                for (size_t q = i; q < j; ++q) dcol.push_back(seen[q].row);   // ascending: sorted by (key, row)
                dptr.push_back((u32)dcol.size());
            }
            i = j;
        }
        const u64 G = shared_key.size();
        std::vector<Seen>().swap(seen);

        // 4. what is left of every row, in its original order, in chunks of `block`
        auto is_shared = [&shared_key](u64 key) { return std::binary_search(shared_key.begin(), shared_key.end(), key); };
        vec left(n, 0);   // neighbours of v that no shared part of v covers
#pragma omp parallel
        {
            std::vector<uint16_t> mask(nb, 0);
            vec touched;
#pragma omp for schedule(dynamic, 1024)
            for (u32 v = 0; v < n; ++v) {
                u32 covered = 0;
                row_patterns(indices_src, indptr_dst[v], indptr_dst[v + 1], rank.data(), block, mask, touched,
                             [&](u32 blk, u32 m) {
                                 if (is_shared(make_key(blk, m))) covered += (u32)__builtin_popcount(m);
                             });
                left[v] = indptr_dst[v + 1] - indptr_dst[v] - covered;
            }
        }
        std::vector<u64> chunk_at(n + 1, 0), col_at(n + 1, 0);
        for (u32 v = 0; v < n; ++v) {
            chunk_at[v + 1] = chunk_at[v] + (left[v] + block - 1) / block;
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
#pragma omp parallel
        {
            std::vector<uint16_t> mask(nb, 0), drop(nb, 0);
            vec touched;
#pragma omp for schedule(dynamic, 1024)
            for (u32 v = 0; v < n; ++v) {
                const u64 beg = indptr_dst[v], end = indptr_dst[v + 1];
                // hubs of v that its shared parts cover, as one mask per block
                vec mine;
                row_patterns(indices_src, beg, end, rank.data(), block, mask, touched, [&](u32 blk, u32 m) {
                    if (is_shared(make_key(blk, m))) {
                        drop[blk] = (uint16_t)m;
                        mine.push_back(blk);
                    }
                });
                u64 at = ncol0 + col_at[v];
                for (u64 j = beg; j < end; ++j) {
                    const u32 s = indices_src[j];
                    const int32_t r = rank[s];
                    if (r >= 0) {
                        const u32 blk = (u32)r / (u32)block, bit = 1u << ((u32)r % (u32)block);
                        if (drop[blk] & bit) {
                            drop[blk] &= (uint16_t)~bit;   // a repeated occurrence is an ordinary neighbour again
                            continue;
                        }
                    }
                    ucol[at++] = s;
                }
                for (u32 blk : mine) drop[blk] = 0;
                const u64 chunks = chunk_at[v + 1] - chunk_at[v];
                for (u64 c = 0; c < chunks; ++c) {
                    const u64 w = G + chunk_at[v] + c;
                    const u64 stop = std::min<u64>((c + 1) * (u64)block, left[v]);
                    uptr[w + 1] = (u32)(ncol0 + col_at[v] + stop);
                    dptr[w + 1] = (u32)(nd0 + chunk_at[v] + c + 1);
                    dcol[nd0 + chunk_at[v] + c] = v;
                }
            }
        }
        vec &hub_ids = bag->arr["hub_ids"];
        hub_ids = cand;
        bag->arr["shared_parts"] = vec{(u32)G};
    } catch (const std::bad_alloc &) {
        delete bag;
        return ROF_ERR_ALLOC;
    }
    *out = bag;
    return ROF_OK;
}
