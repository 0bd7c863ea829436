"""Drop-in for the upstream `reuse_search_ext` pybind module (the CPU reuse-plan builder).

Same six functions, argument order, dtypes (uint32 arrays; int32 accepted) and return orders as
ROF/reuse_search_ext/src/reuse_search_ext.cc:260-271, backed by the OpenMP builder in librof.so
whose arrays equal the upstream ones bit for bit.  One deliberate difference: the per-part
intersection lists are returned as a lazy sequence (`PartIntersectList`) instead of one numpy
array per part, because materialising them all is quadratic in hub degree; indexing, len() and
iteration behave like the upstream list.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import bag_take, check, ptr, u32

__all__ = ["py_inverse_csc_or_csr", "py_split_part", "py_get_part_intersect", "py_greedy_max_reuse",
           "py_reorganize_indices", "py_reorganize_indices_uniquely", "PartIntersectList", "build_plan",
           "hub_pattern_plan"]


class PartIntersectList:
    """Sequence of uint32 arrays, one per part, computed on demand (cc:136-140 builds them all)."""

    def __init__(self, part_ptr, indices_src, indptr_src, indices_dst, part_size, discard):
        self._pp, self._isrc, self._ips, self._idst = part_ptr, indices_src, indptr_src, indices_dst
        self._ps, self._discard = int(part_size), bool(discard)

    def __len__(self):
        return len(self._pp) - 1

    def lists_of(self, which):
        """(ptr, data) CSR of the lists of the parts named in `which`."""
        which = u32(which)
        h = C.c_void_p()
        check(_lib.lib().rof_part_intersect_lists(ptr(self._pp), len(self._pp) - 1, ptr(self._isrc), len(self._isrc),
                                                  ptr(self._ips), ptr(self._idst), len(self._ips) - 1, self._ps,
                                                  int(self._discard), ptr(which), len(which), C.byref(h)))
        r = bag_take(h, ["ptr", "data"])
        return r["ptr"], r["data"]

    def __getitem__(self, i):
        if isinstance(i, slice):
            idx = np.arange(len(self))[i]
            p, d = self.lists_of(idx)
            return [d[p[k]:p[k + 1]] for k in range(len(idx))]
        n = len(self)
        if i < 0:
            i += n
        if not 0 <= i < n:
            raise IndexError(i)
        _, d = self.lists_of(np.array([i], dtype=np.uint32))
        return d

    def __iter__(self):
        step = 1 << 16
        for s in range(0, len(self), step):
            idx = np.arange(s, min(len(self), s + step), dtype=np.uint32)
            p, d = self.lists_of(idx)
            for k in range(len(idx)):
                yield d[p[k]:p[k + 1]]


def py_inverse_csc_or_csr(indptr_dst, indices_src, indptr_src, indices_dst):
    """cc:51-78.  The last two arguments must be empty, as upstream demands (cc:64-68)."""
    if np.size(indptr_src) or np.size(indices_dst):
        raise AssertionError("indptr_src and indices_dst should be empty")
    ip, ix = u32(indptr_dst), u32(indices_src)
    h = C.c_void_p()
    check(_lib.lib().rof_transpose_csr(ptr(ip), ptr(ix), len(ip) - 1, len(ix), C.byref(h)))
    r = bag_take(h, ["indptr", "indices"])
    return [r["indptr"], r["indices"]]


def py_split_part(part_candidates, part2Node, indptr_dst, part_size):
    """cc:82-103 -> [part_ptr, part2Node, num_parts_per_node_acc]; the first two inputs are ignored
    placeholders exactly as upstream (ROF_main.py:71-75 passes empty arrays)."""
    ip = u32(indptr_dst)
    h = C.c_void_p()
    check(_lib.lib().rof_split_part(ptr(ip), len(ip) - 1, int(part_size), C.byref(h)))
    r = bag_take(h, ["part_ptr", "part2Node", "num_parts_per_node_acc"])
    return [r["part_ptr"], r["part2Node"], r["num_parts_per_node_acc"]]


def py_get_part_intersect(part_ptr_on_indices_src, indices_src, indptr_src, indices_dst, part_size,
                          discard_remainder_part=False):
    """cc:108-142 -> [part_intersect_list, [intersection_num_per_part]] (the count array sits in a
    one-element list, which callers index with [0]: ROF_main.py:98-100)."""
    pp, isrc, ips, idst = u32(part_ptr_on_indices_src), u32(indices_src), u32(indptr_src), u32(indices_dst)
    h = C.c_void_p()
    check(_lib.lib().rof_part_intersect_count(ptr(pp), len(pp) - 1, ptr(isrc), len(isrc), ptr(ips), ptr(idst),
                                              len(ips) - 1, int(part_size), int(bool(discard_remainder_part)),
                                              C.byref(h)))
    cnt = bag_take(h, ["intersect_count"])["intersect_count"]
    return [PartIntersectList(pp, isrc, ips, idst, part_size, discard_remainder_part), [cnt]]


def py_greedy_max_reuse(intersection_num_per_part, part_ptr_on_indices_src, indices_src):
    """cc:145-160 -> [index_ordered, index_picked].  Accepts the one-element list the previous call
    returns (pybind flattens it upstream) or the bare array."""
    cnt = u32(np.asarray(intersection_num_per_part))
    pp, isrc = u32(part_ptr_on_indices_src), u32(indices_src)
    if len(cnt) != len(pp) - 1:
        raise ValueError("intersection_num_per_part must have one entry per part")
    h = C.c_void_p()
    check(_lib.lib().rof_greedy_max_reuse(ptr(cnt), len(cnt), ptr(pp), ptr(isrc), len(isrc), C.byref(h)))
    r = bag_take(h, ["index_ordered", "index_picked"])
    return [r["index_ordered"], r["index_picked"]]


def _picked_lists(intersection_per_part, picked):
    if isinstance(intersection_per_part, PartIntersectList):
        return intersection_per_part.lists_of(picked)
    lists = [u32(intersection_per_part[int(p)]) for p in picked]
    p = np.zeros(len(lists) + 1, dtype=np.uint32)
    if lists:
        np.cumsum([len(a) for a in lists], out=p[1:])
    d = np.concatenate(lists) if lists else np.empty(0, dtype=np.uint32)
    return p, u32(d)


def _reorganize(part_ptr, indices_src, intersection_per_part, index_picked, indptr_dst, acc, part_size, which, names):
    pp, isrc, picked, ipd, acc = u32(part_ptr), u32(indices_src), u32(index_picked), u32(indptr_dst), u32(acc)
    gptr, gdst = _picked_lists(intersection_per_part, picked)
    h = C.c_void_p()
    check(_lib.lib().rof_reorganize(ptr(pp), len(pp) - 1, ptr(isrc), len(isrc), ptr(picked), len(picked),
                                    gptr.ctypes.data, ptr(gdst), ptr(ipd), len(ipd) - 1, ptr(acc), int(part_size),
                                    which, C.byref(h)))
    return bag_take(h, names), pp


def py_reorganize_indices(part_ptr_on_indices_src, indices_src, intersection_per_part, index_picked, indptr_dst,
                          num_parts_per_node_acc, parts_size):
    """cc:169-211 -> [new_indices_src, part_ptr, part_pointers_cache, column_index_cache, part_cache_flagindex]."""
    r, pp = _reorganize(part_ptr_on_indices_src, indices_src, intersection_per_part, index_picked, indptr_dst,
                        num_parts_per_node_acc, parts_size, 1,
                        ["new_indices_src", "part_pointers_cache", "column_index_cache", "part_cache_flagindex"])
    return [r["new_indices_src"], pp.copy(), r["part_pointers_cache"], r["column_index_cache"],
            r["part_cache_flagindex"]]


def py_reorganize_indices_uniquely(part_ptr_on_indices_src, indices_src, intersection_per_part, index_picked,
                                   indptr_dst, num_parts_per_node_acc, parts_size):
    """cc:214-257 -> [uniqpart_column_index, uniqpart_pointers, part2Node_ptr, part2Node_col]."""
    r, _ = _reorganize(part_ptr_on_indices_src, indices_src, intersection_per_part, index_picked, indptr_dst,
                       num_parts_per_node_acc, parts_size, 2,
                       ["uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col"])
    return [r["uniqpart_column_index"], r["uniqpart_pointers"], r["part2Node_ptr"], r["part2Node_col"]]


PLAN_ARRAYS = ("part_ptr", "part2Node", "num_parts_per_node_acc", "intersect_count", "index_ordered", "index_picked",
               "picked_dst_ptr", "picked_dst", "new_indices_src", "part_pointers_cache", "column_index_cache",
               "part_cache_flagindex", "uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col")


def build_plan(indptr_dst, indices_src, part_size, indptr_src=None, indices_dst=None, discard_remainder_part=True):
    """The whole upstream call sequence (ROF_evaluation/ROF_main.py:71-127) in one native call.
    Returns a dict of uint32 arrays; omit the out-neighbour CSR for a symmetric graph."""
    ipd, isrc = u32(indptr_dst), u32(indices_src)
    ips = None if indptr_src is None else u32(indptr_src)
    idst = None if indices_dst is None else u32(indices_dst)
    h = C.c_void_p()
    check(_lib.lib().rof_plan_build(ptr(ipd), ptr(isrc), None if ips is None else ips.ctypes.data,
                                    None if idst is None else ptr(idst), len(ipd) - 1, len(isrc), int(part_size),
                                    int(bool(discard_remainder_part)), C.byref(h)))
    return bag_take(h, PLAN_ARRAYS)


def hub_pattern_plan(indptr_dst, indices_src, hubs=16384, block=8):
    """A different reuse search (not upstream's; see rof_plan_hub_patterns in include/rof.h): shared parts are
    subsets of popularity-ranked hub blocks that many rows have in common.  Returns the four v2 arrays (same
    format as py_reorganize_indices_uniquely, reuse_search_ext.cc:214-257) plus "hub_ids", "shared_parts" and
    "part_size" (= block), the partSize to pass along with them."""
    ipd, isrc = u32(indptr_dst), u32(indices_src)
    h = C.c_void_p()
    check(_lib.lib().rof_plan_hub_patterns(ptr(ipd), ptr(isrc), len(ipd) - 1, len(isrc), int(hubs), int(block),
                                           C.byref(h)))
    plan = bag_take(h, ("uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col", "hub_ids",
                        "shared_parts"))
    plan["shared_parts"] = int(plan["shared_parts"][0])
    plan["part_size"] = int(block)
    return plan


def dynamic_greedy_plan(indptr_dst, indices_src, part_size, indptr_src=None, indices_dst=None):
    """The dynamic greedy that upstream sketches and leaves unfinished (reuse_search_ext.h:305-321; see
    rof_plan_dynamic_greedy in include/rof.h): the candidate part with the longest current intersection list is
    picked, conflicting candidates lose its destinations and stay in the race.  Returns the four v2 arrays (format
    of py_reorganize_indices_uniquely, reuse_search_ext.cc:214-257) plus "index_picked" (part indices in pick
    order), "shared_parts", "candidates" and "part_size"; omit the out-neighbour CSR for a symmetric graph."""
    ipd, isrc = u32(indptr_dst), u32(indices_src)
    ips = None if indptr_src is None else u32(indptr_src)
    idst = None if indices_dst is None else u32(indices_dst)
    h = C.c_void_p()
    check(_lib.lib().rof_plan_dynamic_greedy(ptr(ipd), ptr(isrc), None if ips is None else ips.ctypes.data,
                                             None if idst is None else ptr(idst), len(ipd) - 1, len(isrc),
                                             int(part_size), C.byref(h)))
    plan = bag_take(h, ("uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col",
                        "index_picked", "shared_parts", "candidates"))
    plan["shared_parts"] = int(plan["shared_parts"][0])
    plan["candidates"] = int(plan["candidates"][0])
    plan["part_size"] = int(part_size)
    return plan


def reuse_statistics(plan, part_size, num_edges):
    """The four reuse figures the upstream scripts print (ROF_evaluation/cuda/small-main.py:176-188)."""
    cnt = plan["intersect_count"][plan["index_picked"]].astype(np.int64)
    raw_parts = len(plan["intersect_count"])
    return {
        "raw_part_num": raw_parts, "raw_edge_num": int(num_edges),
        "reused_part_num": int(cnt.sum()), "reused_part_reduction": int((cnt - 1).sum()),
        "reused_edge_num": int(cnt.sum()) * part_size, "reused_edge_reduction": int((cnt - 1).sum()) * part_size,
        "reused_part_ratio": float(cnt.sum()) / max(1, raw_parts),
        "reused_edge_reduction_ratio": float((cnt - 1).sum()) * part_size / max(1, num_edges),
    }
