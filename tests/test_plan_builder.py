"""The shipped plan builder (librof.so, CPU/OpenMP) must reproduce the upstream arrays bit for bit:
against the golden plans, the oracle on random graphs, and through the module-level mirror of the
upstream `reuse_search_ext` API."""
import hashlib

import numpy as np
import pytest

from helpers import (STEP_KEYS, V1_KEYS, V2_KEYS, case_inputs, check_plan_invariants, golden_digests, golden_small, sha,
                     toy_csr)

from artifact_amd import reuse_search_ext as R
from artifact_amd._lib import RofError
from artifact_amd.graphgen import make_workload, rmat_csr

CASES = golden_small()


@pytest.mark.parametrize("name", sorted(CASES))
def test_builder_matches_upstream_golden_plans(name):
    ipd, isrc, ips, idst, ps, discard = case_inputs(CASES[name])
    want = CASES[name]["out"]
    got = R.build_plan(ipd, isrc, ps, ips, idst, discard)
    keys = STEP_KEYS + ((V1_KEYS + V2_KEYS) if discard else ())
    for k in keys:
        assert np.array_equal(got[k], want[k]), k
    # the lists of the picked parts
    ip, data = want["intersect_ptr"], want["intersect_data"]
    for i, p in enumerate(got["index_picked"]):
        mine = got["picked_dst"][got["picked_dst_ptr"][i]:got["picked_dst_ptr"][i + 1]]
        assert np.array_equal(mine, data[ip[p]:ip[p + 1]])


@pytest.mark.parametrize("key", sorted(golden_digests()))
def test_builder_matches_upstream_digests(key):
    wl, rest = key.split(">>")
    sd, ps = rest.split("_ps")
    rec = golden_digests()[key]
    ip, ix = make_workload(wl, int(sd))
    assert rec["input_sha256"] == hashlib.sha256(ip.tobytes() + ix.tobytes()).hexdigest()
    got = R.build_plan(ip, ix, int(ps))
    for k, d in rec["arrays"].items():
        if k in got:
            assert len(got[k]) == d["len"] and sha(got[k]) == d["sha256"], k


@pytest.mark.parametrize("name", ["toy_ps3", "rmat200_ps4", "cliques_ps3", "directed_ps3"])
def test_stepwise_api_mirrors_upstream_call_sequence(name):
    """ROF_evaluation/ROF_main.py:71-127, one call per upstream function."""
    ipd, isrc, ips, idst, ps, discard = case_inputs(CASES[name])
    want = CASES[name]["out"]
    if ips is None:
        ips, idst = ipd, isrc
    e = np.empty(0, dtype=np.int32)
    pp, p2n, acc = R.py_split_part(e, e, ipd.astype(np.int32), ps)          # int32 in, like upstream callers
    ilist, cnt = R.py_get_part_intersect(pp, isrc, ips, idst, ps, discard)
    assert isinstance(cnt, list) and len(cnt) == 1                           # callers index [0]
    ordered, picked = R.py_greedy_max_reuse(cnt, pp, isrc)                  # the list is passed as is
    v1 = R.py_reorganize_indices(pp, isrc, ilist, picked, ipd, acc, ps)
    v2 = R.py_reorganize_indices_uniquely(pp, isrc, ilist, picked, ipd, acc, ps)
    for got, k in zip((pp, p2n, acc, cnt[0], ordered, picked), STEP_KEYS):
        assert got.dtype == np.uint32 and np.array_equal(got, want[k]), k
    for got, k in zip(v1, ("new_indices_src", "part_ptr", "part_pointers_cache", "column_index_cache",
                           "part_cache_flagindex")):
        assert np.array_equal(got, want[k]), k
    for got, k in zip(v2, V2_KEYS):
        assert np.array_equal(got, want[k]), k
    # the lazy list behaves like the upstream list of arrays
    assert len(ilist) == len(pp) - 1
    ip, data = want["intersect_ptr"], want["intersect_data"]
    for p in (0, len(ilist) // 2, len(ilist) - 1, -1):
        q = p % len(ilist)
        assert np.array_equal(ilist[p], data[ip[q]:ip[q + 1]])
    assert sum(len(a) for a in ilist) == len(data)
    # a plain python list of arrays is accepted too
    as_list = [data[ip[q]:ip[q + 1]] for q in range(len(ilist))]
    v2b = R.py_reorganize_indices_uniquely(pp, isrc, as_list, picked, ipd, acc, ps)
    for a, b in zip(v2, v2b):
        assert np.array_equal(a, b)


def test_inverse_csr_matches_oracle(oracle):
    ipd, isrc, ips, idst, _, _ = case_inputs(CASES["directed_ps3"])
    e = np.empty(0, dtype=np.uint32)
    got = R.py_inverse_csc_or_csr(ipd, isrc, e, e)
    assert np.array_equal(got[0], ips) and np.array_equal(got[1], idst)
    with pytest.raises(AssertionError):
        R.py_inverse_csc_or_csr(ipd, isrc, ips, idst)                        # reuse_search_ext.cc:64-68


@pytest.mark.parametrize("seed", range(8))
def test_builder_equals_oracle_on_random_graphs(oracle, seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(20, 1500))
    ip, ix = rmat_csr(n, int(rng.integers(2, 20)), 100 + seed, self_loops=bool(seed & 1))
    ps = int(rng.integers(2, 7))
    a, b = R.build_plan(ip, ix, ps), oracle.oracle_plan(ip, ix, ps)
    for k in a:
        if k in b:
            assert np.array_equal(a[k], b[k]), (seed, k)
    check_plan_invariants(ip, ix, ps, a)


def test_long_rows_take_the_position_table_path(oracle):
    """A hub row far beyond the linear-search cut-off, consuming many picked parts."""
    n = 700
    u = np.concatenate([np.zeros(n - 1, dtype=np.int64), np.ones(n - 2, dtype=np.int64), np.full(n - 3, 2)])
    v = np.concatenate([np.arange(1, n), np.arange(2, n), np.arange(3, n)])
    rng = np.random.default_rng(9)
    u = np.concatenate([u, rng.integers(0, n, 3000)])
    v = np.concatenate([v, rng.integers(0, n, 3000)])
    from artifact_amd.graphgen import csr_from_pairs
    ip, ix = csr_from_pairs(u, v, n)
    for ps in (2, 3):
        a, b = R.build_plan(ip, ix, ps), oracle.oracle_plan(ip, ix, ps)
        assert len(a["index_picked"]) > 50
        for k in a:
            if k in b:
                assert np.array_equal(a[k], b[k]), k


def test_unsorted_and_duplicate_neighbour_lists(oracle):
    """Upstream builds std::set from each out-list (h:194,204); rows need not be sorted or unique."""
    rng = np.random.default_rng(4)
    n = 60
    rows = [rng.integers(0, n, rng.integers(0, 12)).tolist() for _ in range(n)]      # repeats, unsorted
    ipd = np.zeros(n + 1, dtype=np.uint32)
    ipd[1:] = np.cumsum([len(r) for r in rows])
    isrc = np.array([c for r in rows for c in r], dtype=np.uint32)
    ips, idst = oracle.oracle_transpose_csr(ipd, isrc)
    perm_idst = idst.copy()
    for v in range(n):                                                                 # shuffle each out-list
        seg = perm_idst[ips[v]:ips[v + 1]]
        rng.shuffle(seg)
    for ps in (2, 3):
        a = R.build_plan(ipd, isrc, ps, ips, perm_idst)
        b = oracle.oracle_plan(ipd, isrc, ps, ips, perm_idst)
        for k in STEP_KEYS + V2_KEYS + V1_KEYS:
            assert np.array_equal(a[k], b[k]), k


def test_degenerate_inputs():
    ip = np.zeros(6, dtype=np.uint32)                        # five isolated nodes
    p = R.build_plan(ip, np.empty(0, dtype=np.uint32), 3)
    assert len(p["part2Node"]) == 0 and p["part_ptr"].tolist() == [0]
    assert p["uniqpart_pointers"].tolist() == [0] and p["part2Node_ptr"].tolist() == [0]
    ip, ix = toy_csr()
    p = R.build_plan(ip, ix, 100)                            # part_size larger than every row: no full part
    assert len(p["index_picked"]) == 0 and np.array_equal(p["uniqpart_column_index"], ix.astype(np.uint32))


def test_invalid_inputs_raise_instead_of_crashing():
    ip, ix = toy_csr()
    bad = ix.copy()
    bad[3] = 99
    with pytest.raises(RofError, match="out of range"):
        R.build_plan(ip, bad, 3)
    with pytest.raises(RofError, match="out of range"):
        R.build_plan(ip[::-1].copy(), ix, 3)
    with pytest.raises(RofError, match="invalid argument"):
        R.build_plan(ip, ix, 0)


def test_reuse_statistics_formulas():
    """ROF_evaluation/cuda/small-main.py:176-188."""
    ip, ix = toy_csr()
    p = R.build_plan(ip, ix, 3)
    s = R.reuse_statistics(p, 3, len(ix))
    assert s["reused_part_num"] == 6 and s["reused_part_reduction"] == 4
    assert s["reused_edge_num"] == 18 and s["reused_edge_reduction"] == 12
    assert s["raw_part_num"] == 14 and s["raw_edge_num"] == 28
