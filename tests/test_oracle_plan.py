"""Pins the plan oracle (oracle/plan_oracle.cpp) before anything is checked against it:
golden plans written by the upstream builder, the live upstream build where present, the worked
example, and structural invariants."""
import numpy as np
import pytest

from helpers import (STEP_KEYS, V1_KEYS, V2_KEYS, case_inputs, check_plan_invariants, golden_digests, golden_small, sha,
                     toy_csr)

from artifact_amd.graphgen import make_workload, rmat_csr

CASES = golden_small()


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_matches_upstream_golden_plans(oracle, name):
    ipd, isrc, ips, idst, ps, discard = case_inputs(CASES[name])
    got = oracle.oracle_plan(ipd, isrc, ps, ips, idst, discard)
    want = CASES[name]["out"]
    keys = STEP_KEYS + ("intersect_ptr", "intersect_data") + ((V1_KEYS + V2_KEYS) if discard else ())
    for k in keys:
        assert np.array_equal(got[k], want[k]), k


@pytest.mark.parametrize("key", sorted(golden_digests()))
def test_oracle_matches_upstream_digests(oracle, key):
    wl, rest = key.split(">>")
    sd, ps = rest.split("_ps")
    rec = golden_digests()[key]
    ip, ix = make_workload(wl, int(sd))
    assert rec["input_sha256"] == __import__("hashlib").sha256(ip.tobytes() + ix.tobytes()).hexdigest(), \
        "generator output changed: regenerate the fixtures"
    got = oracle.oracle_plan(ip, ix, int(ps))
    for k, d in rec["arrays"].items():
        assert len(got[k]) == d["len"] and sha(got[k]) == d["sha256"], k


def test_worked_example_values(oracle):
    """The 10-node example: values fixed by hand-following reuse_search_ext.h."""
    ip, ix = toy_csr()
    p = oracle.oracle_plan(ip, ix, 3)
    assert p["part_ptr"].tolist() == [0, 3, 6, 9, 10, 13, 14, 17, 18, 21, 22, 24, 26, 27, 28]
    assert p["part2Node"].tolist() == [0, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 7, 8, 9]
    assert p["intersect_count"].tolist() == [3, 3, 3, 0, 3, 0, 3, 0, 3, 0, 0, 0, 0, 0]
    assert p["index_picked"].tolist() == [0, 4]
    assert p["part_cache_flagindex"].tolist() == [1, 1, 1, 0, 2, 0, 2, 0, 2, 0, 0, 0, 0, 0]
    assert p["column_index_cache"].tolist() == [3, 4, 5, 0, 1, 2]
    assert p["uniqpart_column_index"].tolist() == [3, 4, 5, 0, 1, 2, 6, 7, 8, 9, 2, 7, 3, 6, 4, 5]
    assert p["uniqpart_pointers"].tolist() == [0, 3, 6, 7, 8, 9, 10, 12, 14, 15, 16]
    assert p["part2Node_ptr"].tolist() == [0, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14]
    assert p["part2Node_col"].tolist() == [0, 1, 2, 3, 4, 5, 2, 3, 4, 5, 6, 7, 8, 9]


@pytest.mark.parametrize("n,deg,ps,seed", [(300, 8, 3, 1), (300, 8, 2, 2), (1000, 12, 4, 3), (97, 5, 5, 4)])
def test_oracle_invariants(oracle, n, deg, ps, seed):
    ip, ix = rmat_csr(n, deg, seed)
    check_plan_invariants(ip, ix, ps, oracle.oracle_plan(ip, ix, ps))


def test_oracle_matches_live_upstream_build(oracle):
    if oracle.ref_module() is None:
        pytest.skip("oracle/_ref not built (upstream tree absent)")
    for seed, ps in ((31, 3), (32, 2), (33, 4)):
        ip, ix = rmat_csr(2000, 10, seed, self_loops=bool(seed & 1))
        a, b = oracle.oracle_plan(ip, ix, ps), oracle.ref_plan(ip, ix, ps)
        for k in b:
            assert np.array_equal(a[k], b[k]), (seed, k)


def test_transpose_csr(oracle):
    import scipy.sparse as sp

    rng = np.random.default_rng(0)
    a = sp.random(50, 50, density=0.1, random_state=rng, format="csr")
    a.sort_indices()
    tp, ti = oracle.oracle_transpose_csr(a.indptr, a.indices)
    at = a.T.tocsr()
    at.sort_indices()
    assert np.array_equal(tp, at.indptr) and np.array_equal(ti, at.indices)
