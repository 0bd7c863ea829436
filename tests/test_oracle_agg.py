"""Pins the aggregation oracle (oracle/agg_oracle.c).  The upstream CUDA kernels cannot run here,
so the checks are mathematical: a brute-force edge loop, the float64 closed form computed with scipy
(a textbook sym-normalised SpMM), correct rounding of the reciprocal square root, and the identity
that v1/v2 plans only re-bracket the same sum."""
from decimal import Decimal, getcontext

import numpy as np
import pytest

from helpers import strict_excess, toy_csr

from artifact_amd.graphgen import features, rmat_csr


def _brute(indptr, indices, x, deg, normalized=True):
    n = len(indptr) - 1
    out = np.zeros((n, x.shape[1]))
    for v in range(n):
        for k in range(indptr[v], indptr[v + 1]):
            u = indices[k]
            out[v] += x[u] / np.sqrt(float(deg[u])) if normalized else x[u]
        if normalized and indptr[v + 1] > indptr[v]:
            out[v] /= np.sqrt(float(deg[v]))
    return out


def test_closed_form_equals_edge_loop_on_toy(oracle):
    ip, ix = toy_csr()
    x = features(10, 4, seed=1).astype(np.float64)
    deg = np.diff(ip).astype(np.float32)
    assert np.allclose(oracle.closed_form(ip, ix, x, deg), _brute(ip, ix, x, deg), rtol=1e-13, atol=1e-13)
    assert np.allclose(oracle.closed_form(ip, ix, x, normalized=False), _brute(ip, ix, x, deg, False), rtol=1e-13)


def test_closed_form_known_answer(oracle):
    # path graph 0-1-2 with degrees 1,2,1: out[1] = (x0/1 + x2/1)/sqrt(2), out[0] = x1/sqrt(2)
    ip = np.array([0, 1, 3, 4], dtype=np.int32)
    ix = np.array([1, 0, 2, 1], dtype=np.int32)
    x = np.array([[1.0], [10.0], [100.0]])
    got = oracle.closed_form(ip, ix, x)
    assert np.allclose(got[:, 0], [10 / np.sqrt(2), 101 / np.sqrt(2), 10 / np.sqrt(2)], rtol=1e-15)


def test_rsqrt_is_correctly_rounded(oracle):
    getcontext().prec = 60
    rng = np.random.default_rng(3)
    vals = np.concatenate([np.arange(1, 300, dtype=np.float32), rng.integers(1, 1 << 20, 300).astype(np.float32),
                           rng.random(50).astype(np.float32) + 0.01])
    got = oracle.rsqrt_rn(vals)
    for d, r in zip(vals, got):
        exact = Decimal(1) / Decimal(float(d)).sqrt()
        err = abs(Decimal(float(r)) - exact)
        lo, hi = np.nextafter(r, np.float32(0)), np.nextafter(r, np.float32(np.inf))
        assert err <= abs(Decimal(float(lo)) - exact) and err <= abs(Decimal(float(hi)) - exact), d
        assert oracle.lib().orc_rsqrt_rn(float(d)) == r


@pytest.mark.parametrize("ps", [2, 3, 5])
def test_kernel_restatements_agree_with_closed_form(oracle, ps):
    ip, ix = rmat_csr(600, 9, seed=40 + ps, self_loops=True)
    n = len(ip) - 1
    x = features(n, 13, seed=4)
    deg = np.diff(ip).astype(np.float32)
    plan = oracle.oracle_plan(ip, ix, ps)
    want = oracle.closed_form(ip, ix, x, deg)
    gnna = oracle.agg_parts(x, deg, ix, plan["part_ptr"], plan["part2Node"])
    v1, cache = oracle.agg_v1(x, deg, plan["new_indices_src"], plan["part_ptr"], plan["part2Node"],
                              plan["part_cache_flagindex"], plan["part_pointers_cache"], plan["column_index_cache"])
    v2 = oracle.agg_v2(x, deg, plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"],
                       plan["part2Node_col"])
    for got in (gnna, v1, v2):
        assert np.allclose(got, want, rtol=1e-5, atol=2e-6)
    assert (cache[:, -1] == 1.0).all()                      # ready flags (cu:485)
    # a cache row is the src-normalised sum of its sources
    r = oracle.rsqrt_rn(deg).astype(np.float64)
    cp, cc = plan["part_pointers_cache"], plan["column_index_cache"]
    for k in range(min(len(cp) - 1, 20)):
        s = cc[cp[k]:cp[k + 1]]
        assert np.allclose(cache[k, :-1], (x[s] * r[s, None]).sum(0), rtol=1e-5, atol=1e-6)


def test_sag_is_plain_sum(oracle):
    ip, ix = rmat_csr(400, 7, seed=50)
    x = features(len(ip) - 1, 6, seed=5)
    plan = oracle.oracle_plan(ip, ix, 3)
    deg = np.diff(ip).astype(np.float32)
    got = oracle.agg_parts(x, deg, ix, plan["part_ptr"], plan["part2Node"], normalized=False)
    assert np.allclose(got, oracle.closed_form(ip, ix, x, normalized=False), rtol=1e-5, atol=1e-5)
    ones = oracle.agg_parts(np.ones((len(ip) - 1, 2), np.float32), deg, ix, plan["part_ptr"], plan["part2Node"], False)
    assert np.array_equal(ones[:, 0], deg)                   # exact: small integers


def test_cpu_baseline_port_matches(oracle):
    ip, ix = rmat_csr(500, 8, seed=60, self_loops=True)
    x = features(len(ip) - 1, 11, seed=6)
    deg = np.diff(ip).astype(np.float32)
    got = oracle.spmm_rows(x, oracle.rsqrt_rn(deg), ip, ix, True)
    assert np.allclose(got, oracle.closed_form(ip, ix, x, deg), rtol=1e-5, atol=2e-6)
    got = oracle.spmm_rows(x, oracle.rsqrt_rn(deg), ip, ix, False)
    assert np.allclose(got, oracle.closed_form(ip, ix, x, normalized=False), rtol=1e-5, atol=1e-5)


def test_reference_order_fp32_itself_misses_the_strict_bar(oracle):
    """The GPU parity checks accept |got - want| <= 1e-6 + 1e-5*|want| + 1e-5*sum|terms|.  The last term is there
    because long fp32 sums whose terms cancel cannot meet the first two in *any* order of summation, the
    reference's included.  Measured here, on the inputs of the randomised GPU cases
    (tests/test_gpu_random_schedules.py; rows of up to n neighbours, widths up to 300): fp32 arithmetic in the
    upstream kernel's own order (oracle/agg_oracle.c: parts of ps neighbours in CSR order) lies beyond the strict bar
    on some of the elements (rows of hundreds to thousands of neighbours), by up to 16x, and always inside the
    summation bound.  The GPU test asserts per case that the kernel's largest error, in units of sum|terms|, is
    within 4x of this reference's."""
    from helpers import closed_form_case, random_schedule_case, reference_order_fp32

    compared = beyond = 0
    worst, worst_300 = 0.0, 0.0
    for seed in [1000 * block + case for block in range(12) for case in range(10)]:
        c = random_schedule_case(seed)
        if c["bf16_in"] or c["bf16_out"]:
            continue
        want, mag = closed_form_case(oracle, c)
        ref32 = reference_order_fp32(oracle, c)
        assert (np.abs(ref32 - want) <= 1e-6 + 1e-5 * np.abs(want) + 1e-5 * mag).all(), seed
        b, w = strict_excess(ref32, want)
        compared += ref32.size
        beyond += b
        worst = max(worst, w)
        if c["feat"] == 300:
            worst_300 = max(worst_300, w)
    print(f"reference-order fp32 against float64 on the randomised cases: {compared} elements, {beyond} "
          f"({100.0 * beyond / compared:.4f} %) beyond 1e-6 + 1e-5*|want|, worst {worst:.1f}x the strict bar "
          f"(width 300: {worst_300:.1f}x)")
    assert beyond > 20 and worst > 10.0


def test_reference_order_fp32_meets_the_strict_bar_on_short_rows(oracle):
    """... and on the small R-MAT graph of the GPU width test (rows of a few dozen neighbours, normalised) the same
    restatement stays at a fraction of the strict bar at every width, so there the bar is a real check."""
    from artifact_amd import reuse_search_ext as R
    from artifact_amd.graphgen import make_workload

    indptr, indices = make_workload("c1", 2)
    n = len(indptr) - 1
    plan = R.build_plan(indptr, indices, 3)
    deg = np.diff(indptr).astype(np.float32)
    for feat in (47, 300):
        x = features(n, feat, seed=7)
        ref32 = oracle.agg_v2(x, deg, plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"],
                              plan["part2Node_col"])
        assert strict_excess(ref32, oracle.closed_form(indptr, indices, x, deg)) [1] < 0.5
