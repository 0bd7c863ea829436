"""The dynamic greedy reuse search (rof_plan_dynamic_greedy).  Upstream only sketches it in a comment
(reuse_search_ext.h:305-321), so there is no upstream output to be on a par with; what is checked is
(1) validity -- the plan, read as upstream's v2 tensors, expands to exactly the graph's edge multiset
(invariant of reuse_search_ext.h:537-636), (2) that it picks what an independent, eager Python statement of the
sketch picks, in the same order, (3) the property the relaxation rests on (two shared parts of one destination
never share a source), (4) that it never saves less than upstream's static greedy on graphs where sources are
contended, and (5) that it runs through the device layout."""
import numpy as np
import pytest
import scipy.sparse as sp

from helpers import V2_KEYS, emulate_schedule, toy_csr

from artifact_amd import reuse_search_ext as R
from artifact_amd._lib import RofError
from artifact_amd.graphgen import make_workload
from artifact_amd.layout import Layout
from test_hub_patterns import edge_multiset, expand


def eager_dynamic_greedy(ip, ix, ps, ip_out=None, ix_out=None):
    """The sketch, literally: candidates = full parts (first of each distinct source tuple) with >= 2 destinations
    in the intersection of their sources' out-neighbour sets; repeat { take the candidate with the largest current
    set (ties: lowest part index); every other candidate sharing a source with it loses its destinations }."""
    n = len(ip) - 1
    if ip_out is None:
        ip_out, ix_out = ip, ix
    outs = [set(ix_out[ip_out[s]:ip_out[s + 1]].tolist()) for s in range(n)]
    cands, seen, p = {}, set(), 0
    for v in range(n):
        row = ix[ip[v]:ip[v + 1]]
        for k in range(0, len(row), ps):
            part = tuple(row[k:k + ps].tolist())
            if len(part) == ps and part not in seen:
                dst = set.intersection(*(outs[s] for s in part))
                if len(dst) >= 2:
                    seen.add(part)
                    cands[p] = (part, dst)
            p += 1
    picks = []
    while True:
        alive = [(len(d), -q) for q, (_, d) in cands.items() if len(d) >= 2]
        if not alive:
            break
        q = -max(alive)[1]
        part, dst = cands.pop(q)
        picks.append((q, part, sorted(dst)))
        for other, (opart, odst) in cands.items():
            if set(opart) & set(part):
                odst -= dst
    return picks


def random_contended_graph(rng, n, ps):
    """Directed; rows are unions of a few overlapping source sets, so that candidates contend for sources."""
    pool = [np.sort(rng.choice(n, ps + int(rng.integers(0, 3)), replace=False)) for _ in range(max(2, n // 6))]
    rows = []
    for v in range(n):
        k = int(rng.integers(0, min(4, len(pool) + 1)))
        cols = np.concatenate([pool[j] for j in rng.choice(len(pool), k, replace=False)] +
                              [rng.choice(n, int(rng.integers(0, 4)), replace=False)]) if k else np.zeros(0, np.int64)
        rows.append(np.unique(cols))
    ip = np.r_[0, np.cumsum([len(r) for r in rows])].astype(np.uint32)
    ix = (np.concatenate(rows) if ip[-1] else np.zeros(0)).astype(np.uint32)
    t = sp.csr_matrix((np.ones(len(ix), np.int8), ix, ip), shape=(n, n)).tocsc()
    return ip, ix, t.indptr.astype(np.uint32), t.indices.astype(np.uint32)


def check_plan(plan, ip, ix, ps, picks=None):
    n = len(ip) - 1
    up, dp = plan["uniqpart_pointers"].astype(np.int64), plan["part2Node_ptr"].astype(np.int64)
    uc, dc = plan["uniqpart_column_index"], plan["part2Node_col"]
    G = plan["shared_parts"]
    assert len(up) == len(dp) and up[0] == 0 and dp[0] == 0 and (np.diff(up) >= 1).all() and (np.diff(up) <= ps).all()
    src, dst = expand(plan)
    assert np.array_equal(edge_multiset(src, dst, n), edge_multiset(ix, np.repeat(np.arange(n), np.diff(ip)), n))
    assert (np.diff(up)[:G] == ps).all() and (np.diff(dp)[:G] >= 2).all() and (np.diff(dp)[G:] == 1).all()
    # no destination consumes two shared parts with a common source
    used = {}
    for g in range(G):
        for d in dc[dp[g]:dp[g + 1]].tolist():
            for s in uc[up[g]:up[g + 1]].tolist():
                assert (d, s) not in used, (d, s, g, used[(d, s)])
                used[(d, s)] = g
    if picks is not None:
        assert G == len(picks) and plan["index_picked"].tolist() == [q for q, _, _ in picks]
        for g, (_, part, dsts) in enumerate(picks):
            assert uc[up[g]:up[g + 1]].tolist() == list(part) and dc[dp[g]:dp[g + 1]].tolist() == dsts


@pytest.mark.parametrize("seed", range(8))
def test_picks_equal_the_eager_statement_on_random_directed_graphs(seed):
    rng = np.random.default_rng(seed)
    for case in range(12):
        n, ps = int(rng.integers(12, 90)), int(rng.integers(2, 5))
        ip, ix, ipo, ixo = random_contended_graph(rng, n, ps)
        plan = R.dynamic_greedy_plan(ip, ix, ps, ipo, ixo)
        check_plan(plan, ip, ix, ps, eager_dynamic_greedy(ip, ix, ps, ipo, ixo))


@pytest.mark.parametrize("wl,sd,ps", [("c1", 4, 3), ("c1", 3, 2), ("c4", 10, 3), ("hr", 8, 3), ("c3", 6, 4)])
def test_picks_equal_the_eager_statement_on_the_workloads(wl, sd, ps):
    ip, ix = make_workload(wl, sd)
    plan = R.dynamic_greedy_plan(ip, ix, ps)
    check_plan(plan, ip, ix, ps, eager_dynamic_greedy(ip, ix, ps))


@pytest.mark.parametrize("wl,sd", [("c4", 5), ("c2", 3), ("hr", 5)])
def test_finds_at_least_what_the_static_greedy_finds(wl, sd):
    """Gathers saved = sum over shared parts of (consumers - 1) * part size.  The dynamic rule's first pick is the
    static rule's first pick, and a part the static rule takes is never lost, only trimmed by earlier picks that
    the static rule would have let block it entirely -- so on these graphs it saves at least as much."""
    ip, ix = make_workload(wl, sd)
    e = len(ix)
    dyn = R.dynamic_greedy_plan(ip, ix, 3)
    check_plan(dyn, ip, ix, 3)
    up = R.build_plan(ip, ix, 3)
    save = lambda p: e - len(p["uniqpart_column_index"])
    assert save(dyn) >= save(up) > 0
    assert dyn["candidates"] >= dyn["shared_parts"] >= len(up["index_picked"])


def test_plan_runs_through_the_device_layout(oracle):
    ip, ix = make_workload("c4", 5)
    n = len(ip) - 1
    plan = R.dynamic_greedy_plan(ip, ix, 3)
    lay = Layout.from_v2(*(plan[k] for k in V2_KEYS), n, 3, min_consumers=2)
    ex, st = lay.export(), lay.stats()
    assert ex["canonical"] and st["materialised_groups"] > 0
    for k in V2_KEYS:
        assert np.array_equal(ex[k].view(np.uint32), plan[k]), k
    x = np.random.default_rng(0).standard_normal((n, 2))
    d = np.diff(ip)
    r = np.zeros(n)
    r[d > 0] = 1.0 / np.sqrt(d[d > 0])
    got = emulate_schedule(ex, n, x, lambda c: r[c], lambda v: r[v], st["partial_rows"])
    assert np.allclose(got, oracle.closed_form(ip, ix, x), rtol=1e-12, atol=1e-12)


def test_arguments_are_checked():
    ip, ix = toy_csr()
    with pytest.raises(RofError):
        R.dynamic_greedy_plan(ip, ix, 1)
    bad = ix.copy()
    bad[0] = 10
    with pytest.raises(RofError, match="out of range"):
        R.dynamic_greedy_plan(ip, bad, 3)
    with pytest.raises(RofError, match="out of range"):       # out-lists that are not the transpose of the in-lists
        n = 12
        ipd = np.arange(0, 3 * n + 1, 3, dtype=np.uint32)
        ixd = np.r_[np.tile([0, 1, 2], 2), np.tile([3, 4, 5], n - 2)].astype(np.uint32)   # rows 0, 1 gather 0, 1, 2
        ipo = np.r_[0, n, 2 * n, np.full(n - 2, 3 * n)].astype(np.uint32)   # yet 0, 1, 2 claim to reach every row
        ixo = np.tile(np.arange(n, dtype=np.uint32), 3)
        R.dynamic_greedy_plan(ipd, ixd, 3, ipo, ixo)
    empty = R.dynamic_greedy_plan(np.zeros(5, np.uint32), np.zeros(0, np.uint32), 3)
    assert empty["shared_parts"] == 0 and empty["uniqpart_pointers"].tolist() == [0]
    toy = R.dynamic_greedy_plan(ip, ix, 3)                      # upstream's worked example: the same two parts
    assert toy["index_picked"].tolist() == [0, 4]
    check_plan(toy, ip, ix, 3, eager_dynamic_greedy(ip, ix, 3))
