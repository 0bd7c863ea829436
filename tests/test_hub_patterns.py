"""The hub-pattern reuse search (rof_plan_hub_patterns): not an upstream algorithm, so there is no parity to
show; what is checked is (1) validity -- the plan, read as upstream's v2 tensors, expands to exactly the
graph's edge multiset, so it computes the same aggregation (invariant of reuse_search_ext.h:537-636),
(2) that it selects what an independent numpy statement of the rule selects, (3) that the CPU restatement
of upstream's v2 kernel gives the closed form on it, and (4) that it runs through the device layout."""
import numpy as np
import pytest

from helpers import V2_KEYS, emulate_schedule, toy_csr

from artifact_amd import reuse_search_ext as R
from artifact_amd._lib import RofError
from artifact_amd.graphgen import make_workload, rmat_csr
from artifact_amd.layout import Layout


def expand(plan):
    """(src, dst) pairs of a v2 plan: every source of a unique part reaches every consumer of that part."""
    up, dp = plan["uniqpart_pointers"].astype(np.int64), plan["part2Node_ptr"].astype(np.int64)
    uc, dc = plan["uniqpart_column_index"].astype(np.int64), plan["part2Node_col"].astype(np.int64)
    src, dst = [], []
    for w in range(len(up) - 1):
        s, d = uc[up[w]:up[w + 1]], dc[dp[w]:dp[w + 1]]
        src.append(np.repeat(s, len(d)))
        dst.append(np.tile(d, len(s)))
    return np.concatenate(src) if src else np.zeros(0, np.int64), np.concatenate(dst) if dst else np.zeros(0, np.int64)


def numpy_selection(ip, ix, hubs, block):
    """The rule restated with numpy set operations: {(block, pattern): sorted consumer rows} of the shared parts,
    hub ranks by (occurrences desc, id asc), a repeated neighbour counted once."""
    n = len(ip) - 1
    occ = np.bincount(ix, minlength=n)
    cand = np.flatnonzero(occ >= 2)
    cand = cand[np.lexsort((cand, -occ[cand]))][:hubs]
    rank = np.full(n, -1, np.int64)
    rank[cand] = np.arange(len(cand))
    seen = {}
    for v in range(n):
        r = np.unique(rank[ix[ip[v]:ip[v + 1]]])
        r = r[r >= 0]
        for blk in np.unique(r // block):
            bits = r[r // block == blk] % block
            if len(bits) >= 2:
                seen.setdefault((int(blk), int((1 << bits).sum())), []).append(v)
    keep = {}
    for (blk, pat), rows in seen.items():
        cnt, ln = len(rows), bin(pat).count("1")
        if (cnt - 1) * ln > cnt + 1:
            keep[(blk, pat)] = rows
    return cand, keep


def edge_multiset(src, dst, n):
    return np.sort(dst.astype(np.int64) * n + src.astype(np.int64))


@pytest.mark.parametrize("wl,sd,hubs,block", [("c1", 2, 64, 4), ("c1", 1, 256, 8), ("c4", 7, 512, 8), ("c2", 5, 100, 3),
                                               ("hr", 7, 1024, 16), ("c3", 7, 64, 2)])
def test_plan_is_valid_and_selects_what_the_rule_selects(wl, sd, hubs, block):
    ip, ix = make_workload(wl, sd)
    n = len(ip) - 1
    plan = R.hub_pattern_plan(ip, ix, hubs, block)
    assert plan["part_size"] == block
    up, dp = plan["uniqpart_pointers"].astype(np.int64), plan["part2Node_ptr"].astype(np.int64)
    G = plan["shared_parts"]
    assert len(up) == len(dp) and up[0] == 0 and dp[0] == 0 and (np.diff(up) >= 1).all() and (np.diff(up) <= block).all()
    # validity: exactly the graph's edges
    src, dst = expand(plan)
    rows = np.repeat(np.arange(n), np.diff(ip))
    assert np.array_equal(edge_multiset(src, dst, n), edge_multiset(ix, rows, n))
    # the selection, against the numpy restatement
    cand, keep = numpy_selection(ip, ix, hubs, block)
    assert np.array_equal(plan["hub_ids"], cand.astype(np.uint32))
    assert G == len(keep)
    uc, dc = plan["uniqpart_column_index"], plan["part2Node_col"]
    for w, key in enumerate(sorted(keep)):                    # shared parts come in (block, pattern) order
        blk, pat = key
        members = sorted(int(cand[blk * block + b]) for b in range(block) if pat >> b & 1)
        assert uc[up[w]:up[w + 1]].tolist() == members
        assert dc[dp[w]:dp[w + 1]].tolist() == keep[key]
    # the rest: one consumer each, nodes ascending, chunks full except a node's last
    assert (np.diff(dp)[G:] == 1).all()
    owners = dc[dp[G]:].astype(np.int64)
    assert (np.diff(owners) >= 0).all()
    lens = np.diff(up)[G:]
    last_of_node = np.r_[owners[1:] != owners[:-1], True] if len(owners) else np.zeros(0, bool)
    assert (lens[~last_of_node] == block).all()


def test_repeated_neighbours_stay_in_the_plan():
    """A CSR with duplicate entries (scipy sums them upstream, ROF_main.py:52-60, but the builder must not lose
    them): the expansion still equals the edge multiset."""
    rng = np.random.default_rng(3)
    n = 60
    rows = [np.sort(np.r_[rng.choice(8, size=5, replace=True), rng.choice(n, size=4, replace=False)]) for _ in range(n)]
    ip = np.r_[0, np.cumsum([len(r) for r in rows])].astype(np.uint32)
    ix = np.concatenate(rows).astype(np.uint32)
    plan = R.hub_pattern_plan(ip, ix, 8, 4)
    assert plan["shared_parts"] > 0
    src, dst = expand(plan)
    assert np.array_equal(edge_multiset(src, dst, n), edge_multiset(ix, np.repeat(np.arange(n), np.diff(ip)), n))


def test_upstream_v2_kernel_restatement_gives_the_closed_form_on_the_plan(oracle):
    ip, ix = make_workload("c4", 7)
    n = len(ip) - 1
    plan = R.hub_pattern_plan(ip, ix, 512, 8)
    assert plan["shared_parts"] > 0
    x = np.random.default_rng(1).standard_normal((n, 5)).astype(np.float32)
    deg = np.diff(ip).astype(np.float32)
    got = oracle.agg_v2(x, deg, *(plan[k] for k in V2_KEYS))
    want = oracle.closed_form(ip, ix, x, deg)
    mag = oracle.closed_form(ip, ix, np.abs(x), deg)
    assert (np.abs(got - want) <= 1e-6 + 1e-5 * mag).all()


def test_plan_runs_through_the_device_layout_and_saves_more_than_upstream_on_a_heavy_tailed_graph(oracle):
    ip, ix = make_workload("c4", 5)                           # R-MAT, 75 000 nodes
    n = len(ip) - 1
    plan = R.hub_pattern_plan(ip, ix, 4096, 8)
    lay = Layout.from_v2(*(plan[k] for k in V2_KEYS), n, 8, min_consumers=3)
    ex, st = lay.export(), lay.stats()
    assert ex["canonical"]
    for k in V2_KEYS:
        assert np.array_equal(ex[k].view(np.uint32), plan[k]), k
    x = np.random.default_rng(0).standard_normal((n, 2))
    r = np.zeros(n)
    d = np.diff(ip)
    r[d > 0] = 1.0 / np.sqrt(d[d > 0])
    got = emulate_schedule(ex, n, x, lambda c: r[c], lambda v: r[v], st["partial_rows"])
    assert np.allclose(got, oracle.closed_form(ip, ix, x), rtol=1e-12, atol=1e-12)
    up = R.build_plan(ip, ix, 3)
    lay_up = Layout.from_v2(*(up[k] for k in V2_KEYS), n, 3, min_consumers=3).stats()
    net = lambda s: len(ix) - s["gathered_rows"] - s["partial_reads"]
    assert net(st) > 2 * net(lay_up) > 0


def test_arguments_are_checked():
    ip, ix = toy_csr()
    for hubs, block in ((1, 4), (8, 1), (8, 17)):
        with pytest.raises(RofError):
            R.hub_pattern_plan(ip, ix, hubs, block)
    bad = ix.copy()
    bad[0] = 10
    with pytest.raises(RofError, match="out of range"):
        R.hub_pattern_plan(ip, bad, 8, 4)
    empty = R.hub_pattern_plan(np.zeros(5, np.uint32), np.zeros(0, np.uint32), 8, 4)
    assert empty["shared_parts"] == 0 and empty["uniqpart_pointers"].tolist() == [0]
    toy = R.hub_pattern_plan(ip, ix, 16, 4)                  # upstream's worked example: too small to share anything much
    src, dst = expand(toy)
    assert np.array_equal(edge_multiset(src, dst, 10), edge_multiset(ix, np.repeat(np.arange(10), np.diff(ip)), 10))
