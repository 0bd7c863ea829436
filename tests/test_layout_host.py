"""Host side of the device layout: lossless round trip to the upstream v2 tensors, agreement of the
three input formats, and a numpy emulation of the execution schedule against the closed form."""
import numpy as np
import pytest

from helpers import V2_KEYS, emulate_schedule, toy_csr

from artifact_amd import reuse_search_ext as R
from artifact_amd._lib import RofError
from artifact_amd.graphgen import csr_from_pairs, make_workload, planted_reuse_csr, rmat_csr, sbm_csr
from artifact_amd.layout import Layout


def _v2(plan, n, ps, **o):
    return Layout.from_v2(plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"],
                          plan["part2Node_col"], n, ps, **o)


def _v1(plan, n, ps, **o):
    return Layout.from_v1(plan["new_indices_src"], plan["part_ptr"], plan["part2Node"], plan["part_cache_flagindex"],
                          plan["part_pointers_cache"], plan["column_index_cache"], n, ps, **o)


@pytest.mark.parametrize("wl,sd,ps", [("c1", 3, 3), ("c1", 2, 2), ("c1", 3, 5), ("c3", 6, 2), ("c2", 6, 4)])
def test_layout_round_trips_to_the_upstream_v2_plan_bit_exactly(wl, sd, ps):
    ip, ix = make_workload(wl, sd)
    n = len(ip) - 1
    plan = R.build_plan(ip, ix, ps)
    ex = _v2(plan, n, ps).export()
    assert ex["canonical"]
    for k in V2_KEYS:
        assert np.array_equal(ex[k].view(np.uint32), plan[k]), k
    # the canonical arrays: groups = picked parts with their consumers, residual = what is left per node
    P = len(plan["index_picked"])
    assert np.array_equal(ex["group_ptr"], plan["uniqpart_pointers"][:P + 1].view(np.int32))
    assert np.array_equal(ex["group_dst"], plan["picked_dst"].view(np.int32))
    assert ex["res_ptr"][-1] + ex["group_ptr"][-1] == len(plan["uniqpart_column_index"])
    # v1 tensors describe the same plan and must give the same canonical arrays
    ex1 = _v1(plan, n, ps).export()
    for k in ("group_ptr", "group_col", "group_dst_ptr", "group_dst", "res_ptr", "res_col"):
        assert np.array_equal(ex[k], ex1[k]), k


def test_toy_layout_literal():
    ip, ix = toy_csr()
    plan = R.build_plan(ip, ix, 3)
    ex = _v2(plan, 10, 3, min_consumers=2).export()
    assert ex["group_ptr"].tolist() == [0, 3, 6] and ex["group_col"].tolist() == [3, 4, 5, 0, 1, 2]
    assert ex["group_dst"].tolist() == [0, 1, 2, 3, 4, 5]
    assert ex["res_ptr"].tolist() == [0, 0, 0, 1, 2, 3, 4, 6, 8, 9, 10]
    assert ex["res_col"].tolist() == [6, 7, 8, 9, 2, 7, 3, 6, 4, 5]
    # two partial-sum tasks, ten destination rows; rows 0..2 read partial row 0, rows 3..5 partial row 1
    assert sorted(ex["g_task_out"].tolist()) == [0, 1]
    rows = {int(o): ex["b_col"][ex["b_task_ptr"][t]:ex["b_task_ptr"][t + 1]].tolist()
            for t, o in enumerate(ex["b_task_out"])}
    # feature rows of a task are listed by descending id (the default entry order), after the partial rows
    assert rows[0] == [10] and rows[2] == [10, 6] and rows[3] == [11, 7] and rows[6] == [7, 2] and rows[9] == [5]
    ex = _v2(plan, 10, 3, min_consumers=2, entry_order="plan").export()
    rows = {int(o): ex["b_col"][ex["b_task_ptr"][t]:ex["b_task_ptr"][t + 1]].tolist()
            for t, o in enumerate(ex["b_task_out"])}
    assert rows[6] == [2, 7] and rows[7] == [3, 6]
    ex = _v2(plan, 10, 3, min_consumers=2, entry_order="ascending").export()
    rows = {int(o): ex["b_col"][ex["b_task_ptr"][t]:ex["b_task_ptr"][t + 1]].tolist()
            for t, o in enumerate(ex["b_task_out"])}
    assert rows[6] == [2, 7] and rows[2] == [10, 6]


OPTS = [dict(), dict(disable_reuse=True), dict(min_consumers=2), dict(min_consumers=-1), dict(hub_split=24, segment=8),
        dict(hub_split=33, segment=32, min_consumers=2), dict(entry_order="plan", min_consumers=2),
        dict(entry_order="ascending", hub_split=24, segment=8)]


@pytest.mark.parametrize("opts", OPTS, ids=[str(o) for o in OPTS])
def test_schedule_computes_the_closed_form(oracle, opts):
    ip, ix = rmat_csr(400, 10, seed=77, self_loops=True)
    n = len(ip) - 1
    for ps in (2, 3):
        plan = R.build_plan(ip, ix, ps)
        lay = _v2(plan, n, ps, **opts)
        ex, st = lay.export(), lay.stats()
        x = np.random.default_rng(0).standard_normal((n, 3))
        r = 1.0 / np.sqrt(np.diff(ip).astype(np.float64))
        got = emulate_schedule(ex, n, x, lambda c: r[c], lambda v: r[v], st["partial_rows"])
        assert np.allclose(got, oracle.closed_form(ip, ix, x), rtol=1e-12, atol=1e-12)
        # bookkeeping used by the roofline report
        nref = int(ex["g_task_nref"].sum() + ex["s_task_nref"].sum() + ex["b_task_nref"].sum())
        nlds = int(ex["b_task_nlds"].sum())
        total = len(ex["g_col"]) + len(ex["s_col"]) + len(ex["b_col"]) + len(ex["b_lg_col"])
        assert st["partial_reads"] == nref and st["gathered_rows"] == total - nref - nlds and st["lds_reads"] == nlds
        assert st["edges"] == len(ix) and st["tasks_b"] == n
        assert st["partial_rows"] == st["materialised_groups"] + st["hub_segments"]
        if opts.get("disable_reuse"):
            assert st["gathered_rows"] == len(ix) and st["materialised_groups"] == 0
        if opts.get("min_consumers") == 2:                   # every group shared: the upstream saving (h:537-605)
            cnt = plan["intersect_count"][plan["index_picked"]].astype(np.int64)
            assert len(ix) - st["gathered_rows"] == ps * int((cnt - 1).sum())


def test_sharing_is_gated_by_the_bytes_it_saves():
    """Sharing through the workspace (workgroup-local sharing switched off): the same plan is executed with its
    groups shared when rows are wide and folded back when they are narrow: what one more launch has to repay is
    bytes (net saved gathers x row bytes, 16 per lane)."""
    ip, ix = make_workload("hr", 5)                          # 32 768 nodes, most neighbours in shared anchor sets
    n = len(ip) - 1
    plan = R.build_plan(ip, ix, 3)
    cnt = plan["intersect_count"][plan["index_picked"]].astype(np.int64)
    cnt = cnt[cnt >= 3]                                      # groups the per-group rule shares at ps = 3
    net = int(((cnt - 1) * 3 - cnt).sum())
    assert net * 32 * 16 < 256_000_000 <= net * 64 * 16      # 512-byte rows: below the gate; 1024-byte rows: above
    narrow = _v2(plan, n, 3, lanes_per_row=32, local_groups=-1).stats()
    wide = _v2(plan, n, 3, lanes_per_row=64, local_groups=-1).stats()
    assert narrow["materialised_groups"] == 0 and narrow["gathered_rows"] == len(ix)
    assert wide["materialised_groups"] == len(cnt)
    assert len(ix) - wide["gathered_rows"] - wide["partial_reads"] == net
    forced = _v2(plan, n, 3, lanes_per_row=32, min_consumers=3).stats()   # an explicit threshold bypasses the gate
    assert forced["materialised_groups"] == len(cnt)


@pytest.mark.parametrize("lanes,wl,sd,ps", [(16, "hr", 5, 3), (16, "hr", 6, 2), (64, "hr", 6, 4), (12, "hr", 5, 3),
                                            (32, "c1", 2, 2), (8, "c2", 5, 3)])
def test_consumers_of_a_group_are_clustered_into_workgroups_that_sum_it_in_lds(oracle, lanes, wl, sd, ps):
    """Short destinations that share groups are placed in one cluster (workgroup) whose local groups are summed once
    into LDS rows.  The exported schedule is executed in float64 (which also checks that LDS rows are read only
    inside the cluster that sums them) and the bookkeeping is checked.  local_groups=8: clusters that save 8 gathers
    are kept whatever they save in total (by default a plan's clusters must repay their launch: 64 MB of gathers,
    which these small graphs do not hold)."""
    ip, ix = make_workload(wl, sd)
    n = len(ip) - 1
    plan = R.build_plan(ip, ix, ps)
    lay = _v2(plan, n, ps, lanes_per_row=lanes, local_groups=8)
    if wl != "hr":
        assert _v2(plan, n, ps, lanes_per_row=lanes).stats()["cluster_workgroups"] == 0  # too little to repay a launch
    ex, st = lay.export(), lay.stats()
    sh = ex["b_shape"]
    x = np.random.default_rng(1).standard_normal((n, 2))
    r = 1.0 / np.sqrt(np.maximum(np.diff(ip), 1).astype(np.float64))
    got = emulate_schedule(ex, n, x, lambda c: r[c], lambda v: r[v], st["partial_rows"])
    assert np.allclose(got, oracle.closed_form(ip, ix, x), rtol=1e-12, atol=1e-12)
    assert st["cluster_workgroups"] == sh["lg_blocks"] and st["local_groups"] == len(ex["b_lg_task_ptr"]) - 1
    assert st["lds_reads"] == int(ex["b_task_nlds"].sum()) and st["lds_rows"] == (sh["lg_max_rows"] if sh["lg_blocks"] else 0)
    if wl == "hr":
        # planted reuse: almost every destination is served from LDS and most gathers disappear without any
        # partial row going through the workspace
        assert st["cluster_workgroups"] > 0 and st["materialised_groups"] == 0
        assert st["gathered_rows"] < 0.65 * len(ix)
        lens = np.diff(ex["b_lg_ptr"])
        assert lens.min() >= 1 and lens.max() <= st["lds_rows"] <= 32
        tf = ex["b_lg_task_first"]
        assert np.diff(tf).max() <= 64
        # every local group is read by at least two tasks of its cluster
        for b in range(min(sh["lg_blocks"], 50)):
            rows = []
            for t in range(tf[b], tf[b + 1]):
                rows += ex["b_col"][ex["b_task_ptr"][t]:ex["b_task_ptr"][t] + ex["b_task_nlds"][t]].tolist()
            cnt = np.bincount(rows, minlength=lens[b])
            assert (cnt >= 2).all()
    off = _v2(plan, n, ps, lanes_per_row=lanes, local_groups=-1).stats()
    assert off["cluster_workgroups"] == 0 and off["lds_reads"] == 0


@pytest.mark.parametrize("seed", range(12))
def test_random_graphs_with_shared_neighbour_sets_through_clusters(oracle, seed):
    """Random directed graphs whose rows are built from a pool of shared neighbour sets (so that many short rows
    consume the same groups), random lane counts, cuts and cluster thresholds: the exported schedule, run in float64,
    gives the closed form, and every structural rule of the clusters holds (helpers.emulate_schedule)."""
    import scipy.sparse as sp

    rng = np.random.default_rng(100 + seed)
    n = int(rng.integers(200, 1500))
    ps = int(rng.integers(2, 5))
    sets = [np.sort(rng.choice(n, ps * int(rng.integers(1, 4)), replace=False)) for _ in range(int(rng.integers(3, 40)))]
    rows = []
    for v in range(n):
        kind = rng.random()
        if kind < 0.1:
            rows.append(np.zeros(0, dtype=np.int64))
        elif kind < 0.75:
            pick = rng.choice(len(sets), int(rng.integers(1, 4)), replace=False)
            extra = rng.choice(n, int(rng.integers(0, 6)), replace=False)
            rows.append(np.unique(np.concatenate([sets[j] for j in pick] + [extra])))
        else:
            rows.append(np.unique(rng.choice(n, int(rng.integers(1, min(n, 200))), replace=False)))
    ip = np.r_[0, np.cumsum([len(r) for r in rows])].astype(np.int32)
    ix = np.concatenate(rows).astype(np.int32)
    t = sp.csr_matrix((np.ones(len(ix), np.int8), ix, ip), shape=(n, n)).tocsc()
    plan = R.build_plan(ip, ix, ps, t.indptr, t.indices)
    opts = dict(lanes_per_row=int(rng.choice([4, 8, 12, 16, 32, 64])), local_groups=int(rng.choice([1, 4, 8, 30])),
                hub_split=int(rng.choice([0, 24, 100])), segment=int(rng.choice([0, 8])),
                elem_bytes=int(rng.choice([2, 4])), entry_order=str(rng.choice(["descending", "plan", "ascending"])),
                share_scope=str(rng.choice(["all", "long_rows"])), min_consumers=int(rng.choice([0, 0, 2])))
    lay = _v2(plan, n, ps, **opts)
    ex, st = lay.export(), lay.stats()
    if opts["share_scope"] == "long_rows" and st["materialised_groups"]:
        # only rows that are cut into segments may reference a shared group: the references sit in segment tasks
        # (or in a row that sharing shortened below the cut), never in a row that was short to begin with
        b_ref_rows = ex["b_task_out"][(ex["b_task_nref"] > 0) & (np.diff(ex["b_task_ptr"]) > ex["b_task_nref"])]
        cut = st["hub_split"]   # the cut the layout took: the caller's, or the rule's for these sizes
        assert all(np.diff(ip)[v] > cut for v in b_ref_rows), opts
    x = rng.standard_normal((n, 2))
    w = rng.uniform(0.5, 2.0, n)
    got = emulate_schedule(ex, n, x, lambda c: w[c], lambda v: w[v], st["partial_rows"])
    a = sp.csr_matrix((np.ones(len(ix)), ix, ip), shape=(n, n))
    want = w[:, None] * (a @ (w[:, None] * x))
    assert np.allclose(got, want, rtol=1e-11, atol=1e-11), opts
    assert st["lds_reads"] == int(ex["b_task_nlds"].sum()) and st["cluster_workgroups"] == ex["b_shape"]["lg_blocks"]
    total = len(ex["g_col"]) + len(ex["s_col"]) + len(ex["b_col"]) + len(ex["b_lg_col"])
    nref = int(ex["g_task_nref"].sum() + ex["s_task_nref"].sum() + ex["b_task_nref"].sum())
    assert st["gathered_rows"] == total - nref - st["lds_reads"] <= len(ix)


@pytest.mark.parametrize("lanes,elem,row,cut,seg", [(64, 4, 0, 256, 32), (64, 4, 1024, 256, 32), (64, 4, 640, 1024, 128),
                                                    (32, 4, 0, 1024, 128), (20, 4, 0, 512, 128), (16, 4, 0, 1024, 128),
                                                    (12, 4, 0, 640, 160), (8, 0, 0, 640, 160),
                                                    (32, 2, 0, 256, 48), (20, 2, 0, 512, 128), (16, 2, 0, 1280, 320)])
def test_long_rows_are_cut_by_width_and_their_segments_swept_by_source_id(lanes, elem, row, cut, seg):
    """Default cut and segment by the rows a wavefront gathers at once, the bytes of a row and whether the caches
    can hold the matrix (the measured table in csrc/layout.cpp; this 600 000-row matrix is beyond them at 32 lanes
    and more, and at 20 lanes, where they hold it, two thirds of its edges lie in rows beyond the fine cut of 128: the
    dense rule's 512 / 128); the segment tasks come in the order of the highest source id they gather (each task lists its sources
    by descending id), long tasks before packed ones."""
    ip, ix = make_workload("c4", 2)                          # 600 000 rows: enough segments to fill the machine
    n = len(ip) - 1
    lay = Layout.from_csr(ip, ix, lanes_per_row=lanes, elem_bytes=elem, row_bytes=row)
    assert (lay.export()["hub_split"], lay.export()["segment"]) == (cut, seg)
    st0 = lay.stats()                                        # the same through the counters, without an export
    assert (st0["hub_split"], st0["segment"]) == (cut, seg)
    assert st0["longest_row_task"] == int(np.diff(lay.export()["b_task_ptr"]).max())
    ex, st = lay.export(), lay.stats()
    deg = np.diff(ip)
    assert st["hub_segments"] == int(np.ceil(deg[deg > cut] / seg).sum())
    b_len, b_ref = np.diff(ex["b_task_ptr"]), ex["b_task_nref"]
    assert b_len[b_ref == 0].max() <= cut and (b_len[b_ref > 0] == b_ref[b_ref > 0]).all()
    s_ptr, s_col = ex["s_task_ptr"], ex["s_col"]
    s_len = np.diff(s_ptr)
    assert s_len.max() == seg and (ex["s_task_nref"] == 0).all()
    for t in range(0, len(s_len), 997):                      # sources inside a task: descending
        assert (np.diff(s_col[s_ptr[t]:s_ptr[t + 1]]) < 0).all()
    first = s_col[s_ptr[:-1]]
    nw = st["wave_tasks_a"]
    groups = max(1, 64 // lanes)
    if nw + (len(s_len) - nw + groups - 1) // groups < 2 * 8192:
        # too few segment tasks to fill the machine twice: such a launch is bound by its longest task and runs
        # longest first, with the lower cut between wavefront-wide and packed tasks
        assert nw == int((s_len > 32).sum()) and (np.diff(s_len[:nw]) <= 0).all()
        return
    assert (np.diff(first[:nw]) <= 0).all() and (np.diff(first[nw:]) <= 0).all()
    assert nw == int((s_len > 64).sum()) and (s_len[:nw] > 64).all()
    # with the plan's own order inside tasks there is no sweep: segments come longest first
    ex2 = Layout.from_csr(ip, ix, lanes_per_row=lanes, elem_bytes=elem, row_bytes=row, entry_order="plan").export()
    first2 = ex2["s_col"][ex2["s_task_ptr"][:-1]]
    assert not (np.diff(first2[:nw]) <= 0).all() or nw < 2 or not (np.diff(first2[nw:]) <= 0).all()


def test_a_cluster_never_needs_more_lds_rows_than_fit_at_the_widest_launch():
    """A layout may be run at another width than it was built for; the widest LDS row there is (bf16 features at 64
    lanes: (64 * 8 + 4) * 4 = 2064 bytes) times the rows of any cluster stays within the 64 KB a workgroup may ask
    for, also for the default width, which gets the most rows."""
    ip, ix = make_workload("hr", 6)
    n = len(ip) - 1
    plan = R.build_plan(ip, ix, 3)
    for lanes, elem in ((0, 0), (4, 4), (4, 2), (16, 4), (64, 2)):
        ex = _v2(plan, n, 3, lanes_per_row=lanes, elem_bytes=elem, local_groups=1).export()
        assert 0 < ex["b_shape"]["lg_max_rows"] <= 31 and ex["b_shape"]["lg_max_rows"] * 2064 <= 64 * 1024


def test_small_matrices_keep_the_fine_cut():
    """A matrix that the 256 MB Infinity Cache can hold is cut at 128 / 32 up to three rows per wavefront (the
    2^18-node workload at 256 floats is exactly 256 MB), whatever the row bytes."""
    ip, ix = make_workload("c2", 0)
    for lanes, row, want in ((64, 640, (128, 32)), (64, 1000, (128, 32)), (32, 0, (128, 32)), (20, 0, (128, 32)),
                             (16, 0, (1024, 128)), (64, 1024, (128, 32)), (64, 2048, (256, 32))):
        ex = Layout.from_csr(ip, ix, lanes_per_row=lanes, row_bytes=row).export()
        assert (ex["hub_split"], ex["segment"]) == want, (lanes, row)


def test_a_row_of_the_whole_graph_gets_longer_segments():
    """The row that adds up a long row's partial sums is itself a chain of dependent reads, one per segment; a row
    so long that this chain would outlast the launch is cut into fewer, longer segments: at most
    max(64, chain limit / 2) of them at these four rows per wavefront (partial rows are read cold, at about twice the
    cached cost per entry; at wider rows a read costs no less than a memory latency shared by the reads in flight)."""
    n = 20000
    rng = np.random.default_rng(4)
    u, v = rng.integers(1, n, 2 * n), rng.integers(1, n, 2 * n)
    ip, ix = csr_from_pairs(np.r_[u, np.zeros(n - 1, np.int64)], np.r_[v, np.arange(1, n)], n, False)
    assert np.diff(ip)[0] == n - 1                           # node 0 is everybody's neighbour
    lay = Layout.from_csr(ip, ix, lanes_per_row=16)
    ex, st = lay.export(), lay.stats()
    limit = 3 * (15000 + len(ix) * 256 * 60 // 1000000) // (4 * (10 + 256 * 14 // 100))
    most = max(64, limit // 2)
    assert st["segment"] * most < n - 1                      # the rule's segments would be too many
    s_len = np.diff(ex["s_task_ptr"])
    hub = int(np.nonzero(ex["b_task_out"] == 0)[0][0])
    assert ex["b_task_nref"][hub] == np.diff(ex["b_task_ptr"])[hub] <= most
    assert s_len.max() == -(-(n - 1) // most) and st["longest_row_task"] <= max(st["hub_split"], most)
    x = np.random.default_rng(5).standard_normal((n, 2))
    got = emulate_schedule(ex, n, x, lambda c: 1.0, lambda r: 1.0, st["partial_rows"])
    want = np.zeros((n, 2))
    np.add.at(want, np.repeat(np.arange(n), np.diff(ip)), x[ix])
    assert np.allclose(got, want, rtol=1e-11, atol=1e-11)
    # one row per wavefront, rows of 640 bytes: a read costs 350 ns (700 ns of latency, two reads in flight)
    wide = Layout.from_csr(ip, ix, lanes_per_row=64, row_bytes=640)
    launch_ns = 15000 + len(ix) * 640 * 60 // 1000000
    most_wide = max(64, 3 * launch_ns // (4 * 350))
    exw = wide.export()
    hub = int(np.nonzero(exw["b_task_out"] == 0)[0][0])
    assert np.diff(exw["b_task_ptr"])[hub] == -(-(n - 1) // -(-(n - 1) // most_wide)) <= most_wide


def test_the_relative_cluster_gate_applies_only_to_graphs_with_local_sources():
    """A cluster takes its rows out of the tile order.  Where rows gather from their own neighbourhood (block model)
    that order is worth more than a small saving, and a cluster must remove an eighth of its rows' gathers; elsewhere
    every cluster that saves 8 gathers is kept (sets of 3 anchors x 64 members + 24 random neighbours: each cluster
    removes a tenth of its rows' gathers, and all of them together made the layer 9 % faster than none)."""
    def clusters(ip, ix, ps, **kw):
        plan = R.build_plan(ip, ix, ps)
        v2 = (plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"], plan["part2Node_col"],
              len(ip) - 1, ps)
        return [Layout.from_v2(*v2, lanes_per_row=16, **o).stats()["cluster_workgroups"] for o in ({}, dict(local_groups=8))]
    default, every = clusters(*planted_reuse_csr(1 << 18, 3, 64, 24, seed=5), 3)
    assert default == every > 8000
    default, every = clusters(*sbm_csr(64, 4096, 24, 2, 6), 2)
    assert default == 0 and every > 2000


def test_dense_graphs_are_cut_by_what_their_rows_look_like():
    """Dense graphs (two thirds of the edges in rows of more than 128 entries) are cut by whether a set of sources
    that one L2 can hold is popular (45 % of all gathers go to the 4 MB / row bytes longest rows).  Popular: the
    segments' cost counts, and wide rows on a cached matrix take 512 / 128 (256 / 64 for rows of 1 KB) instead of the
    fine 128 / 32.  Not popular: only the narrow bands of fine segments hit in L2; wide rows keep 128 / 32, and from
    four rows per wavefront, where half of the rows are that long, the cut comes down to 256 / 64 so that the rows are
    swept at all."""
    def cut_of(ip, ix, **kw):
        st = Layout.from_csr(ip, ix, **kw).stats()
        return st["hub_split"], st["segment"]
    ip, ix = rmat_csr(1 << 16, 100, seed=81)                 # dense and skewed: 80 % of the edges in rows > 128
    deg = np.diff(ip)
    assert deg[deg > 128].sum() * 3 >= len(ix) * 2 and (deg > 128).sum() * 2 < len(deg)
    assert cut_of(ip, ix, lanes_per_row=32) == (512, 128) and cut_of(ip, ix, lanes_per_row=20) == (512, 128)
    assert cut_of(ip, ix, lanes_per_row=64, row_bytes=640) == (512, 128)
    assert cut_of(ip, ix, lanes_per_row=64, row_bytes=1024) == (256, 64)
    ip, ix = make_workload("c2", 2)                          # average degree 14: half of the edges beyond 128
    assert cut_of(ip, ix, lanes_per_row=32) == (128, 32) and cut_of(ip, ix, lanes_per_row=64, row_bytes=1024) == (128, 32)
    u = np.repeat(np.arange(1 << 15), 150)                   # uniform degrees around 300: every row beyond 128
    ip, ix = csr_from_pairs(u, np.random.default_rng(3).integers(0, 1 << 15, len(u)), 1 << 15, False)
    assert np.diff(ip).min() > 200
    assert cut_of(ip, ix, lanes_per_row=32) == (128, 32)     # no popular sources: fine segments
    assert cut_of(ip, ix, lanes_per_row=8) == (256, 128)     # 4 MB: an L2 holds the matrix, the small-launch cut stays
    # 2^17 rows x 128 bytes = 16 MB, every row about 300 entries and none popular: cut below them
    u = np.repeat(np.arange(1 << 17), 150)
    ip, ix = csr_from_pairs(u, np.random.default_rng(4).integers(0, 1 << 17, len(u)), 1 << 17, False)
    deg = np.diff(ip)
    assert (deg > 256).sum() > 0.99 * len(deg) and deg.max() < 640
    assert cut_of(ip, ix, lanes_per_row=8) == (256, 64)      # the table alone says 640 / 160: no row would be cut
    assert cut_of(ip, ix, lanes_per_row=8, disable_reuse=True, hub_split=640)[0] == 640   # a caller's cut stands


def test_small_launches_cut_long_rows_lower():
    """A launch that cannot fill the machine twice (fewer than 16 384 wavefronts of rows) is bound by its longest
    chain of dependent gathers: 256 / 128 from five rows per wavefront, 128 / 64 at four, 128 / 32 for wide bf16
    rows.  Beyond that size the cut still steps down (1024 -> 640 -> 384 -> 256) while a chain of `cut` entries
    would outlast 3/4 of the launch, priced at (10 + 0.14 x row bytes) ns an entry against 15 us + 60 us per GB
    gathered.  bf16 rows of 256 columns take segments of 128 entries instead of 48 when the caches hold the matrix."""
    def cut_of(ip, ix, **kw):
        st = Layout.from_csr(ip, ix, **kw).stats()
        return st["hub_split"], st["segment"]
    ip, ix = make_workload("c1", 0)                          # 2^14 rows
    assert cut_of(ip, ix, lanes_per_row=8) == (256, 128)
    assert cut_of(ip, ix, lanes_per_row=12) == (256, 128)
    assert cut_of(ip, ix, lanes_per_row=16) == (128, 64)
    assert cut_of(ip, ix, lanes_per_row=32) == (128, 32)     # up to three rows per wavefront: the fine cut anyway
    assert cut_of(ip, ix, lanes_per_row=32, elem_bytes=2) == (128, 32)
    assert cut_of(ip, ix, lanes_per_row=16, elem_bytes=2) == (256, 128)     # 1280 / 320 stepped down
    ip, ix = rmat_csr(1 << 17, 8, seed=24)                   # 1.0 M edges
    e = len(ix)
    for lanes, rule in ((16, 1024), (12, 640), (8, 640)):
        limit = 3 * (15000 + e * lanes * 16 * 60 // 1000000) // (4 * (10 + lanes * 16 * 14 // 100))
        want = next(c for c in ((rule, 0), (640, 160), (384, 96), (256, 128)) if c[0] <= max(limit, 256) and c[0] <= rule)
        got = cut_of(ip, ix, lanes_per_row=lanes)
        assert got[0] == want[0] and got[0] < rule and (want[1] == 0 or got[1] == want[1]), (lanes, got, limit)
    assert cut_of(ip, ix, lanes_per_row=32, elem_bytes=2) == (256, 128)     # 64 MB of bf16 rows: cached
    ip, ix = make_workload("c4", 2)                          # 600 000 rows, 15 M edges: no chain outlasts the launch
    assert cut_of(ip, ix, lanes_per_row=16) == (1024, 128) and cut_of(ip, ix, lanes_per_row=12) == (640, 160)
    assert cut_of(ip, ix, lanes_per_row=32, elem_bytes=2) == (256, 48)      # 307 MB of bf16 rows


def test_small_graphs_keep_long_rows_whole_for_a_workgroup_each():
    """A small launch (the library's own cut) with at most 256 rows of more than 256 entries, the longest of
    at most 16 x 96 entries per lane group, keeps those rows whole: they lead the task list (longest first) and the
    launch gives each 16, 8 or 4 wavefronts of one workgroup.  No segment, no partial row, no second launch; the cut the
    rule would have used is still reported."""
    ip, ix = make_workload("c1", 0)                          # 2^14 rows, 106 of them beyond 256 entries, the longest 2486
    deg = np.diff(ip)
    lay = Layout.from_csr(ip, ix, lanes_per_row=8)
    st, ex = lay.stats(), lay.export()
    assert st["workgroup_rows"] == int((deg > 256).sum()) == 106 and st["hub_segments"] == 0 and st["partial_rows"] == 0
    assert (st["hub_split"], st["segment"]) == (256, 128) and st["longest_row_task"] == deg.max()
    lens = np.diff(ex["b_task_ptr"])
    assert (lens[:106] > 256).all() and (lens[106:] <= 256).all() and (np.diff(lens[:106].astype(np.int64)) <= 0).all()
    assert sorted(ex["b_task_out"][:106].tolist()) == sorted(np.nonzero(deg > 256)[0].tolist())
    # every entry of every row is still there
    assert len(ex["b_col"]) == len(ix) and st["gathered_rows"] == len(ix)
    assert Layout.from_csr(ip, ix, lanes_per_row=8, elem_bytes=2).stats()["workgroup_rows"] == 106     # bf16 rows alike
    # a caller's cut or a scope that needs segments: the segments stay
    for kw in (dict(hub_split=256), dict(segment=64), dict(share_scope="long_rows")):
        st = Layout.from_csr(ip, ix, lanes_per_row=8, **kw).stats()
        assert st["workgroup_rows"] == 0 and st["hub_segments"] > 0, kw
    # one row per wavefront: 2^14 rows are no small launch, and 2486 entries would be 155 per lane group
    assert Layout.from_csr(ip, ix, lanes_per_row=64).stats()["workgroup_rows"] == 0
    # too many long rows for a workgroup each (697 beyond 256 entries): segments
    ip, ix = rmat_csr(1 << 16, 24, seed=91, a=0.5, b=0.2, c=0.2)
    st = Layout.from_csr(ip, ix, lanes_per_row=8).stats()
    assert int((np.diff(ip) > 256).sum()) > 256 and st["workgroup_rows"] == 0 and st["hub_segments"] > 0
    # a row too long for one workgroup: 2^13 nodes, one of which every node is a neighbour of
    n = 1 << 13
    u = np.concatenate([np.arange(n), np.zeros(n, np.int64), np.arange(n)])
    v = np.concatenate([(np.arange(n) + 1) % n, np.arange(n), np.zeros(n, np.int64)])
    ip, ix = csr_from_pairs(u, v, n, False)
    st = Layout.from_csr(ip, ix, lanes_per_row=32).stats()   # two rows per wavefront: at most 3072 entries
    assert st["workgroup_rows"] == 0 and st["hub_segments"] > 0
    assert Layout.from_csr(ip, ix, lanes_per_row=8).stats()["workgroup_rows"] == 1      # 12 288 at eight


def test_xcd_run_follows_the_locality_of_the_graph():
    """Block-structured graphs (rows gather from their own neighbourhood) keep a whole tile of destinations on
    one XCD; graphs without that locality use short runs."""
    ip, ix = make_workload("c3", 4)                          # SBM: 24 of 26 neighbours inside the row's own block
    assert Layout.from_csr(ip, ix).export()["xcd_run"] == 256               # 4096-row tile / (4 wavefronts x 4 rows)
    assert Layout.from_csr(ip, ix, lanes_per_row=64).export()["xcd_run"] == 1024
    ip, ix = make_workload("c4", 3)                          # R-MAT, 300 000 nodes: 9 % of the neighbours are nearby
    assert Layout.from_csr(ip, ix).export()["xcd_run"] == 4


def test_long_tasks_come_first_and_short_tasks_are_sorted_inside_tiles():
    ip, ix = make_workload("c1", 1)
    n = len(ip) - 1
    lay = Layout.from_csr(ip, ix)
    ex, st = lay.export(), lay.stats()
    lens = np.diff(ex["b_task_ptr"])
    nw = st["wave_tasks_b"]
    assert (lens[:nw] > 32).all() and (lens[nw:] <= 32).all() and (np.diff(lens[:nw]) <= 0).all()   # small launch: cut 32
    assert sorted(ex["b_task_out"].tolist()) == list(range(n))
    assert lens.max() <= 2048                                # longer rows were segmented
    ip, ix = make_workload("c4", 2)                          # 600 000 rows fill the machine: cut 64
    lay = Layout.from_csr(ip, ix, lanes_per_row=12)
    ex, st = lay.export(), lay.stats()
    lens, nw = np.diff(ex["b_task_ptr"]), st["wave_tasks_b"]
    assert (lens[:nw] > 64).all() and (lens[nw:] <= 64).all() and lens[nw:].max() > 32


def test_non_canonical_v2_input_is_still_executed_correctly(oracle):
    ip, ix = rmat_csr(200, 8, seed=5)
    n = len(ip) - 1
    plan = R.build_plan(ip, ix, 3)
    up, dp = plan["uniqpart_pointers"].astype(np.int64), plan["part2Node_ptr"].astype(np.int64)
    uc, dc = plan["uniqpart_column_index"], plan["part2Node_col"]
    perm = np.random.default_rng(1).permutation(len(up) - 1)                 # shuffle the unique parts
    uc2 = np.concatenate([uc[up[w]:up[w + 1]] for w in perm])
    dc2 = np.concatenate([dc[dp[w]:dp[w + 1]] for w in perm])
    up2 = np.concatenate([[0], np.cumsum(np.diff(up)[perm])])
    dp2 = np.concatenate([[0], np.cumsum(np.diff(dp)[perm])])
    lay = Layout.from_v2(uc2, up2, dp2, dc2, n, 3)
    ex, st = lay.export(), lay.stats()
    assert not ex["canonical"]
    x = np.random.default_rng(2).standard_normal((n, 2))
    got = emulate_schedule(ex, n, x, lambda c: 1.0, lambda v: 1.0, st["partial_rows"])
    assert np.allclose(got, oracle.closed_form(ip, ix, x, normalized=False), rtol=1e-12, atol=1e-12)


def test_invalid_plan_tensors_are_rejected_on_the_host():
    ip, ix = toy_csr()
    plan = R.build_plan(ip, ix, 3)
    bad = plan["uniqpart_column_index"].copy()
    bad[0] = 10                                               # node id == N
    with pytest.raises(RofError, match="out of range"):
        Layout.from_v2(bad, plan["uniqpart_pointers"], plan["part2Node_ptr"], plan["part2Node_col"], 10, 3)
    with pytest.raises(RofError, match="out of range"):
        Layout.from_v2(plan["uniqpart_column_index"], plan["uniqpart_pointers"][::-1].copy(), plan["part2Node_ptr"],
                       plan["part2Node_col"], 10, 3)
    with pytest.raises(ValueError):
        Layout.from_v2(plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"][:-1],
                       plan["part2Node_col"], 10, 3)
    flag = plan["part_cache_flagindex"].copy()
    flag[0] = 7                                               # only 2 cache rows exist
    with pytest.raises(RofError, match="out of range"):
        Layout.from_v1(plan["new_indices_src"], plan["part_ptr"], plan["part2Node"], flag,
                       plan["part_pointers_cache"], plan["column_index_cache"], 10, 3)


def test_algorithmic_bytes_formula():
    ip, ix = toy_csr()
    plan = R.build_plan(ip, ix, 3)
    lay = _v2(plan, 10, 3, min_consumers=2)
    f = 8
    # 16 gathered rows, 6 partial reads, 2 partial rows, 10 nodes
    assert lay.algorithmic_bytes(f) == 16 * (4 + 4 * f) + 6 * (4 + 4 * f) + 2 * 4 * f + 10 * (4 * f + 8) + 4 * 3
    a, b = lay.launch_bytes(f)
    assert a + b == lay.algorithmic_bytes(f) and a == 6 * (4 + 4 * f) + 2 * 4 * f + 4 * 3
    plain = _v2(plan, 10, 3, disable_reuse=True)
    assert plain.algorithmic_bytes(f) == 28 * (4 + 4 * f) + 10 * (4 * f + 8) + 4


def test_recorded_layout_choices_are_replayed_without_a_gpu():
    """`LayoutFamily(choices=...)` rebuilds the width classes it has a record for with the recorded cut, segment and
    launch settings (plain data, as `choices()` returns it and `ROF_inputInfo.save` stores it); other classes follow
    the rules."""
    from artifact_amd.layout import LayoutFamily
    ip, ix = make_workload("c4", 4)
    rec = {"12,4,0": {"cut": 512, "segment": 64, "tuning": {"xcd_run_partial": 0, "xcd_run_dst": 16, "wave_cap": 6,
                                                            "lds_pad": 0, "deep": 1}}}
    fam = LayoutFamily(lambda lpr, eb, rb=0, **kw: Layout.from_csr(ip, ix, lanes_per_row=lpr, elem_bytes=eb, row_bytes=rb, **kw),
                       autotune=False, choices=rec)
    lay = fam.get(47)
    st = lay.stats()
    assert (st["hub_split"], st["segment"]) == (512, 64) and lay.tuning() == rec["12,4,0"]["tuning"]
    assert fam.choices() == rec and fam.chosen[(12, 4, 0)]["replayed"]
    other = fam.get(32)                                       # no record for 8 lanes: the rule's cut, default settings
    assert (other.stats()["hub_split"], other.stats()["segment"]) == (640, 160) and other.tuning()["wave_cap"] == -1
    assert fam.choices() == rec
    fam.close()
