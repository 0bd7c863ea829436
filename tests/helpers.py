"""Shared helpers of the test-suite (inputs, golden fixtures, a numpy emulation of the schedule)."""
import hashlib
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")

V1_KEYS = ("new_indices_src", "part_pointers_cache", "column_index_cache", "part_cache_flagindex")
V2_KEYS = ("uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col")
STEP_KEYS = ("part_ptr", "part2Node", "num_parts_per_node_acc", "intersect_count", "index_ordered", "index_picked")

TOY_ADJ = {0: [3, 4, 5], 1: [3, 4, 5], 2: [3, 4, 5, 6], 3: [0, 1, 2, 7], 4: [0, 1, 2, 8], 5: [0, 1, 2, 9], 6: [2, 7],
           7: [3, 6], 8: [4], 9: [5]}


# What the fp32 parity checks saw in this session: how many elements were compared, how many of them met the bar
# only through its summation term, and by how much those exceeded the strict bar (see close_fp32).
FP32_BAR_STATS = {"compared": 0, "beyond_strict": 0, "max_excess_ratio": 0.0, "max_excess_abs": 0.0}


def close_fp32(got, want64, mag=None, rtol=1e-5, atol=1e-6, extra=None, what=""):
    """Assert |got - want| <= atol + rtol*|want| + rtol*mag.  The first two terms are the stated bar for fp32 sums
    (rel 1e-5 / abs 1e-6); `mag` = the sum of the absolute values of the summands, which makes the last term the
    standard bound on fp32 re-association error (upstream's own result depends on the order its atomics land in,
    reuse_conv_kernel.cu:16-21, so it is only defined up to that).  Elements that pass only thanks to the last
    term are counted in FP32_BAR_STATS and reported at the end of the test session."""
    got = np.asarray(got, dtype=np.float64)
    want64 = np.asarray(want64, dtype=np.float64)
    err = np.abs(got - want64)
    strict = atol + rtol * np.abs(want64)
    tol = strict.copy()
    if mag is not None:
        tol = tol + rtol * np.asarray(mag, dtype=np.float64)
    if extra is not None:
        strict, tol = strict + extra, tol + extra
    beyond = err > strict
    FP32_BAR_STATS["compared"] += int(err.size)
    if beyond.any():
        FP32_BAR_STATS["beyond_strict"] += int(beyond.sum())
        FP32_BAR_STATS["max_excess_ratio"] = max(FP32_BAR_STATS["max_excess_ratio"], float((err[beyond] / strict[beyond]).max()))
        FP32_BAR_STATS["max_excess_abs"] = max(FP32_BAR_STATS["max_excess_abs"], float((err[beyond] - strict[beyond]).max()))
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off, max err {err.max():.3e}"


def toy_csr():
    indptr = np.zeros(11, dtype=np.int32)
    idx = []
    for v in range(10):
        idx += TOY_ADJ[v]
        indptr[v + 1] = len(idx)
    return indptr, np.array(idx, dtype=np.int32)


def golden_small():
    """{case: {"in": {...}, "out": {...}}} from tests/golden/plans_small.npz (written by the upstream builder)."""
    z = np.load(os.path.join(GOLDEN, "plans_small.npz"))
    cases = {}
    for key in z.files:
        name, kind, arr = key.split("/")
        cases.setdefault(name, {"in": {}, "out": {}})[kind][arr] = z[key]
    return cases


def golden_digests():
    with open(os.path.join(GOLDEN, "plans_digest.json")) as f:
        return json.load(f)


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(np.asarray(a, dtype=np.uint32)).tobytes()).hexdigest()


def case_inputs(c):
    i = c["in"]
    ps, discard = int(i["ps_discard"][0]), bool(i["ps_discard"][1])
    return i["indptr_dst"], i["indices_src"], i.get("indptr_src"), i.get("indices_dst"), ps, discard


def emulate_schedule(ex, n, x, w_of, s_of, n_slots):
    """Run the exported schedule (groups, segments, rows) in float64 numpy, checking its structure: references only
    to partial rows that an earlier launch wrote, one writer per output row, LDS rows only inside the cluster
    (workgroup) that sums them."""
    feat = x.shape[1]
    part = np.zeros((n_slots, feat))
    written = np.zeros(n_slots, dtype=bool)
    out = np.zeros((n, feat))
    for ph in ("g", "s", "b"):
        tp, nr, to, col = ex[ph + "_task_ptr"], ex[ph + "_task_nref"], ex[ph + "_task_out"], ex[ph + "_col"]
        nlds = ex.get("b_task_nlds") if ph == "b" else None
        if nlds is None or len(nlds) == 0:
            nlds = np.zeros(len(to), dtype=np.int64)
        block_of, lds = None, {}
        if ph == "b" and ex.get("b_shape", {}).get("lg_blocks", 0) > 0:
            sh = ex["b_shape"]
            tf = ex["b_lg_task_first"]
            assert len(tf) == sh["lg_blocks"] + 1 and tf[0] == sh["n_regular"] >= sh["n_wave"] and (np.diff(tf) >= 2).all()
            assert tf[-1] == len(to)

            def block_of(t):   # cluster that owns task t, or None
                b = int(np.searchsorted(tf, t, side="right")) - 1
                return b if 0 <= b < sh["lg_blocks"] else None
            lp, ltp, lcol = ex["b_lg_ptr"], ex["b_lg_task_ptr"], ex["b_lg_col"]
            assert len(lp) == sh["lg_blocks"] + 1 and lp[0] == 0 and lp[-1] == len(ltp) - 1
            for b in range(sh["lg_blocks"]):
                rows = []
                assert 0 < lp[b + 1] - lp[b] <= sh["lg_max_rows"]
                for j in range(lp[b], lp[b + 1]):
                    acc = np.zeros(feat)
                    for i in range(ltp[j], ltp[j + 1]):
                        assert 0 <= lcol[i] < n
                        acc += w_of(lcol[i]) * x[lcol[i]]
                    rows.append(acc)
                lds[b] = rows
        seen = set()
        for t in range(len(to)):
            acc = np.zeros(feat)
            for i in range(tp[t], tp[t + 1]):
                c = col[i]
                if i < tp[t] + nlds[t]:
                    rows = lds.get(block_of(t))
                    assert rows is not None and 0 <= c < len(rows), "LDS row outside the workgroup that sums it"
                    acc += rows[c]
                elif i < tp[t] + nlds[t] + nr[t]:
                    assert c >= n and written[c - n], "reference to a partial row that is not ready"
                    acc += part[c - n]
                else:
                    assert 0 <= c < n
                    acc += w_of(c) * x[c]
            assert to[t] not in seen, "two writers for one output row"
            seen.add(int(to[t]))
            if ph == "b":
                out[to[t]] = acc * (s_of(to[t]) if tp[t + 1] > tp[t] else 1.0)
            else:
                part[to[t]] = acc
        if ph != "b":
            for t in to:
                written[t] = True
        else:
            assert seen == set(range(n)), "every destination row must be written exactly once"
    return out


def check_plan_invariants(ipd, isrc, ps, plan, discard=True):
    """Structural facts every valid plan satisfies (independent of tie-breaking)."""
    ipd = np.asarray(ipd).astype(np.int64)
    isrc = np.asarray(isrc).astype(np.int64)
    n, e = len(ipd) - 1, len(isrc)
    pp, p2n = plan["part_ptr"].astype(np.int64), plan["part2Node"].astype(np.int64)
    # P1: chunks tile every row in order, at most ps long, never crossing a row
    assert pp[0] == 0 and pp[-1] == e and (np.diff(pp) >= 1).all() and (np.diff(pp) <= ps).all()
    assert (np.diff(p2n) >= 0).all()
    assert (ipd[p2n] <= pp[:-1]).all() and (pp[1:] <= ipd[p2n + 1]).all()
    acc = plan["num_parts_per_node_acc"].astype(np.int64)
    assert np.array_equal(acc, np.cumsum((np.diff(ipd) + ps - 1) // ps))
    cnt = plan["intersect_count"].astype(np.int64)
    picked = plan["index_picked"].astype(np.int64)
    # P3: picked chunks are full, disjoint in sources, cnt >= 2 and non-increasing in pick order
    used = set()
    for p in picked:
        srcs = isrc[pp[p]:pp[p + 1]]
        if discard:
            assert len(srcs) == ps
        assert cnt[p] >= 2
        assert used.isdisjoint(srcs.tolist())
        used.update(srcs.tolist())
    assert (np.diff(cnt[picked]) <= 0).all()
    order = plan["index_ordered"].astype(np.int64)
    assert np.array_equal(np.sort(order), np.arange(len(cnt))) and (np.diff(cnt[order]) <= 0).all()
    if "uniqpart_pointers" not in plan:
        return
    # P5: expanding the v2 plan reproduces the edge multiset
    uc, up = plan["uniqpart_column_index"].astype(np.int64), plan["uniqpart_pointers"].astype(np.int64)
    dp, dc = plan["part2Node_ptr"].astype(np.int64), plan["part2Node_col"].astype(np.int64)
    assert len(up) == len(dp)
    src_l, dst_l = [], []
    for w in range(len(up) - 1):
        s = uc[up[w]:up[w + 1]]
        d = dc[dp[w]:dp[w + 1]]
        src_l.append(np.repeat(s, len(d)))
        dst_l.append(np.tile(d, len(s)))
    got = np.sort(np.concatenate(dst_l) * n + np.concatenate(src_l)) if src_l else np.empty(0, dtype=np.int64)
    want = np.sort(np.repeat(np.arange(n), np.diff(ipd)) * n + isrc)
    assert np.array_equal(got, want)
    # P6: saved gathers
    assert e - len(uc) == int(((cnt[picked] - 1) * np.diff(pp)[picked]).sum())
    # P4: v1 rows are permutations; flagged chunks equal their cache rows
    new = plan["new_indices_src"].astype(np.int64)
    for v in range(n):
        assert np.array_equal(np.sort(new[ipd[v]:ipd[v + 1]]), np.sort(isrc[ipd[v]:ipd[v + 1]]))
    flag = plan["part_cache_flagindex"].astype(np.int64)
    cp, cc = plan["part_pointers_cache"].astype(np.int64), plan["column_index_cache"].astype(np.int64)
    for p in np.nonzero(flag)[0]:
        k = flag[p] - 1
        assert np.array_equal(new[pp[p]:pp[p + 1]], cc[cp[k]:cp[k + 1]])
