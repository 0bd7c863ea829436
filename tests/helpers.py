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


def strict_excess(got, want64, rtol=1e-5, atol=1e-6):
    """(elements beyond the strict bar atol + rtol*|want|, largest error as a multiple of that bar)."""
    err = np.abs(np.asarray(got, dtype=np.float64) - np.asarray(want64, dtype=np.float64))
    strict = atol + rtol * np.abs(np.asarray(want64, dtype=np.float64))
    return int((err > strict).sum()), float((err / strict).max()) if err.size else 0.0


def summation_error(got, want64, mag):
    """Largest error in units of the sum of the absolute values of the terms (the quantity that bounds the
    re-association error of an fp32 sum: about sqrt(terms) * 2^-24 for a sequential sum of random terms)."""
    err = np.abs(np.asarray(got, dtype=np.float64) - np.asarray(want64, dtype=np.float64))
    mag = np.asarray(mag, dtype=np.float64)
    ok = mag > 0
    return float((err[ok] / mag[ok]).max()) if ok.any() else 0.0


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


# ---- the randomised schedule cases of tests/test_gpu_random_schedules.py (the GPU test runs them; the CPU suite
# measures on the same inputs how far fp32 arithmetic in upstream's own order is from float64)
LANES = [0, 4, 8, 10, 12, 16, 20, 32, 64]


def random_csr(rng, n, ps):
    """Rows of 0..40 neighbours, a few hubs of up to n, and rows made of one to three of a few shared
    neighbour sets of `ps` ids each (each set inside its own id range, so the sets stay whole when a row is cut
    into parts and the plan builder finds parts to share); columns sorted and unique per row."""
    kind = rng.random(n)
    deg = np.where(kind < 0.15, 0, rng.integers(1, 41, n))
    hubs = rng.choice(n, max(1, n // 200), replace=False)
    deg[hubs] = rng.integers(n // 4, n + 1, len(hubs))
    kind[hubs] = 0.5
    sets = max(1, min(n // (2 * ps), n // 50 + 1))
    width = n // sets
    shared = [j * width + np.sort(rng.choice(width, ps, replace=False)) for j in range(sets)]
    rows = []
    for v in range(n):
        if kind[v] > 0.6:
            rows.append(np.concatenate([shared[j] for j in np.sort(rng.choice(sets, min(sets, int(rng.integers(1, 4))),
                                                                              replace=False))]))
            continue
        rows.append(np.unique(rng.choice(n, min(int(deg[v]), n), replace=False)))
    ip = np.r_[0, np.cumsum([len(r) for r in rows])].astype(np.int32)
    ix = (np.concatenate(rows) if ip[-1] else np.zeros(0)).astype(np.int32)
    return ip, ix


def bf16_round(a):
    """float32 -> nearest-even bfloat16 -> float32 (the rounding torch's .to(bfloat16) performs on finite values)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    return ((u + 0x7fff + ((u >> 16) & 1)) & np.uint32(0xffff0000)).astype(np.uint32).view(np.float32)




def random_schedule_case(seed):
    """Inputs and options of one randomised case (graph, schedule options, width, stride, types, epilogue)."""
    rng = np.random.default_rng(seed)
    n = int(rng.integers(12, 3000))
    ps = int(rng.integers(2, 6))
    ip, ix = random_csr(rng, n, ps)
    opts = dict(hub_split=int(rng.choice([0, 8, 33, 100])), segment=int(rng.choice([0, 1, 5, 16])),
                lanes_per_row=int(rng.choice(LANES)), entry_order=str(rng.choice(["descending", "plan", "ascending"])),
                tile_rows=int(rng.choice([0, 64])), elem_bytes=int(rng.choice([0, 2, 4])),
                local_groups=int(rng.choice([0, 0, 1, 30, -1])))
    if seed % 3 == 2:        # (chosen from the seed, not drawn: the cases keep the inputs they always had)
        opts["share_scope"] = "long_rows"
    use_plan = rng.random() < 0.6
    min_consumers = int(rng.choice([0, 2, 3])) if use_plan else 0
    feat = int(rng.choice([1, 2, 3, 5, 8, 17, 32, 47, 64, 100, 129, 256, 300]))
    ld = feat + int(rng.choice([0, 0, 1, 3, 8]))
    bf16_in, bf16_out = rng.random() < 0.35, rng.random() < 0.3
    normalized = rng.random() < 0.6
    bias = rng.standard_normal(feat).astype(np.float32) if rng.random() < 0.5 else None
    relu = rng.random() < 0.5
    self_weight = float(rng.choice([0.0, 0.0, 0.7, -1.25]))
    pad = bool(rng.random() < 0.4)                         # rows taken as whole vectors where the stride allows it
    x = rng.standard_normal((n, feat)).astype(np.float32)
    if bf16_in:
        x = bf16_round(x)
    deg = rng.integers(1, 50, n).astype(np.float32)        # the degrees are an input of their own (cu:254)
    return dict(n=n, ps=ps, ip=ip, ix=ix, opts=opts, use_plan=use_plan, min_consumers=min_consumers, feat=feat, ld=ld,
                bf16_in=bf16_in, bf16_out=bf16_out, normalized=normalized, bias=bias, relu=relu,
                self_weight=self_weight, pad=pad, x=x, deg=deg)


def closed_form_case(oracle, c):
    """float64 closed form of one randomised case and the sum of the absolute values of its terms:
    out[v] = relu( rs(deg v) * sum_u rs(deg u) x[u]  +  self_weight * x[v]  +  bias )."""
    n, ip, ix, feat = c["n"], c["ip"], c["ix"], c["feat"]
    rs = oracle.rsqrt_rn(c["deg"]).astype(np.float64) if c["normalized"] else np.ones(n)
    x64 = c["x"].astype(np.float64)
    rows = np.repeat(np.arange(n), np.diff(ip))
    want, mag = np.zeros((n, feat)), np.zeros((n, feat))
    np.add.at(want, rows, x64[ix] * rs[ix, None])
    np.add.at(mag, rows, np.abs(x64[ix]) * rs[ix, None])
    want, mag = want * rs[:, None], mag * rs[:, None]
    want, mag = want + c["self_weight"] * x64, mag + abs(c["self_weight"]) * np.abs(x64)
    if c["bias"] is not None:
        want, mag = want + c["bias"], mag + np.abs(c["bias"])
    if c["relu"]:
        want = np.maximum(want, 0.0)
    return want, mag


def reference_order_fp32(oracle, c):
    """The layer of one randomised case in fp32, summed the way the upstream GNNA kernel sums it: every row in
    parts of `ps` neighbours in CSR order (oracle/agg_oracle.c, reuse_conv_kernel.cu:205-286), then the epilogue in
    the order the library applies it (own row, bias, ReLU), each step rounded to fp32."""
    n, ps, ip, ix = c["n"], c["ps"], c["ip"], c["ix"]
    part_ptr, part2node = [0], []
    for v in range(n):
        for q in range(ip[v], ip[v + 1], ps):
            part_ptr.append(min(q + ps, ip[v + 1]))
            part2node.append(v)
    agg = oracle.agg_parts(c["x"], c["deg"], ix, np.asarray(part_ptr, dtype=np.int32),
                           np.asarray(part2node, dtype=np.int32), normalized=c["normalized"])
    r = agg.astype(np.float64)
    if c["self_weight"] != 0.0:
        r = (np.float32(c["self_weight"]).astype(np.float64) * c["x"].astype(np.float64) + r).astype(np.float32).astype(np.float64)
    if c["bias"] is not None:
        r = (r + c["bias"].astype(np.float64)).astype(np.float32).astype(np.float64)
    if c["relu"]:
        r = np.maximum(r, 0.0)
    return r
