#!/usr/bin/env python3
"""Benchmark of the reuse-aware aggregation layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4] [--part-size 3]

A step is one aggregation layer: out = D^-1/2 A D^-1/2 (XW) evaluated through the reuse plan on a
feature matrix that is already resident in HBM (the dense update X*W is not part of the step), with
the operands laid out as the operator API lays them out: the update's rows in a stride that is a
multiple of four floats, the output a packed [N, F] tensor.  The default workload is the 2.4M-node
R-MAT graph with aggregated width 47.  Prints one JSON line: GEdges/s (original edge count / time);
the HBM roofline of the destination-row launch -- its duration measured with HIP events on the launch
stream, its HBM-side bytes measured by running this same script under `rocprofv3 --pmc` in child
processes (FETCH_SIZE, WRITE_SIZE, TCC hits/misses; scaled by a copy of known size) before this
process touches the GPU; the same kernels with reuse disabled; part sizes 2..5; and a CPU baseline
(the oracle's destination-parallel SpMM) timed on this machine's host cores.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import shutil
import subprocess
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM-side bytes per launch (partial-sum launch, destination-row launch) and TCC hit rates from the committed
# rocprofv3 summaries under profiles/ (FETCH_SIZE x its copy-calibrated factor + WRITE_SIZE).  Used only when the
# live counter runs are switched off or fail, and only for the configurations they were measured on:
# (workload, part size, width, packed output) with default layout options; the JSON then says "offline profile".
def _offline(read0, written0, hit0, read1, written1, hit1):
    launch = {1: {"read_bytes": read1, "written_bytes": written1, "bytes": read1 + written1, "tcc_hit_rate": hit1,
                  "tcc_miss_x_128B": None}}
    if read0 is not None:
        launch[0] = {"read_bytes": read0, "written_bytes": written0, "bytes": read0 + written0, "tcc_hit_rate": hit0,
                     "tcc_miss_x_128B": None}
    return {"fetch_scale": 2.0, "write_scale": 1.0, "launch": launch}


PROFILED_TRAFFIC = {
    ("c4", 3, 47, True): _offline(1.77e9, 0.029e9, 0.69, 5.87e9, 0.50e9, 0.44),     # profiles/rof_rows_kernel_c4_f47.md
    ("c5", 3, 256, True): _offline(21.47e9, 2.12e9, 0.57, 19.93e9, 4.50e9, 0.40),   # profiles/rof_rows_kernel_c5_bf16.md
    ("c3", 3, 64, True): _offline(None, None, None, 1.04e9, 0.27e9, 0.82),          # profiles/rof_rows_kernel_c3_f64.md
    ("hr", 3, 64, True): _offline(None, None, None, 1.36e9, 0.27e9, 0.20),          # profiles/rof_cluster_kernel_hr_f64.md
}
COPY_BYTES = 1 << 30   # size of the calibration copy the counter runs include
CHILD_AGGREGATIONS = 4  # aggregations a counter run executes

DESCR = {
    "c1": "c1: R-MAT 2^14 nodes, avg deg 16, self loops, GCN sym-norm, F=32, fp32",
    "c2": "c2: R-MAT 2^18 nodes, avg deg 14, self loops, GCN sym-norm, F=256, fp32",
    "c3": "c3: SBM 2^20 nodes (256 blocks), deg 24+2, GIN sum aggregation, F=64, fp32",
    "c4": "c4: R-MAT 2.4M nodes, 62.4M directed edges, GCN sym-norm, aggregated width 47, fp32",
    "c5": "c5: R-MAT 2^22 nodes, avg deg 32, self loops, GCN sym-norm, F=256, bf16 in / fp32 accumulate",
    "hr": "hr: planted-reuse graph 2^20 nodes (12 shared anchors + ~4 random neighbours per node), GCN, F=64, fp32",
}
FEAT = {"c1": 32, "c2": 256, "c3": 64, "c4": 47, "c5": 256, "hr": 64}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def load_or_build(name, part_size, cache_dir):
    """Graph + plan, cached on local disk so repeated runs on one machine skip the CPU preprocessing."""
    from artifact_amd import reuse_search_ext as R
    from artifact_amd.graphgen import make_workload

    path = os.path.join(cache_dir, f"rof_{name}_ps{part_size}.npz") if cache_dir else None
    gpath = os.path.join(cache_dir, f"rof_{name}_graph.npz") if cache_dir else None
    if path and os.path.exists(path):
        z = np.load(path)
        log(f"[bench] loaded cached graph+plan {path}")
        return {k: z[k] for k in z.files}, 0.0, 0.0
    t0 = time.time()
    if gpath and os.path.exists(gpath):
        z = np.load(gpath)
        indptr, indices = z["indptr"], z["indices"]
    else:
        indptr, indices = make_workload(name)
        if gpath:
            try:
                os.makedirs(cache_dir, exist_ok=True)
                np.savez(gpath, indptr=indptr, indices=indices)
            except OSError:
                pass
    t_gen = time.time() - t0
    log(f"[bench] graph {name}: N={len(indptr) - 1} E={len(indices)} in {t_gen:.1f}s")
    t0 = time.time()
    plan = R.build_plan(indptr, indices, part_size)
    t_plan = time.time() - t0
    log(f"[bench] reuse plan (CPU, {os.cpu_count()} cores visible): {t_plan:.1f}s, picked {len(plan['index_picked'])}")
    d = {"indptr": indptr, "indices": indices}
    for k in ("uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col", "intersect_count",
              "index_picked"):
        d[k] = plan[k]
    if path:
        try:
            os.makedirs(cache_dir, exist_ok=True)
            np.savez(path, **d)
        except OSError:
            pass
    return d, t_gen, t_plan


def cpu_baseline(indptr, indices, x32, normalized, budget_s=20.0):
    """Oracle port, destination-parallel over the host threads, on the same graph and features."""
    from oracle import oracle as O

    deg = np.diff(indptr).astype(np.float32)
    with np.errstate(divide="ignore"):
        rs = O.rsqrt_rn(deg)
    rs[~np.isfinite(rs)] = 0.0
    out = np.empty_like(x32)
    O.spmm_rows(x32, rs, indptr, indices, normalized, out=out)          # warm-up
    times = []
    t_all = time.time()
    while len(times) < 5 and (time.time() - t_all < budget_s or len(times) < 2):
        t0 = time.time()
        O.spmm_rows(x32, rs, indptr, indices, normalized, out=out)
        times.append(time.time() - t0)
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return float(np.median(times)), len(times), threads, out


MODEL_STEPS = {
    "c2": "2-layer GCN forward 128->256->40, ReLU between",
    "c3": "3-layer GIN forward 64->64->64->64 (sum aggregation, eps = 0), ReLU between",
    "c4": "one GCN layer 100->47, forward + backward (loss = sum of outputs)",
    "c5": "2-layer GCN training step 256->256->256: forward, cross-entropy, backward through both aggregations",
}


def model_step(name, d, n, ps, deg, dev, timed):
    """Milliseconds per model step of the named workload: `upstream_sequence_ms` runs update -> aggregate ->
    bias pass -> ReLU pass per layer in fp32 as upstream's layers do; `fused_ms` lets each layer pick the
    cheaper order and apply bias and ReLU in the aggregation store (c5: bfloat16 rows and GEMM operands)."""
    import types

    import torch
    import torch.nn.functional as F

    from artifact_amd.layout import Layout, LayoutFamily
    from artifact_amd.reuse_conv import ROF_GCNConv, ROF_GINConv

    fam = LayoutFamily(lambda lpr, eb, rb=0, **kw: Layout.from_v2(d["uniqpart_column_index"], d["uniqpart_pointers"],
                                                      d["part2Node_ptr"], d["part2Node_col"], n, ps,
                                                      lanes_per_row=lpr, elem_bytes=eb, row_bytes=rb, **kw))
    dummy = torch.zeros(1, dtype=torch.int32, device=dev)   # the plan tensors are not read when a layout is attached
    info = types.SimpleNamespace(degrees=deg, layouts={"ROF_v2": fam}, partSize=ps, warpPerBlock=4,
                                 **{k: dummy for k in ("column_index", "part_pointers", "part2Node",
                                                       "part_cache_flagindex", "part_pointers_cache",
                                                       "column_index_cache", "uniqpart_column_index",
                                                       "uniqpart_pointers", "part2Node_ptr", "part2Node_col")})
    torch.manual_seed(0)
    res = {"what": MODEL_STEPS[name]}
    if name == "c3":
        layers = [ROF_GINConv(64, 64).to(dev) for _ in range(3)]
        x = torch.randn((n, 64), device=dev)

        def gin():
            h = x
            with torch.no_grad():
                for i, layer in enumerate(layers):
                    h = layer(h, info)
                    if i != 2:
                        h = torch.relu_(h)
            return h

        res["forward_ms"] = timed(gin, 10)
        fam.close()
        return res
    dims = {"c2": [128, 256, 40], "c4": [100, 47], "c5": [256, 256, 256]}[name]
    train = name in ("c4", "c5")
    x = torch.randn((n, dims[0]), device=dev)
    if name == "c5":
        x = (torch.rand((n, dims[0]), device=dev) * 2 - 1).to(torch.bfloat16)
        labels = torch.randint(0, dims[-1], (n,), device=dev)
    nl = len(dims) - 1

    def build(**kw):
        return [ROF_GCNConv(dims[i], dims[i + 1], add_self_loops=False, kernel_type="ROF_v2",
                            **{k: (v(i) if callable(v) else v) for k, v in kw.items()}).to(dev) for i in range(nl)]

    base = build(bias=False)                       # bias and ReLU as separate passes, as upstream
    base_b = [torch.zeros(dims[i + 1], device=dev, requires_grad=train) for i in range(nl)]
    fused = build(order="auto", activation=lambda i: "relu" if i != nl - 1 else None,
                  compute_dtype="bf16" if name == "c5" else None, out_dtype=lambda i: "bf16" if i != nl - 1 else None)
    xf = x.float() if name == "c5" else x

    def loss_of(out):
        return F.cross_entropy(out, labels) if name == "c5" else out.sum()

    def run_base():
        with torch.set_grad_enabled(train):
            h = xf
            for i, layer in enumerate(base):
                h = layer(h, info) + base_b[i]
                if i != nl - 1:
                    h = torch.relu(h)
            if train:
                loss_of(h).backward()

    def run_fused():
        with torch.set_grad_enabled(train):
            h = x
            for layer in fused:
                h = layer(h, info)
            if train:
                loss_of(h).backward()

    res["upstream_sequence_ms"] = timed(run_base, 10)
    res["fused_ms"] = timed(run_fused, 10)
    res["speedup"] = res["upstream_sequence_ms"] / res["fused_ms"]
    fam.close()
    return res


def build_layouts(d, n, ps, lpr, in_bytes, args, want_forced=True):
    """(reuse, reuse-disabled, forced-sharing or None) layouts of one plan, not yet uploaded."""
    from artifact_amd.layout import Layout

    v2 = (d["uniqpart_column_index"], d["uniqpart_pointers"], d["part2Node_ptr"], d["part2Node_col"], n, ps)
    common = dict(hub_split=args.hub_split, segment=args.segment, lanes_per_row=lpr, entry_order=args.entry_order,
                  tile_rows=args.tile_rows, elem_bytes=in_bytes, share_scope=args.share_scope,
                  row_bytes=args.row_bytes)
    reuse = Layout.from_v2(*v2, min_consumers=args.min_consumers, **common)
    plain = Layout.from_v2(*v2, disable_reuse=True, **common)
    # when the cost model folds every group back (the plan saves too little), also time the plan with its
    # profitable groups forced to be shared, so the cost of the reuse machinery stays visible
    forced = None
    if want_forced and reuse.stats()["materialised_groups"] == 0 and len(d["index_picked"]) and not args.min_consumers:
        forced = Layout.from_v2(*v2, min_consumers=3, **common)
    return reuse, plain, forced


def make_features(name, n, feat, bf16, dev, packed=False):
    """Feature rows as the dense update leaves them: N(0,1) fp32 (uniform(-1,1) -> bf16 for c5) in rows
    allocated up to a multiple of 4 (8) elements.  Returns (view [n, feat], fp32 host copy, row stride)."""
    import torch

    from artifact_amd.graphgen import features

    mult = 8 if bf16 else 4
    ld = feat if packed else (feat + mult - 1) // mult * mult   # packed: rows `feat` elements apart, as a gradient arrives
    x32 = features(n, feat, seed=2000 + (int(name[1]) if name[1].isdigit() else 6), kind="uniform" if bf16 else "normal")
    xbuf = torch.zeros((n, ld), dtype=torch.bfloat16 if bf16 else torch.float32, device=dev)
    xbuf[:, :feat] = torch.from_numpy(x32).to(dev)
    x = xbuf[:, :feat]
    if bf16:
        x32 = x.to(torch.float32).cpu().numpy()
    return x, x32, ld


def apply_tuning(lay, args):
    """Launch tuning from the command line (all defaults: the library's own choices)."""
    if lay is not None and (args.xcd_run or args.xcd_run_partial or args.lds_pad > 0 or args.wave_cap >= 0):
        lay.set_tuning(xcd_run_partial=args.xcd_run_partial, xcd_run_dst=args.xcd_run, wave_cap=args.wave_cap,
                       lds_pad=max(0, args.lds_pad))


def traffic_child(args):
    """Body of a counter run (this script under `rocprofv3 --pmc ...`): the default layout of the workload, one
    calibration copy of COPY_BYTES and a few aggregations, nothing else on the GPU."""
    import ctypes

    import torch

    from artifact_amd import _lib
    from artifact_amd.layout import lanes_per_row

    L = _lib.lib()
    dev = torch.device("cuda:0")
    name, ps = args.workload, args.part_size
    feat = args.feat or FEAT[name]
    bf16, normalized = name == "c5", name != "c3"
    d, _, _ = load_or_build(name, ps, args.cache_dir)
    n = len(d["indptr"]) - 1
    args.row_bytes = feat * (2 if bf16 else 4)
    reuse, _, _ = build_layouts(d, n, ps, lanes_per_row(feat, bf16), 2 if bf16 else 4, args, want_forced=False)
    apply_tuning(reuse, args)
    reuse.upload()
    if normalized:
        reuse.set_degrees(torch.from_numpy(np.diff(d["indptr"]).astype(np.float32)).to(dev))
    x, _, ld = make_features(name, n, feat, bf16, dev, args.packed_input)
    pad = args.padded_output and ld != feat
    out = torch.empty((n, ld if pad else feat), dtype=torch.float32, device=dev)[:, :feat]
    a = torch.empty(COPY_BYTES // 4, dtype=torch.float32, device=dev).normal_()
    b = torch.empty_like(a)
    torch.cuda.synchronize()
    _lib.check(L.rof_device_copy(ctypes.c_void_p(b.data_ptr()), ctypes.c_void_p(a.data_ptr()), COPY_BYTES,
                                 ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    for _ in range(CHILD_AGGREGATIONS):
        reuse.aggregate(x, normalized, out=out, feat_dim=feat, pad_columns=pad)
    torch.cuda.synchronize()


def read_counter_csv(path):
    """One rocprofv3 counter_collection.csv of a counter run -> ({(counter, phase): value per aggregation},
    {counter: value of the calibration copy}).  Phase 0 = the partial-sum launches (shared groups, segments of long
    rows; template argument PHASE of the kernel name <XT, VEC, LPR, PHASE, OFF32> is 0, 3 with streamed partial
    rows or 5 with more gathers in flight), phase 1 = the destination rows and their clusters (PHASE 1, 2 or 4, or
    rof_coop_kernel on small graphs).  A phase may consist of two launches, so the dispatches of one phase are summed and divided
    by the number of aggregations the run executes."""
    acc, copy = collections.defaultdict(float), {}
    with open(path) as f:
        for row in csv.DictReader(f):
            k = row["Kernel_Name"]
            if "rof_copy_kernel" in k:
                copy[row["Counter_Name"]] = float(row["Counter_Value"])
            elif "rof_coop_kernel" in k:   # the destination-row launch of a small graph (long rows: a workgroup each)
                acc[(row["Counter_Name"], 1)] += float(row["Counter_Value"])
            elif "rof_rows_kernel" in k or "rof_cluster_kernel" in k:
                phase = int(k.split("<")[1].split(">")[0].split(",")[3])
                if phase not in (0, 1, 2, 3, 4, 5):
                    raise ValueError(f"unknown launch kind in kernel name {k!r}")
                acc[(row["Counter_Name"], 0 if phase in (0, 3, 5) else 1)] += float(row["Counter_Value"])
    return {k: v / CHILD_AGGREGATIONS for k, v in acc.items()}, copy


def run_group(cmd, cwd, env, limit_s):
    """Run `cmd` as the leader of a process group of its own and return (exit status, output).  On a time-out the
    whole group is killed -- the profiler and the Python process it started -- so that no GPU holder outlives us."""
    import signal

    p = subprocess.Popen(cmd, cwd=cwd, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, start_new_session=True)
    try:
        out, _ = p.communicate(timeout=limit_s)
        return p.returncode, out.decode(errors="replace")
    except subprocess.TimeoutExpired:
        try:
            os.killpg(p.pid, signal.SIGKILL)
        except ProcessLookupError:
            pass
        out, _ = p.communicate()
        return -9, out.decode(errors="replace") + f"\n[killed after {limit_s} s]"
    finally:
        try:   # whatever happened: nothing of the group is left behind
            os.killpg(p.pid, signal.SIGKILL)
        except (ProcessLookupError, PermissionError):
            pass


def measure_traffic(args, passthrough):
    """HBM-side bytes per launch from rocprofv3 counter runs of this script (one counter set per run, as the
    hardware collects them), started as child processes *before* this process initialises the GPU.
    Returns a dict, or {"error": ...} when the profiler is missing or a run fails."""
    prof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(prof):
        return {"error": "rocprofv3 not found"}
    if "rocprof" in os.environ.get("LD_PRELOAD", "") or os.environ.get("ROCPROFILER_REGISTER_FORCE_LOAD"):
        return {"error": "this process already runs under a profiler"}
    tmp = tempfile.mkdtemp(prefix="rof_pmc_", dir="/tmp")
    env = dict(os.environ, TMPDIR="/tmp")
    per = {}     # (counter, phase) -> mean value per dispatch; phase 0 = partial-sum launch, 1 = destination rows
    copy = {}    # counter -> value of the calibration copy
    try:
        for tag, counters in (("fetch", ["FETCH_SIZE"]), ("write", ["WRITE_SIZE"]), ("tcc", ["TCC_HIT_sum", "TCC_MISS_sum"])):
            out_dir = os.path.join(tmp, tag)
            cmd = [prof, "--pmc", *counters, "-d", out_dir, "-o", "rof", "-f", "csv",
                   "--", sys.executable, os.path.abspath(__file__), "--traffic-child", *passthrough]
            log(f"[bench] counter run: {' '.join(cmd)}")
            rc, text = run_group(cmd, "/tmp", env, 240)
            files = glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True)
            if rc != 0 or not files:
                return {"error": f"rocprofv3 --pmc {' '.join(counters)} failed (rc {rc}): " + text[-300:]}
            rows_per_phase, copy_values = read_counter_csv(files[0])
            copy.update(copy_values)
            per.update(rows_per_phase)
    except (OSError, subprocess.SubprocessError, ValueError, KeyError, IndexError) as ex:
        return {"error": f"counter runs failed: {ex!r}"[:300]}
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    if "FETCH_SIZE" not in copy or "WRITE_SIZE" not in copy or ("FETCH_SIZE", 1) not in per:
        return {"error": "counter output lacks the expected kernels"}
    # the counters report KiB; what they read for a copy of known size gives the factor that turns them into bytes
    f_scale = COPY_BYTES / (copy["FETCH_SIZE"] * 1024.0)
    w_scale = COPY_BYTES / (copy["WRITE_SIZE"] * 1024.0)
    res = {"source": "live: this script under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE / TCC_HIT_sum TCC_MISS_sum, "
                     f"one counter set per child process, mean over {CHILD_AGGREGATIONS} aggregations",
           "fetch_scale": f_scale, "write_scale": w_scale, "launch": {}}
    for phase in (0, 1):
        if ("FETCH_SIZE", phase) not in per:
            continue
        rd = per[("FETCH_SIZE", phase)] * 1024.0 * f_scale
        wr = per.get(("WRITE_SIZE", phase), 0.0) * 1024.0 * w_scale
        hit, miss = per.get(("TCC_HIT_sum", phase)), per.get(("TCC_MISS_sum", phase))
        res["launch"][phase] = {"read_bytes": rd, "written_bytes": wr, "bytes": rd + wr,
                                "tcc_hit_rate": hit / (hit + miss) if hit is not None and miss else None,
                                "tcc_miss_x_128B": miss * 128.0 if miss is not None else None,
                                "tcc_hit_x_128B": hit * 128.0 if hit is not None else None}
    return res


def read_calibration(L, dev, gather_lanes=0):
    """What plain streaming reaches on this device, as yardsticks for the gather launches' fetch rate: reads of a
    buffer far beyond the caches (2 GiB: HBM), reads of a buffer that the 256 MB Infinity Cache holds but the L2s do
    not (128 MiB, read repeatedly), reads that the L2s serve (16 MiB, read 128 times in one launch), and
    a 1 GiB device-to-device copy (read + write).  GB/s, HIP events on the current stream, best of three."""
    import ctypes

    import torch

    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    big = torch.empty((2 << 30) // 4, dtype=torch.float32, device=dev).normal_()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def rate(fn, nbytes, reps):
        best = 0.0
        for _ in range(3):
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            best = max(best, nbytes * reps / (e0.elapsed_time(e1) * 1e-3) / 1e9)
        return best

    def read(buf, nbytes, repeat=1):
        return lambda: _check_rc(L.rof_device_read(ctypes.c_void_p(buf.data_ptr()), nbytes, repeat,
                                                   ctypes.c_void_p(sink.data_ptr()), st))

    res = {"hbm_stream_read_GBs": rate(read(big, 2 << 30), 2 << 30, 4),
           "infinity_cache_read_GBs": rate(read(big, 128 << 20), 128 << 20, 64),
           # 16 MiB read 128 times in one launch: a workgroup reads the same pieces every time, so each XCD's 4 MB L2
           # holds its eighth of the buffer after the first pass
           "l2_read_GBs": rate(read(big, 16 << 20, 128), (16 << 20) * 128, 4)}
    if gather_lanes in (4, 8, 10, 12, 16, 20, 32, 64):
        # nothing but gathers of rows as wide as the workload's (16 bytes per lane), pseudo-random, two in flight: from
        # a table that the L2s hold, that the Infinity Cache holds, and that only HBM holds; GB/s of gathered row bytes
        row = 16 * gather_lanes
        got = ctypes.c_uint64()
        gres = {"row_bytes": row}
        for tag, table_bytes, iters in (("l2", 1 << 20, 1000), ("infinity_cache", 48 << 20, 250), ("hbm", 2 << 30, 250)):
            rows = 1 << int(np.floor(np.log2(table_bytes // row)))

            def gather(rows=rows, iters=iters):
                _check_rc(L.rof_device_gather(ctypes.c_void_p(big.data_ptr()), rows, gather_lanes, iters,
                                              ctypes.c_void_p(sink.data_ptr()), st, ctypes.byref(got)))

            gather()
            gres[tag + "_GBs"] = rate(gather, got.value * row, 1)
        res["row_gathers"] = gres
    half = big[: (1 << 30) // 4]
    other = big[(1 << 30) // 4:]
    res["copy_read_plus_write_GBs"] = rate(lambda: _check_rc(L.rof_device_copy(
        ctypes.c_void_p(other.data_ptr()), ctypes.c_void_p(half.data_ptr()), 1 << 30, st)), 2 << 30, 4)
    del big, half, other
    return res


def _check_rc(rc):
    from artifact_amd import _lib

    _lib.check(rc)


def restrided(t):
    """Copy of `t` whose row stride is a multiple of four floats (the alternative to gathering packed rows in
    place that the backward figures compare against)."""
    f = t.shape[1]
    pad = (-f) % 4
    if pad == 0:
        return t
    buf = t.new_empty(t.shape[0], f + pad)
    buf[:, :f].copy_(t)
    buf[:, f:].zero_()
    return buf


def part_size_sweep(name, sizes, have, n, e, x, deg, normalized, feat, lpr, in_bytes, args, out):
    """ms / GEdges/s per aggregation for each part size (upstream's drivers default to 3 and 5:
    ROF_evaluation/ROF_main.py:73, cuda/middle-rof.py:20), with what the plan picked and what it saves."""
    rows = []
    for ps in sizes:
        d = have.get(ps) or load_or_build(name, ps, args.cache_dir)[0]
        reuse, plain, forced = build_layouts(d, n, ps, lpr, in_bytes, args)
        row = {"part_size": ps, "picked_parts": int(len(d["index_picked"]))}
        for tag, lay in (("reuse", reuse), ("reuse_disabled", plain), ("reuse_forced", forced)):
            if lay is None:
                continue
            lay.upload()
            if normalized:
                lay.set_degrees(deg)
            lay.aggregate(x, normalized, out=out, feat_dim=feat)
            ms = float(np.median([lay.aggregate_timed(x, 10, normalized, out=out, feat_dim=feat)[0] for _ in range(3)]))
            st = lay.stats()
            row[tag + "_ms"] = ms
            if tag == "reuse":
                row.update(GEdges_per_s=e / (ms * 1e-3) / 1e9, materialised_groups=st["materialised_groups"],
                           clusters=st["cluster_workgroups"], local_groups=st["local_groups"],
                           plan_saved_gathers_frac=1.0 - len(d["uniqpart_column_index"]) / max(1, e))
            if tag == "reuse_forced":
                row["forced_saved_gathers_frac"] = 1.0 - (st["gathered_rows"] + st["partial_reads"] - st["hub_segments"]) / max(1, e)
            lay.close()
        rows.append(row)
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c4", choices=sorted(DESCR))
    ap.add_argument("--part-size", type=int, default=3)
    ap.add_argument("--feat", type=int, default=0, help="override the aggregated width")
    ap.add_argument("--cache-dir", default="/tmp/rof_bench_cache")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-traffic", action="store_true", help="skip the rocprofv3 counter runs (HBM-side bytes)")
    ap.add_argument("--no-sweep", action="store_true", help="skip the part-size sweep 2..5")
    ap.add_argument("--quick", action="store_true", help="only the headline timing: no counters, sweep, model step or CPU leg")
    ap.add_argument("--traffic-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--xcd-run", type=int, default=0, help="launch tuning: workgroups per XCD run, destination rows")
    ap.add_argument("--xcd-run-partial", type=int, default=0, help="same for the partial-sum launches")
    ap.add_argument("--wave-cap", type=int, default=-1,
                    help="launch tuning: wavefronts per SIMD of the destination-row launch (0 = all, 2..7; -1 = the library's rule)")
    ap.add_argument("--padded-output", action="store_true",
                    help="store the output in rows of the input's stride (47 floats in rows of 48, rof_epilogue."
                         "pad_columns) instead of the packed [N, feat] tensor the operator API returns")
    ap.add_argument("--packed-input", action="store_true",
                    help="gather rows that are `feat` elements apart (47 floats = 188 bytes), the way the backward pass "
                         "meets its gradient, instead of rows in a stride that is a multiple of 16 bytes")
    ap.add_argument("--hub-split", type=int, default=0, help="layout tuning: rows longer than this are segmented")
    ap.add_argument("--segment", type=int, default=0, help="layout tuning: entries per segment")
    ap.add_argument("--min-consumers", type=int, default=0, help="layout tuning: share groups with >= this many consumers")
    ap.add_argument("--autotune", action="store_true",
                    help="also time the layout that LayoutFamily(autotune=True) picks (candidate cuts of long rows and "
                         "launch settings chosen by timing) against the size rules' choice")
    ap.add_argument("--share-scope", default="all", choices=["all", "long_rows"],
                    help="layout tuning: which consumers read shared groups from the workspace")
    ap.add_argument("--lds-pad", type=int, default=-1, help="launch tuning: unused LDS bytes per workgroup")
    ap.add_argument("--entry-order", default="descending", choices=["descending", "plan", "ascending"],
                    help="layout tuning: order of the gathered rows inside a task")
    ap.add_argument("--tile-rows", type=int, default=0, help="layout tuning: destinations per length-sorted tile")
    ap.add_argument("--search", default="upstream", choices=["upstream", "hub", "dynamic"],
                    help="reuse search: upstream's greedy (bit-exact plan), the hub-pattern search, or the dynamic "
                         "greedy that upstream sketches")
    ap.add_argument("--hubs", type=int, default=16384, help="--search hub: number of hub sources")
    ap.add_argument("--block", type=int, default=8, help="--search hub: hubs per block (= part size of the plan)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every machine of this build has a single MI355X and the aggregation "
                 "path has no multi-GPU part; run with --gpus 1")
    if args.traffic_child:
        return traffic_child(args)
    if args.quick:
        args.no_traffic = args.no_sweep = args.no_cpu_baseline = True

    name, ps = args.workload, args.part_size
    feat = args.feat or FEAT[name]
    normalized = name != "c3"
    bf16 = name == "c5"
    default_opts = (not (args.hub_split or args.segment or args.tile_rows or args.xcd_run
                         or args.xcd_run_partial or args.lds_pad >= 0 or args.wave_cap >= 0 or args.share_scope != "all")
                    and args.search == "upstream" and args.entry_order == "descending")

    # ---- host side first: graph and plan (cached on disk), then the counter runs in child processes; this
    # process has not touched the GPU yet.  (PyTorch is imported before librof.so is loaded so that both use the
    # HIP runtime PyTorch brings; importing it does not initialise the device.)
    import torch

    if torch.cuda.device_count() == 0:   # (counting devices does not initialise one)
        sys.exit("bench.py needs a GPU: no HIP device is visible")
    d, t_gen, t_plan = load_or_build(name, ps, args.cache_dir)
    traffic = {"error": "switched off (--no-traffic / --quick) or non-default options"}
    if not args.no_traffic and default_opts:
        passthrough = ["--workload", name, "--part-size", str(ps), "--cache-dir", args.cache_dir]
        if args.feat:
            passthrough += ["--feat", str(args.feat)]
        if args.padded_output:
            passthrough += ["--padded-output"]
        if args.packed_input:
            passthrough += ["--packed-input"]
        if args.min_consumers:
            passthrough += ["--min-consumers", str(args.min_consumers)]
        traffic = measure_traffic(args, passthrough)
        if "error" in traffic:
            log(f"[bench] live counters unavailable: {traffic['error']}")

    from artifact_amd import _lib
    from artifact_amd.layout import Layout, lanes_per_row

    L = _lib.lib()   # raises if the HIP library is missing
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")

    indptr, indices = d["indptr"], d["indices"]
    n, e = len(indptr) - 1, len(indices)
    if args.search == "hub":
        from artifact_amd import reuse_search_ext as R

        t0 = time.time()
        hp = R.hub_pattern_plan(indptr, indices, args.hubs, args.block)
        t_plan = time.time() - t0
        for k in ("uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col"):
            d[k] = hp[k]
        d["index_picked"] = np.arange(hp["shared_parts"], dtype=np.uint32)
        ps = args.block
        log(f"[bench] hub-pattern plan: {t_plan:.1f}s, {hp['shared_parts']} shared parts")
    if args.search == "dynamic":
        from artifact_amd import reuse_search_ext as R

        t0 = time.time()
        dp = R.dynamic_greedy_plan(indptr, indices, ps)
        t_plan = time.time() - t0
        for k in ("uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col", "index_picked"):
            d[k] = dp[k]
        log(f"[bench] dynamic greedy plan: {t_plan:.1f}s, {dp['shared_parts']} shared parts of {dp['candidates']} "
            f"candidates")
    deg = torch.from_numpy(np.diff(indptr).astype(np.float32)).to(dev)

    calibration = None if args.quick else read_calibration(L, dev, lanes_per_row(feat, bf16))
    x, x32, ld = make_features(name, n, feat, bf16, dev, args.packed_input)
    in_bytes = 2 if bf16 else 4
    lpr = lanes_per_row(feat, bf16)
    args.row_bytes = feat * in_bytes
    t0 = time.time()
    reuse, plain, forced = build_layouts(d, n, ps, lpr, in_bytes, args)
    t_layout = time.time() - t0
    for lay in (reuse, plain) + ((forced,) if forced else ()):
        apply_tuning(lay, args)
        lay.upload()
        if normalized:
            lay.set_degrees(deg)
    # The output is the packed [N, feat] tensor the operator returns (reuse_conv_kernel.cu:303,1000).  With
    # --padded-output it has rows as wide as the input rows (47 floats in rows of 48, rof_epilogue.pad_columns);
    # columns 0 .. feat-1 are the same either way.
    pad = args.padded_output and ld != feat
    ldo = ld if pad else feat
    out = torch.empty((n, ldo), dtype=torch.float32, device=dev)[:, :feat]
    out_plain = torch.empty((n, ldo), dtype=torch.float32, device=dev)[:, :feat]

    # ---- warm-up: W steps, and at least ~0.3 s of work so the clocks have settled
    t0 = time.perf_counter()
    done = 0
    while done < args.warmup or time.perf_counter() - t0 < 0.3:
        reuse.aggregate(x, normalized, out=out, feat_dim=feat, pad_columns=pad)
        plain.aggregate(x, normalized, out=out_plain, feat_dim=feat, pad_columns=pad)
        done += 1
        if done % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps between synchronisations
    t0 = time.perf_counter()
    for _ in range(args.steps):
        reuse.aggregate(x, normalized, out=out, feat_dim=feat, pad_columns=pad)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- launch-bound workloads only: the same step captured in a HIP graph and replayed, alone and eight to a graph
    # (a model's forward pass holds several aggregations).  The call only enqueues kernels -- no allocation, no
    # synchronisation, no memset -- so a replay costs the host one graph launch instead of one launch per kernel.
    graph_replay = None
    if wall_ms < 0.1:
        graph_replay = {"steps_per_graph": [], "ms_per_step": []}
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            reuse.aggregate(x, normalized, out=out, feat_dim=feat, pad_columns=pad)
        torch.cuda.current_stream().wait_stream(side)
        for per_graph in (1, 8):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(per_graph):
                    reuse.aggregate(x, normalized, out=out, feat_dim=feat, pad_columns=pad)
            replays = max(1, args.steps // per_graph)
            for _ in range(max(2, replays // 4)):
                graph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(replays):
                graph.replay()
            torch.cuda.synchronize()
            graph_replay["steps_per_graph"].append(per_graph)
            graph_replay["ms_per_step"].append((time.perf_counter() - t0) * 1e3 / (replays * per_graph))
            del graph

    # ---- HIP-event timings on the launch stream; reuse and reuse-disabled alternate so that drift
    # of clocks or temperature hits both alike
    per = max(5, args.steps // 4)
    ev_r, ev_p = [], []
    for _ in range(4):
        ev_r.append(reuse.aggregate_timed(x, per, normalized, out=out, feat_dim=feat, pad_columns=pad)[0])
        ev_p.append(plain.aggregate_timed(x, per, normalized, out=out_plain, feat_dim=feat, pad_columns=pad)[0])
    ev_ms, plain_ms = float(np.median(ev_r)), float(np.median(ev_p))
    # per-call spread the way the upstream micro-benchmark samples it (10 warm-ups + 100 timed runs,
    # ROF_evaluation/cuda/small-main.py:364-390), one HIP-event pair per call
    singles = sorted(reuse.aggregate_timed(x, 1, normalized, out=out, feat_dim=feat, pad_columns=pad)[0] for _ in range(100))
    spread = {"runs": 100, "median_ms": float(np.median(singles)), "p10_ms": float(np.percentile(singles, 10)),
              "p90_ms": float(np.percentile(singles, 90))}
    forced_info = None
    if forced is not None:
        out_f = torch.empty((n, ldo), dtype=torch.float32, device=dev)[:, :feat]
        forced.aggregate(x, normalized, out=out_f, feat_dim=feat, pad_columns=pad)
        ev_f, ev_p2 = [], []
        for _ in range(4):
            ev_f.append(forced.aggregate_timed(x, per, normalized, out=out_f, feat_dim=feat, pad_columns=pad)[0])
            ev_p2.append(plain.aggregate_timed(x, per, normalized, out=out_plain, feat_dim=feat, pad_columns=pad)[0])
        fs = forced.stats()
        forced_info = {"min_consumers": 3, "event_ms": float(np.median(ev_f)),
                       "speedup_vs_reuse_disabled": float(np.median(ev_p2) / np.median(ev_f)),
                       "materialised_groups": fs["materialised_groups"],
                       "saved_gathers_frac": 1.0 - (fs["gathered_rows"] + fs["partial_reads"] - fs["hub_segments"]) / max(1, e),
                       "max_abs_diff_vs_reuse_disabled": float((out_f - out_plain).abs().max())}
        del out_f
    ms_a, ms_b = reuse.launch_times(x, max(5, args.steps // 2), normalized, out=out, feat_dim=feat, pad_columns=pad)
    pms_a, pms_b = plain.launch_times(x, max(5, args.steps // 2), normalized, out=out_plain, feat_dim=feat, pad_columns=pad)
    torch.cuda.synchronize()
    max_diff = float((out - out_plain).abs().max())

    extra = {}
    if args.autotune:
        # the cut of long rows and the launch settings chosen by timing candidates (LayoutFamily(autotune=True)) against
        # the size rules' choice, timed in turn
        from artifact_amd.layout import LayoutFamily

        v2 = (d["uniqpart_column_index"], d["uniqpart_pointers"], d["part2Node_ptr"], d["part2Node_col"], n, ps)
        t0 = time.time()
        fam = LayoutFamily(lambda lpr_, eb, rb=0, **kw: Layout.from_v2(*v2, lanes_per_row=lpr_, elem_bytes=eb, row_bytes=rb, **kw),
                           autotune=True)
        tuned = fam.get(feat, bf16, normalized)
        t_tune = time.time() - t0
        if normalized:
            tuned.set_degrees(deg)
        tuned.aggregate(x, normalized, out=out_plain, feat_dim=feat, pad_columns=pad)
        ev_t, ev_d = [], []
        for _ in range(4):
            ev_t.append(tuned.aggregate_timed(x, per, normalized, out=out_plain, feat_dim=feat, pad_columns=pad)[0])
            ev_d.append(reuse.aggregate_timed(x, per, normalized, out=out, feat_dim=feat, pad_columns=pad)[0])
        extra["autotune"] = {"chosen": {f"{k}": v for k, v in fam.chosen.items()}, "seconds": t_tune,
                             "event_ms": float(np.median(ev_t)), "rule_event_ms": float(np.median(ev_d)),
                             "speedup_over_rule": float(np.median(ev_d) / np.median(ev_t)),
                             "max_abs_diff_vs_rule": float((out - out_plain).abs().max())}
        fam.close()
    if not args.no_sweep and not args.feat and args.search == "upstream":
        extra["part_size_sweep"] = part_size_sweep(name, (2, 3, 4, 5), {ps: d}, n, e, x, deg, normalized, feat, lpr,
                                                   in_bytes, args, out_plain)

    # ---- the backward aggregation (same plan on the gradient, reuse_conv_kernel.cu:1021-1041): the gradient
    # arrives packed [N, F] and is gathered in place; the result is an intermediate and keeps padded rows
    if not bf16 and not args.quick:
        grad = torch.randn((n, feat), device=dev)
        gout = torch.empty((n, ld), dtype=torch.float32, device=dev)[:, :feat]
        ev0, ev1, ev2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        t_pad, t_agg = [], []
        for _ in range(10):
            ev0.record()
            gp = restrided(grad)
            ev1.record()
            reuse.aggregate(gp, normalized, out=gout, feat_dim=feat, pad_columns=True)
            ev2.record()
            torch.cuda.synchronize()
            t_pad.append(ev0.elapsed_time(ev1))
            t_agg.append(ev1.elapsed_time(ev2))
        t_packed = []
        for _ in range(10):
            ev0.record()
            reuse.aggregate(grad, normalized, out=gout, feat_dim=feat, pad_columns=True)
            ev1.record()
            torch.cuda.synchronize()
            t_packed.append(ev0.elapsed_time(ev1))
        # packed_rows_ms is what the operator path does (rows gathered in place at 4-byte alignment); the other two
        # numbers are the alternative of re-striding the gradient to 16-byte rows first
        extra["backward_aggregation"] = {"packed_rows_ms": float(np.median(t_packed)),
                                         "restride_ms": float(np.median(t_pad)), "aggregate_ms": float(np.median(t_agg))}
        del grad, gp, gout

    # ---- continuity with the upstream micro-benchmark (ROF_evaluation/cuda/small-main.py:357-478): the whole
    # ROF.reuse_forward_v2 call, dense update included, 10 warm-ups + 100 runs, events on the current stream
    dims = {"c1": (32, 32), "c2": (128, 256), "c4": (100, 47)}.get(name)
    if dims and not args.feat and not args.quick:
        from artifact_amd import ROF as rof_api
        from artifact_amd.layout import LayoutFamily

        fam = LayoutFamily(lambda _lpr: reuse)
        xin = torch.randn((n, dims[0]), device=dev)
        wgt = torch.randn((dims[0], dims[1]), device=dev)
        dummy = torch.zeros(1, dtype=torch.int32, device=dev)   # plan tensors are not read when a layout is passed
        call = lambda: rof_api.reuse_forward_v2(xin, wgt, dummy, deg, dummy, dummy, dummy, ps, min(32, dims[1]), 4,
                                                layout=fam)[0]
        for _ in range(10):
            call()
        ts, tg = [], []
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(100):
            e0.record()
            call()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1))
        for _ in range(20):
            e0.record()
            rof_api._update(xin, wgt)
            e1.record()
            torch.cuda.synchronize()
            tg.append(e0.elapsed_time(e1))
        extra["whole_reuse_forward_v2"] = {"in_dim": dims[0], "out_dim": dims[1], "mean_ms": float(np.mean(ts)),
                                           "std_ms": float(np.std(ts)), "median_ms": float(np.median(ts)),
                                           "dense_update_ms": float(np.median(tg)),
                                           "minus_dense_update_ms": float(np.median(ts) - np.median(tg))}
        fam._by_lpr.clear()   # the layout is owned by this function, not by the family
        del xin, wgt

    # ---- the rest of the layer: bias + ReLU stored by the aggregation kernel against the two elementwise
    # passes upstream runs after its operator (reuse_conv.py:147-150, ROF_main.py:181); and, where the
    # layer's dimensions are known, both orders of update and aggregation
    def timed(fn, reps=20):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ts = []
        for _ in range(reps):
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1))
        return float(np.median(ts))

    if normalized and not args.feat and not args.quick:
        bias_t = torch.randn(feat, device=dev)
        t_fused = timed(lambda: reuse.aggregate(x, True, out=out_plain, feat_dim=feat, bias=bias_t, relu=True))
        t_sep = timed(lambda: torch.relu_(reuse.aggregate(x, True, out=out_plain, feat_dim=feat).add_(bias_t)))
        extra["epilogue"] = {"fused_bias_relu_ms": t_fused, "separate_passes_ms": t_sep, "speedup": t_sep / t_fused}
    if dims and not args.feat and not bf16 and not args.quick:
        from artifact_amd import ROF as rof_api

        fin, fout = dims
        xin = torch.randn((n, fin), device=dev)
        wgt = torch.randn((fin, fout), device=dev)
        fam_in, fam_out = lanes_per_row(fin, False), lanes_per_row(fout, False)
        lays = {lpr: reuse}
        for want in (fam_in, fam_out):
            if want not in lays:
                lays[want] = Layout.from_v2(d["uniqpart_column_index"], d["uniqpart_pointers"], d["part2Node_ptr"],
                                            d["part2Node_col"], n, ps, lanes_per_row=want)
                lays[want].upload()
                lays[want].set_degrees(deg)
        hbuf = torch.empty((n, fin), device=dev)
        obuf = torch.empty((n, fout), device=dev)

        def update_first():
            tmp, f = rof_api._update(xin, wgt)
            lays[fam_out].aggregate(tmp, True, out=obuf, feat_dim=f)

        def aggregate_first():
            lays[fam_in].aggregate(xin, True, out=hbuf, feat_dim=fin)
            torch.mm(hbuf, wgt, out=obuf)

        extra["layer_order"] = {"in_dim": fin, "out_dim": fout, "update_first_ms": timed(update_first),
                                "aggregate_first_ms": timed(aggregate_first),
                                "aggregate_only_at_in_dim_ms": timed(
                                    lambda: lays[fam_in].aggregate(xin, True, out=hbuf, feat_dim=fin))}
        for k, lay in lays.items():
            if lay is not reuse:
                lay.close()
        del xin, wgt, hbuf, obuf

    # ---- the workload's model step end to end (dense updates, bias, activation, backward where the workload has
    # one), upstream's sequence of separate passes against the fused layer; the aggregation layouts are shared
    if not args.feat and name in MODEL_STEPS and not args.quick:
        extra["model_step"] = model_step(name, d, n, ps, deg, dev, timed)

    st = reuse.stats()
    bytes_a, bytes_b = reuse.launch_bytes(feat, in_bytes)
    b_alg = reuse.algorithmic_bytes(feat, in_bytes)
    b_alg_plain = plain.algorithmic_bytes(feat, in_bytes)
    b_noreuse_model = e * (4 + feat * in_bytes) + n * (feat * 4 + 8)
    b_min = n * feat * in_bytes + 4 * e + n * feat * 4      # every feature row once, every column id, every output row
    if "error" in traffic:
        key = (name, ps, feat, not pad)
        off = PROFILED_TRAFFIC.get(key) if default_opts and not args.min_consumers else None
        if off:
            traffic = dict(off, source="offline profile (profiles/): the live counter runs were not available: "
                                       + traffic["error"])
    tl = traffic.get("launch", {})

    def gather_model(t, ms):
        """The launch against what nothing-but-gathers reaches on this device: its L2 hits priced at the rate of row
        gathers that the L2s serve, its L2 misses at the rate of row gathers from HBM (and from the Infinity Cache),
        in 128-byte lines (a gathered row of R bytes occupies ceil(R / 128) lines).  An estimate, not a bound: misses
        with locality (the swept launch) or served by the Infinity Cache come faster than random rows from HBM, stores
        are priced like gathers.  A launch close to it does little else than wait for its lines."""
        g = (calibration or {}).get("row_gathers")
        if not g or not t or not t.get("tcc_hit_x_128B") or not t.get("tcc_miss_x_128B") or ms <= 0:
            return None
        per_row = -(-g["row_bytes"] // 128) * 128.0 / g["row_bytes"]      # line bytes fetched per useful byte
        hit_b, miss_b = t["tcc_hit_x_128B"], t["tcc_miss_x_128B"]
        ms_of = lambda tag: (hit_b / (g["l2_GBs"] * per_row) + miss_b / (g[tag] * per_row)) / 1e9 * 1e3
        return {"row_bytes": g["row_bytes"], "l2_hit_bytes": hit_b, "l2_miss_bytes": miss_b,
                "line_GBs": {"l2": g["l2_GBs"] * per_row, "infinity_cache": g["infinity_cache_GBs"] * per_row,
                             "hbm": g["hbm_GBs"] * per_row},
                "model_ms_misses_from_hbm": ms_of("hbm_GBs"), "model_ms_misses_from_infinity_cache": ms_of("infinity_cache_GBs"),
                "measured_ms": ms, "measured_over_model_hbm": ms / ms_of("hbm_GBs")}

    def roof(phase, label, alg_bytes, ms):
        t = tl.get(phase)
        tb = t["bytes"] if t and ms > 0 else None
        return {
            "bound": "hbm", "kernel": label,
            # What `traffic` counts: the fills and write-backs of the L2s (FETCH_SIZE / WRITE_SIZE), i.e. everything
            # that crosses from the XCDs to the memory side.  The 256 MB Infinity Cache sits behind those counters, so
            # a part of it never reaches HBM: `frac` is an upper bound of the HBM fraction, and only for a feature
            # matrix several times that cache (the 2^22-node bf16 workload) is it close to one.
            "traffic_kind": "L2 fills + write-backs (served by HBM and by the Infinity Cache behind the counters)",
            "achievable_read_GBs": calibration,
            # achieved / frac: memory-side bytes the launch really moved (profiler counters) over its duration
            "achieved": tb / (ms * 1e-3) / 1e9 if tb else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": tb / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS if tb else None,
            "traffic": tb, "traffic_read": t["read_bytes"] if t else None, "traffic_written": t["written_bytes"] if t else None,
            "tcc_hit_rate": t.get("tcc_hit_rate") if t else None,
            "tcc_miss_x_128B": t.get("tcc_miss_x_128B") if t else None,
            "gather_model": gather_model(t, ms),
            "ms_per_launch": ms,
            # the model figure: one gathered row per edge whether or not a cache served it; exceeds the HBM peak
            # when rows gathered many times come from L2 / Infinity Cache
            "algorithmic_bytes": alg_bytes, "algorithmic_GBs": alg_bytes / (ms * 1e-3) / 1e9 if ms > 0 else None,
            "algorithmic_frac": alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS if ms > 0 else None,
        }

    layer_traffic = (tl[1]["bytes"] + (tl[0]["bytes"] if 0 in tl else 0.0)) if 1 in tl else None
    result = {
        "metric": "GEdges/s per aggregation layer (reuse plan), 1 MI355X",
        "value": e / (wall_ms * 1e-3) / 1e9,
        "unit": "GEdges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16->f32" if bf16 else "f32",
        "data": "synthetic",
        "config": {"workload": DESCR[name], "nodes": n, "edges": e, "feat": feat, "row_stride": ld, "out_row_stride": ldo,
                   "output": "padded rows (pad_columns)" if pad else "packed [N, feat], as the operator API returns it",
                   "part_size": ps, "normalized": normalized, "search": args.search},
        "roofline": roof(1, ("rof_coop_kernel (destination-row launch of a small graph: long rows get several wavefronts of a workgroup each)"
                             if st.get("workgroup_rows") else "rof_rows_kernel (destination-row launch)"), bytes_b, ms_b),
        # the launch before it (segments of long rows, swept in the order of their source ids): same kernel
        # template, second in duration
        "roofline_partial_launch": roof(0, "rof_rows_kernel (partial-sum launch)", bytes_a, ms_a),
        "traffic_source": traffic.get("source", traffic.get("error")),
        "traffic_counter_scale": {"FETCH_SIZE": traffic.get("fetch_scale"), "WRITE_SIZE": traffic.get("write_scale")},
        "layer": {
            "event_ms": ev_ms, "event_ms_runs": ev_r, "graph_replay": graph_replay, "per_call": spread, "launch1_ms": ms_a, "launch2_ms": ms_b,
            "traffic": layer_traffic,
            "frac_of_hbm_peak": layer_traffic / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS if layer_traffic else None,
            "b_min": b_min, "traffic_over_b_min": layer_traffic / b_min if layer_traffic else None,
            "algorithmic_bytes": b_alg, "algorithmic_GBs": b_alg / (ev_ms * 1e-3) / 1e9,
            "algorithmic_frac": b_alg / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "no_reuse_model_bytes": b_noreuse_model,
        },
        "reuse_disabled": {
            "event_ms": plain_ms, "launch1_ms": pms_a, "launch2_ms": pms_b, "GEdges_per_s": e / (plain_ms * 1e-3) / 1e9,
            "algorithmic_GBs": b_alg_plain / (plain_ms * 1e-3) / 1e9, "speedup_of_reuse": plain_ms / ev_ms,
            "max_abs_diff_vs_reuse": max_diff,
        },
        "reuse_forced": forced_info,
        "plan": {"groups": st["groups"], "materialised_groups": st["materialised_groups"],
                 "folded_by_cost_model": bool(st["materialised_groups"] == 0 and st["local_groups"] == 0 and st["groups"] > 0),
                 "gathered_rows": st["gathered_rows"], "partial_reads": st["partial_reads"],
                 "partial_rows": st["partial_rows"], "hub_segments": st["hub_segments"],
                 "local_groups": st["local_groups"], "lds_reads": st["lds_reads"], "clusters": st["cluster_workgroups"],
                 "saved_gathers_frac": 1.0 - (st["gathered_rows"] + st["partial_reads"] - st["hub_segments"]) / max(1, e),
                 "executed_as": ("reuse-disabled schedule (the cost model folded every group)"
                                 if st["materialised_groups"] == 0 and st["local_groups"] == 0 else
                                 "groups shared" + (" in LDS by clustered workgroups" if st["local_groups"] else "")
                                 + (" and" if st["local_groups"] and st["materialised_groups"] else "")
                                 + (" through workspace rows" if st["materialised_groups"] else "")),
                 "cpu_graph_s": t_gen, "cpu_plan_s": t_plan, "cpu_layout_s": t_layout},
    }

    result.update(extra)

    if not args.no_cpu_baseline:
        from oracle import oracle as O  # checker + CPU baseline leg only

        cpu_s, runs, threads, cpu_out = cpu_baseline(indptr, indices, np.ascontiguousarray(x32), normalized)
        got = out.cpu().numpy()
        err = float(np.abs(got - cpu_out).max())
        result["cpu_baseline"] = {
            "value": e / cpu_s / 1e9, "unit": "GEdges/s", "cores": threads, "kind": "port",
            "sample": f"the full {name} layer (same graph and features), median of {runs} passes of the oracle's "
                      f"destination-parallel SpMM (oracle/agg_oracle.c) after one warm-up",
            "ms_per_layer": cpu_s * 1e3, "max_abs_diff_gpu_vs_cpu": err,
        }
        try:
            torch.set_num_threads(threads)
            rs = O.rsqrt_rn(np.diff(indptr).astype(np.float32))
            rs[~np.isfinite(rs)] = 0.0
            vals = torch.from_numpy((rs[np.repeat(np.arange(n), np.diff(indptr))] * rs[indices]).astype(np.float32)
                                    if normalized else np.ones(e, dtype=np.float32))
            a = torch.sparse_csr_tensor(torch.from_numpy(indptr.astype(np.int64)),
                                        torch.from_numpy(indices.astype(np.int64)), vals, size=(n, n))
            xt = torch.from_numpy(np.ascontiguousarray(x32))
            torch.sparse.mm(a, xt)
            ts = []
            for _ in range(3):
                t0 = time.time()
                torch.sparse.mm(a, xt)
                ts.append(time.time() - t0)
            result["cpu_baseline"]["torch_sparse_mm_GEdges_per_s"] = e / float(np.median(ts)) / 1e9
        except Exception as ex:  # the library leg is informative only
            result["cpu_baseline"]["torch_sparse_mm_error"] = str(ex)[:200]
        try:   # one thread of scipy's CSR x dense, as a sanity line
            import scipy.sparse as sp

            rs = O.rsqrt_rn(np.diff(indptr).astype(np.float32))
            rs[~np.isfinite(rs)] = 0.0
            data = (rs[np.repeat(np.arange(n), np.diff(indptr))] * rs[indices]).astype(np.float32) if normalized \
                else np.ones(e, dtype=np.float32)
            a = sp.csr_matrix((data, indices, indptr), shape=(n, n))
            xs = np.ascontiguousarray(x32)
            t0 = time.time()
            a @ xs
            result["cpu_baseline"]["scipy_1_thread_GEdges_per_s"] = e / (time.time() - t0) / 1e9
        except Exception as ex:
            result["cpu_baseline"]["scipy_error"] = str(ex)[:200]

        # the host half of the path: upstream's own plan builder (compiled from its sources into oracle/_ref,
        # when that build is present) beside this library's, same graph, same threads, results compared
        try:
            from artifact_amd.graphgen import make_workload

            from artifact_amd import reuse_search_ext as RS

            ip_s, ix_s = make_workload("c2", 1)
            t0 = time.time()
            mine = RS.build_plan(ip_s, ix_s, 3)
            t_mine = time.time() - t0
            pb = {"sample": f"R-MAT {len(ip_s) - 1} nodes, {len(ix_s)} edges, part size 3 (half of c2)",
                  "threads": threads, "this_library_s": t_mine, "upstream_s": None}
            if O.ref_module() is not None:
                t0 = time.time()
                theirs = O.ref_plan(ip_s, ix_s, 3)
                pb["upstream_s"] = time.time() - t0
                pb["speedup"] = pb["upstream_s"] / t_mine
                pb["identical"] = all(np.array_equal(mine[k], theirs[k]) for k in theirs
                                      if k in mine and isinstance(theirs[k], np.ndarray))
            result["cpu_baseline"]["plan_builder"] = pb
        except Exception as ex:
            result["cpu_baseline"]["plan_builder_error"] = str(ex)[:200]

    print(json.dumps(result))


if __name__ == "__main__":
    main()
