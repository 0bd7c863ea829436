"""Device layout of a reuse plan: host-side handle around `rof_layout` (include/rof.h).

A layout is built from plan arrays in any of the three upstream tensor formats and owns the
device copy of its execution schedule.  `aggregate` runs the two kernel launches on the current
PyTorch stream; PyTorch is used only for device memory and the stream handle.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import LayoutOpts, RofError, bag_take, check, i32, ptr

ROF_F32, ROF_BF16 = 0, 1
NOALLOC_WORKSPACE_BYTES = 64 << 20   # ROF_NOALLOC_WORKSPACE_BYTES of include/rof.h

STAT_NAMES = ("nodes", "edges", "groups", "materialised_groups", "gathered_rows", "partial_reads", "partial_rows",
              "hub_segments", "tasks_a", "tasks_b", "device_bytes", "part_size", "wave_tasks_a", "wave_tasks_b",
              "canonical", "gathered_rows_a", "local_groups", "lds_reads", "cluster_workgroups", "lds_rows", "hub_split",
              "segment", "longest_row_task", "workgroup_rows")

EXPORT_NAMES = ("group_ptr", "group_col", "group_dst_ptr", "group_dst", "res_ptr", "res_col", "canonical", "xcd_run", "long_row_cut",
                "uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr", "part2Node_col",
                "g_task_ptr", "g_task_nref", "g_task_out", "g_col", "s_task_ptr", "s_task_nref", "s_task_out", "s_col",
                "b_task_ptr", "b_task_nref", "b_task_out", "b_col", "b_task_nlds", "b_lg_ptr", "b_lg_task_ptr", "b_lg_col", "b_lg_task_first",
                "b_shape")


def column_sums(t):
    """float32 column sums of a 2-D float32 / bfloat16 CUDA tensor with unit column stride (rof_column_sums):
    the bias gradient of a layer.  Fixed summation order, so the result is bitwise repeatable."""
    import torch

    if not t.is_cuda or t.dim() != 2 or t.stride(1) != 1 or t.dtype not in (torch.float32, torch.bfloat16):
        raise RofError("column_sums needs a 2-D float32 or bfloat16 CUDA tensor with unit column stride")
    n, f = t.shape
    out = torch.empty(f, dtype=torch.float32, device=t.device)
    if f == 0:
        return out
    L = _lib.lib()
    nbytes = L.rof_column_sums_workspace_bytes(max(n, 1), f)
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=t.device)
    with torch.cuda.device(t.device):
        check(L.rof_column_sums(C.c_void_p(t.data_ptr()), ROF_BF16 if t.dtype == torch.bfloat16 else ROF_F32,
                                t.stride(0) if n > 1 else max(f, t.stride(0)), n, f, C.c_void_p(out.data_ptr()),
                                C.c_void_p(ws.data_ptr()), nbytes, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    return out


def lanes_per_row(feat_dim, bf16=False):
    """Lanes one gathered row occupies in the kernel: the smallest of 4, 8, 10, 12, 16, 20, 32, 64 that
    covers ceil(F / elements per 16-byte load) (mirrors rof_lanes_per_row in csrc/agg_kernels.hip)."""
    need = -(-int(feat_dim) // (8 if bf16 else 4))
    for lpr in (4, 8, 10, 12, 16, 20, 32, 64):
        if lpr >= need:
            return lpr
    return 64


ENTRY_ORDERS = {"descending": 0, "plan": 1, "ascending": 2}
SHARE_SCOPES = {"all": 0, "long_rows": 1}


def _opts(min_consumers=0, disable_reuse=False, hub_split=0, segment=0, lanes_per_row=0, entry_order="descending",
          tile_rows=0, elem_bytes=0, local_groups=0, share_scope="all", row_bytes=0):
    o = LayoutOpts()
    o.min_consumers = int(min_consumers)
    o.disable_reuse = int(bool(disable_reuse))
    o.hub_split = int(hub_split)
    o.segment = int(segment)
    o.lanes_per_row = int(lanes_per_row)
    o.entry_order = ENTRY_ORDERS[entry_order]
    o.tile_rows = int(tile_rows)
    o.elem_bytes = int(elem_bytes)
    o.local_groups = int(local_groups)
    o.share_scope = SHARE_SCOPES[share_scope]
    o.row_bytes = int(row_bytes)
    return o


# (cut, segment) candidates that an autotuned family times against the rule's choice, by element size
CUT_CANDIDATES = {4: ((128, 32), (512, 64), (1024, 128), (2048, 256)), 2: ((256, 48), (256, 128), (640, 160), (1280, 320))}


def autotune_default():
    """Whether layout families time their candidates by default: the environment variable ROF_AUTOTUNE=1."""
    import os

    return os.environ.get("ROF_AUTOTUNE", "0") not in ("", "0", "false", "no")


class LayoutFamily:
    """Layouts of one plan, one per width class (lanes per row, element size, and at one row per wavefront whether a
    row has 1024 bytes): how finely long rows are cut depends on how many rows a wavefront gathers at once and on how
    wide a partial-sum row is against a gathered one, i.e. on the feature width and type the layout will be used with.

    `build(lanes_per_row, elem_bytes, row_bytes, **overrides)` returns a Layout (builders that take only the first
    one or two arguments are accepted; they cannot be autotuned).  With `autotune` the first use of a width class on a
    GPU builds the rule's layout and the candidates of CUT_CANDIDATES, times one aggregation of random rows of that
    width with each (HIP events, two rounds in turn), keeps the fastest and lets it choose its launch settings by
    timing too (`Layout.calibrate`); `chosen[key]` records what was taken.  That costs a few layout builds and a few
    dozen aggregations per width class, once.  `choices` (what `choices()` of an earlier family returned, e.g. read back
    from a saved plan) replays recorded decisions instead of timing: the same cut, segment and launch settings, hence
    the same summation order and the same bits as the run that made them."""

    def __init__(self, build, autotune=None, choices=None):
        self._build = build
        self._by_lpr = {}
        self.autotune = autotune_default() if autotune is None else bool(autotune)
        self.chosen = {}
        self._replay = {}
        for k, v in (choices or {}).items():
            key = tuple(int(p) for p in k.split(",")) if isinstance(k, str) else tuple(k)
            self._replay[key] = {"cut": int(v["cut"]), "segment": int(v["segment"]),
                                 "tuning": {n: int(x) for n, x in v.get("tuning", {}).items()}}
        try:
            import inspect

            params = inspect.signature(build).parameters.values()
            self._nargs = sum(p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD) for p in params)
            self._kw = any(p.kind == p.VAR_KEYWORD for p in params)
        except (TypeError, ValueError):
            self._nargs, self._kw = 1, False

    def _make(self, key, **over):
        lpr, eb, rb = key
        if self._nargs >= 3:
            return self._build(lpr, eb, rb, **over)
        return self._build(lpr, eb) if self._nargs == 2 else self._build(lpr)

    def get(self, feat_dim, bf16=False, normalized=True):
        lpr, eb = lanes_per_row(feat_dim, bf16), 2 if bf16 else 4
        # one row per wavefront covers widths from 81 floats up: rows of 1024 bytes and more are their own class
        rb = (1024 if feat_dim * eb >= 1024 else 512) if (lpr == 64 and eb == 4) else 0
        key = (lpr, eb, rb)
        lay = self._by_lpr.get(key)
        if lay is None:
            rec = self._replay.get(key)
            if rec is not None and self._nargs >= 3 and self._kw:
                lay = self._make(key, hub_split=rec["cut"], segment=rec["segment"])
                lay.set_tuning(**rec["tuning"])
                self.chosen[key] = dict(rec, replayed=True)
            else:
                lay = self._make(key)
                if self.autotune and self._nargs >= 3 and self._kw:
                    lay = self._autotune(key, lay, int(feat_dim), bool(bf16), bool(normalized))
            self._by_lpr[key] = lay
        return lay

    def choices(self):
        """The decisions taken by timing (or replayed) so far, in a form that JSON can carry: {"lanes,elem bytes,row
        class": {"cut", "segment", "tuning"}}.  Pass it as `choices=` to a family of the same plan to get the same
        layouts without timing."""
        return {",".join(str(p) for p in k): {"cut": int(v["cut"]), "segment": int(v["segment"]),
                                             "tuning": {n: int(x) for n, x in v["tuning"].items()}}
                for k, v in self.chosen.items()}

    def _autotune(self, key, first, feat, bf16, normalized):
        import torch

        if not torch.cuda.is_available():
            return first
        n = first.num_nodes
        mult = 8 if bf16 else 4
        ld = -(-feat // mult) * mult
        x = torch.randn((n, ld), device="cuda").to(torch.bfloat16 if bf16 else torch.float32)[:, :feat]
        out = torch.empty((n, feat), dtype=torch.float32, device="cuda")
        st = first.stats()
        rule = (st["hub_split"], st["segment"])
        cands = {rule: first}
        # other cuts can only matter when some row is long enough to be cut by one of them
        if st["hub_segments"] or st["longest_row_task"] > min(c for c, _ in CUT_CANDIDATES[key[1]]):
            for cut, seg in CUT_CANDIDATES[key[1]]:
                if (cut, seg) not in cands:
                    cands[(cut, seg)] = self._make(key, hub_split=cut, segment=seg)
        if normalized:
            deg = torch.ones(n, dtype=torch.float32, device="cuda")
            for lay in cands.values():
                lay.set_degrees(deg)
        for lay in cands.values():
            lay.aggregate(x, normalized=normalized, out=out, feat_dim=feat)
        ms = {k: [] for k in cands}
        for _ in range(2):
            for k, lay in cands.items():
                ms[k].append(lay.aggregate_timed(x, 3, normalized=normalized, out=out, feat_dim=feat)[0])
        ms = {k: min(v) for k, v in ms.items()}
        best = min(ms, key=ms.get)
        if ms[best] > 0.99 * ms[rule]:      # the rule's choice unless a candidate is measurably faster
            best = rule
        for k, lay in cands.items():
            if k != best:
                lay.close()
        lay = cands[best]
        tuning = lay.calibrate(x, normalized=normalized, out=out, feat_dim=feat)
        lay._deg_key = None                  # the degrees used for timing were placeholders
        self.chosen[key] = {"cut": best[0], "segment": best[1], "rule": rule, "ms": {f"{c}/{s}": v for (c, s), v in ms.items()},
                            "tuning": tuning}
        return lay

    def close(self):
        for lay in self._by_lpr.values():
            lay.close()
        self._by_lpr.clear()


class Layout:
    """Owns one rof_layout.  Build with from_v2 / from_v1 / from_parts (host numpy int32 arrays)."""

    def __init__(self, handle, num_nodes):
        self._h = handle
        self.num_nodes = int(num_nodes)
        self._deg_key = None
        self._workspace = None
        self._uploaded = False               # the library's upload is idempotent; this saves the call on every launch
        self._ws_bytes = {}                  # feat_dim -> bytes of partial-sum rows (fixed once the layout is built)

    # ---- construction -------------------------------------------------------------------
    @classmethod
    def from_v2(cls, uniqpart_column_index, uniqpart_pointers, part2Node_ptr, part2Node_col, num_nodes, part_size,
                **opts):
        uc, up, dp, dc = i32(uniqpart_column_index), i32(uniqpart_pointers), i32(part2Node_ptr), i32(part2Node_col)
        if len(up) < 1 or len(up) != len(dp):
            raise ValueError("uniqpart_pointers and part2Node_ptr must both have one entry per unique part plus one")
        h = C.c_void_p()
        o = _opts(**opts)
        check(_lib.lib().rof_layout_from_v2(ptr(uc), up.ctypes.data, dp.ctypes.data, ptr(dc), len(up) - 1,
                                            int(num_nodes), int(part_size), C.byref(o), C.byref(h)))
        return cls(h, num_nodes)

    @classmethod
    def from_v1(cls, column_index, part_pointers, part2Node, part_cache_flagindex, part_pointers_cache,
                column_index_cache, num_nodes, part_size, **opts):
        col, pp, p2n = i32(column_index), i32(part_pointers), i32(part2Node)
        fl, cp, cc = i32(part_cache_flagindex), i32(part_pointers_cache), i32(column_index_cache)
        if len(pp) != len(p2n) + 1 or len(fl) != len(p2n) or len(cp) < 1:
            raise ValueError("inconsistent v1 plan array lengths")
        h = C.c_void_p()
        o = _opts(**opts)
        check(_lib.lib().rof_layout_from_v1(ptr(col), pp.ctypes.data, ptr(p2n), len(p2n), ptr(fl), cp.ctypes.data,
                                            ptr(cc), len(cp) - 1, int(num_nodes), int(part_size), C.byref(o),
                                            C.byref(h)))
        return cls(h, num_nodes)

    @classmethod
    def from_parts(cls, column_index, part_pointers, part2Node, num_nodes, part_size, **opts):
        col, pp, p2n = i32(column_index), i32(part_pointers), i32(part2Node)
        if len(pp) != len(p2n) + 1:
            raise ValueError("part_pointers must have one entry per part plus one")
        h = C.c_void_p()
        o = _opts(**opts)
        check(_lib.lib().rof_layout_from_parts(ptr(col), pp.ctypes.data, ptr(p2n), len(p2n), int(num_nodes),
                                               int(part_size), C.byref(o), C.byref(h)))
        return cls(h, num_nodes)

    @classmethod
    def from_csr(cls, indptr, indices, part_size=1 << 30, **opts):
        """No reuse: every row of a destination-centric CSR is one part."""
        ip = i32(indptr)
        n = len(ip) - 1
        return cls.from_parts(indices, ip, np.arange(n, dtype=np.int32), n, min(int(part_size), 1 << 30), **opts)

    # ---- host-side inspection ------------------------------------------------------------
    def export(self):
        h = C.c_void_p()
        check(_lib.lib().rof_layout_export(self._h, C.byref(h)))
        r = bag_take(h, EXPORT_NAMES, dtype=np.int32)
        r["canonical"] = bool(r["canonical"][0])
        r["xcd_run"] = int(r["xcd_run"][0])
        r["hub_split"], r["segment"] = (int(v) for v in r.pop("long_row_cut"))
        r["b_shape"] = dict(zip(("n_wave", "n_regular", "lg_blocks", "lg_max_rows"),
                                (int(v) for v in r["b_shape"])))
        return r

    def stats(self):
        s = (C.c_int64 * len(STAT_NAMES))()
        check(_lib.lib().rof_layout_stats_n(self._h, s, len(STAT_NAMES)))
        return {k: int(s[i]) for i, k in enumerate(STAT_NAMES)}

    def set_tuning(self, xcd_run_partial=0, xcd_run_dst=0, wave_cap=-1, lds_pad=0, deep=-1):
        """Launch tuning of this layout (rof_layout_set_tuning in include/rof_bench.h); the defaults are the
        library's own choices."""
        t = _lib.LaunchTuning(int(xcd_run_partial), int(xcd_run_dst), int(wave_cap), int(lds_pad), int(deep))
        check(_lib.lib().rof_layout_set_tuning(self._h, C.byref(t)))
        return self

    def tuning(self):
        t = _lib.LaunchTuning()
        check(_lib.lib().rof_layout_get_tuning(self._h, C.byref(t)))
        return {"xcd_run_partial": t.xcd_run_partial, "xcd_run_dst": t.xcd_run_dst, "wave_cap": t.wave_cap,
                "lds_pad": t.lds_pad, "deep": t.deep}

    def algorithmic_bytes(self, feat_dim, in_bytes=4):
        """Bytes one aggregation must move at least once per use, as counted for the roofline:
        every gathered row with its 4-byte column id, every partial-sum row read (fp32) and written,
        and per node one output row plus row pointer and norm."""
        s = self.stats()
        return (s["gathered_rows"] * (4 + feat_dim * in_bytes) + s["partial_reads"] * (4 + feat_dim * 4)
                + s["partial_rows"] * feat_dim * 4 + s["nodes"] * (feat_dim * 4 + 8) + 4 * (s["partial_rows"] + 1))

    # ---- device side ---------------------------------------------------------------------
    def upload(self, stream=0):
        if not self._uploaded:
            check(_lib.lib().rof_layout_upload(self._h, C.c_void_p(stream)))
            self._uploaded = True
        return self

    def set_degrees(self, degrees, stream=None):
        """degrees: float32 CUDA tensor [num_nodes] (the in-degree vector of ROF_main.py:138,144)."""
        import torch

        if degrees.dtype != torch.float32 or not degrees.is_cuda or not degrees.is_contiguous():
            raise RofError("degrees must be a contiguous float32 CUDA tensor")
        if degrees.numel() != self.num_nodes:
            raise RofError("degrees must have one entry per node")
        key = (degrees.data_ptr(), degrees._version)
        if key == self._deg_key:
            return self
        st = torch.cuda.current_stream().cuda_stream if stream is None else stream
        self.upload(st)
        check(_lib.lib().rof_layout_set_degrees(self._h, C.c_void_p(degrees.data_ptr()), C.c_void_p(st)))
        self._deg_key = key
        self._deg_ref = degrees   # keep the pointer's owner alive while it is the cache key
        return self

    def workspace_bytes(self, feat_dim):
        f = int(feat_dim)
        need = self._ws_bytes.get(f)
        if need is None:
            need = self._ws_bytes[f] = int(_lib.lib().rof_layout_workspace_bytes(self._h, f))
        return need

    def _args(self, x, out, feat_dim, workspace, out_dtype=None):
        import torch

        if not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
            raise RofError("x must be a 2-D CUDA tensor with unit column stride")
        if x.shape[0] < self.num_nodes:
            raise RofError("x must have one row per node")
        if x.dtype == torch.float32:
            dt = ROF_F32
        elif x.dtype == torch.bfloat16:
            dt = ROF_BF16
        else:
            raise RofError("x must be float32 or bfloat16")
        f = x.shape[1] if feat_dim is None else int(feat_dim)
        if out is None:
            out = torch.empty((self.num_nodes, f), dtype=out_dtype or torch.float32, device=x.device)
        if (out.dtype != (out_dtype or torch.float32) or not out.is_cuda or out.dim() != 2 or out.stride(1) != 1):
            raise RofError("out must be a 2-D CUDA tensor of the requested dtype (float32 unless out_dtype says "
                           "bfloat16) with unit column stride")
        if out.shape[0] < self.num_nodes or out.shape[1] < f:
            raise RofError("out is too small")
        need = self.workspace_bytes(f)
        if workspace is None:
            if self._workspace is None or self._workspace.numel() * 4 < need or self._workspace.device != x.device:
                self._workspace = torch.empty(max(1, (need + 3) // 4), dtype=torch.float32, device=x.device)
            workspace = self._workspace
        return dt, f, out, workspace

    def aggregate(self, x, normalized=True, out=None, feat_dim=None, workspace=None, bias=None, relu=False,
                  out_dtype=None, self_weight=0.0, pad_columns=False):
        """out[v] = act(s(v) * sum_u w(u) x[u] + self_weight * x[v] + bias) through the plan; x may be a
        column-padded view.  bias (float32 [feat_dim] on the device), the node's own row and relu are applied as
        each output row is stored; out_dtype=torch.bfloat16 stores the fp32 sums rounded to bf16.
        pad_columns=True: x is a view into rows that are allocated up to the next multiple of 4 columns (8 for
        bfloat16) and the kernel may work on whole 16-byte pieces; an output allocated here then has rows of that
        width and the first feat_dim columns are returned as a view (see rof_epilogue in include/rof.h)."""
        import torch

        if out_dtype not in (None, torch.float32, torch.bfloat16):
            raise RofError("out_dtype must be float32 or bfloat16")
        pad = 0
        if pad_columns:
            f0 = x.shape[1] if feat_dim is None else int(feat_dim)
            wide = 8 if x.dtype == torch.bfloat16 else 4
            padded = -(-f0 // wide) * wide
            if padded != f0 and f0 >= wide and x.stride(0) >= padded:
                pad = padded
                if out is None:
                    out = torch.empty((self.num_nodes, padded), dtype=out_dtype or torch.float32,
                                      device=x.device)[:, :f0]
                if out.stride(0) < padded:
                    raise RofError("pad_columns needs output rows allocated up to the padded width")
                if bias is not None:
                    bias = torch.cat([bias, bias.new_zeros(padded - f0)])
        dt, f, out, workspace = self._args(x, out, feat_dim, workspace, out_dtype)
        st = torch.cuda.current_stream().cuda_stream
        self.upload(st)
        if bias is not None:
            if (bias.dtype != torch.float32 or bias.device != x.device or bias.dim() != 1
                    or bias.numel() != (pad or f) or not bias.is_contiguous()):
                raise ValueError("bias must be a contiguous float32 vector of feat_dim elements on the device of x")
        if bias is None and not relu and out.dtype == torch.float32 and not self_weight and not pad:
            ep = None                        # the plain aggregation: no epilogue struct to build
        else:
            ep = C.byref(_lib.Epilogue(bias.data_ptr() if bias is not None else None, int(bool(relu)),
                                       ROF_BF16 if out.dtype == torch.bfloat16 else ROF_F32, float(self_weight),
                                       int(bool(pad))))
        check(_lib.lib().rof_aggregate_epilogue(
            self._h, C.c_void_p(x.data_ptr()), dt, x.stride(0), C.c_void_p(out.data_ptr()), out.stride(0), f,
            int(bool(normalized)), ep, C.c_void_p(workspace.data_ptr()),
            workspace.numel() * workspace.element_size(), C.c_void_p(st)))
        return out

    def aggregate_noalloc(self, x, out, normalized=True, feat_dim=None, bias=None, relu=False, self_weight=0.0):
        """`aggregate` into a caller-provided `out` through rof_aggregate_noalloc: the partial-sum rows live in the
        library's static device array (NOALLOC_WORKSPACE_BYTES per GPU), and neither the library nor this wrapper
        allocates device memory.  Raises when the layout needs more than that, or was not uploaded yet (uploading
        allocates).  Calls that overlap on one GPU share the array and must be serialised by the caller."""
        import torch

        if out is None:
            raise RofError("aggregate_noalloc needs an output tensor: it allocates nothing")
        dt, f, out, _ = self._args(x, out, feat_dim, out, out.dtype)   # no workspace tensor is created
        if bias is not None and (bias.dtype != torch.float32 or bias.device != x.device or bias.dim() != 1
                                 or bias.numel() != f or not bias.is_contiguous()):
            raise ValueError("bias must be a contiguous float32 vector of feat_dim elements on the device of x")
        ep = _lib.Epilogue(bias.data_ptr() if bias is not None else None, int(bool(relu)),
                           ROF_BF16 if out.dtype == torch.bfloat16 else ROF_F32, float(self_weight), 0)
        L = _lib.lib()
        rc = L.rof_aggregate_noalloc(self._h, C.c_void_p(x.data_ptr()), dt, x.stride(0), C.c_void_p(out.data_ptr()),
                                     out.stride(0), f, int(bool(normalized)), C.byref(ep),
                                     C.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc == -7:
            raise RofError("librof: " + L.rof_last_device_error().decode() + " (status -7)")
        check(rc)
        return out

    def _plain_epilogue(self, x, out, f, pad_columns):
        """Epilogue argument of the timing helpers: none, or just the permission to work on whole vectors."""
        import torch

        if not pad_columns:
            return None
        wide = 8 if x.dtype == torch.bfloat16 else 4
        padded = -(-f // wide) * wide
        if x.stride(0) < padded or out.stride(0) < padded:
            raise RofError("pad_columns needs input and output rows allocated up to the padded width")
        return C.byref(_lib.Epilogue(None, 0, ROF_F32, 0.0, 1))

    def aggregate_timed(self, x, iters, normalized=True, out=None, feat_dim=None, workspace=None, pad_columns=False):
        """Mean milliseconds per aggregation over `iters` back-to-back calls, measured with HIP events
        recorded on the stream the kernels run on."""
        import torch

        dt, f, out, workspace = self._args(x, out, feat_dim, workspace)
        st = torch.cuda.current_stream().cuda_stream
        self.upload(st)
        ms = C.c_float()
        check(_lib.lib().rof_aggregate_timed(self._h, C.c_void_p(x.data_ptr()), dt, x.stride(0),
                                             C.c_void_p(out.data_ptr()), out.stride(0), f, int(bool(normalized)),
                                             self._plain_epilogue(x, out, f, pad_columns),
                                             C.c_void_p(workspace.data_ptr()),
                                             workspace.numel() * workspace.element_size(), C.c_void_p(st), int(iters),
                                             C.byref(ms)))
        return float(ms.value), out

    def calibrate(self, x, normalized=True, out=None, feat_dim=None, workspace=None, pad_columns=False, rounds=3, iters=3):
        """Choose this layout's launch settings (wavefront cap, gathers in flight, XCD run) by timing the aggregation
        on these operands (rof_layout_calibrate); returns the settings now in force."""
        import torch

        dt, f, out, workspace = self._args(x, out, feat_dim, workspace)
        st = torch.cuda.current_stream().cuda_stream
        self.upload(st)
        t = _lib.LaunchTuning()
        check(_lib.lib().rof_layout_calibrate(self._h, C.c_void_p(x.data_ptr()), dt, x.stride(0),
                                              C.c_void_p(out.data_ptr()), out.stride(0), f, int(bool(normalized)),
                                              self._plain_epilogue(x, out, f, pad_columns),
                                              C.c_void_p(workspace.data_ptr()),
                                              workspace.numel() * workspace.element_size(), C.c_void_p(st),
                                              int(rounds), int(iters), C.byref(t)))
        return self.tuning()

    def launch_times(self, x, iters, normalized=True, out=None, feat_dim=None, workspace=None, pad_columns=False):
        """(ms of the partial-sum launch, ms of the destination-row launch), HIP-event means over `iters`."""
        import torch

        dt, f, out, workspace = self._args(x, out, feat_dim, workspace)
        st = torch.cuda.current_stream().cuda_stream
        self.upload(st)
        ms = (C.c_float * 2)()
        check(_lib.lib().rof_aggregate_launch_times(self._h, C.c_void_p(x.data_ptr()), dt, x.stride(0),
                                                    C.c_void_p(out.data_ptr()), out.stride(0), f,
                                                    int(bool(normalized)), self._plain_epilogue(x, out, f, pad_columns),
                                                    C.c_void_p(workspace.data_ptr()),
                                                    workspace.numel() * workspace.element_size(), C.c_void_p(st),
                                                    int(iters), C.byref(ms)))
        return float(ms[0]), float(ms[1])

    def launch_bytes(self, feat_dim, in_bytes=4):
        """Algorithmic bytes of (launch 1, launch 2): the split of `algorithmic_bytes`."""
        s = self.stats()
        a = s["gathered_rows_a"] * (4 + feat_dim * in_bytes) + s["partial_rows"] * feat_dim * 4 + 4 * (s["partial_rows"] + 1)
        return a, self.algorithmic_bytes(feat_dim, in_bytes) - a

    def close(self):
        if self._h is not None:
            _lib.lib().rof_layout_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
