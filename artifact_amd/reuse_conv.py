"""Layer API of the reuse-aware GCN convolution: drop-in for ROF/reuse_conv/reuse_conv.py.

`ROF_GCNConvFunc` and `ROF_GCNConv` keep the upstream names, argument meaning, parameter set,
initialisers and error behaviour (reuse_conv.py:30-150); `ROF_inputInfo` restates the plan container
whose class is missing from the upstream tree but whose contract is fixed by its call sites
(ROF_evaluation/ROF_main.py:164-178, reuse_conv.py:34-37,145-146).  `ROF_GINConv` is the sum-aggregation
layer the GIN workload needs; upstream has only its kernel (ROF.SAG, reuse_conv_kernel.cu:123-196).
"""
from __future__ import annotations

import json
import math

import numpy as np
import torch

from . import ROF
from . import reuse_search_ext
from .layout import Layout, LayoutFamily, column_sums

__all__ = ["ROF_GCNConvFunc", "ROF_GCNLayerFunc", "ROF_GCNConv", "ROF_GINConv", "ROF_inputInfo", "build_input_info"]

_TENSOR_FIELDS = ("row_pointers", "column_index", "degrees", "part_pointers", "part2Node", "part_cache_flagindex",
                  "part_pointers_cache", "column_index_cache", "uniqpart_column_index", "uniqpart_pointers",
                  "part2Node_ptr", "part2Node_col")


class ROF_inputInfo:
    """Plan container: positional constructor of ROF_main.py:164-174, attributes of the same names,
    `dimWorker` / `part_result_cache` set later by the layer (reuse_conv.py:145-146), in-place `.to`."""

    def __init__(self, row_pointers, column_index, degrees, part_pointers, part2Node, partSize, warpPerBlock,
                 part_cache_flagindex, part_pointers_cache, column_index_cache, uniqpart_column_index,
                 uniqpart_pointers, part2Node_ptr, part2Node_col):
        self.row_pointers = row_pointers
        self.column_index = column_index
        self.degrees = degrees
        self.part_pointers = part_pointers
        self.part2Node = part2Node
        self.partSize = partSize
        self.warpPerBlock = warpPerBlock
        self.part_cache_flagindex = part_cache_flagindex
        self.part_pointers_cache = part_pointers_cache
        self.column_index_cache = column_index_cache
        self.uniqpart_column_index = uniqpart_column_index
        self.uniqpart_pointers = uniqpart_pointers
        self.part2Node_ptr = part2Node_ptr
        self.part2Node_col = part2Node_col
        self.dimWorker = 0
        self.part_result_cache = None
        self.layouts = {}   # kernel_type -> LayoutFamily built from host arrays (skips the device->host round trip)

    def to(self, device):
        for name in _TENSOR_FIELDS:
            t = getattr(self, name)
            if isinstance(t, torch.Tensor):
                setattr(self, name, t.to(device))
        if isinstance(self.part_result_cache, torch.Tensor):
            self.part_result_cache = self.part_result_cache.to(device)
        return self

    @property
    def reuse_size(self):
        return int(self.part_pointers_cache.shape[0]) - 1

    # ---- on-disk form of the (expensive) plan; upstream caches the whole object with torch.save
    # (ROF_evaluation/cuda/middle-main.py:440-452), which also works; this form is plain numpy
    def save(self, path):
        """Write every plan tensor plus the two scalars to an .npz file -- and, as a JSON string, what an autotuning
        layout family has chosen by timing so far (cut of long rows and launch settings per width class), so that a
        later run takes the same layouts without timing and sums in the same order."""
        arrays = {name: getattr(self, name).detach().cpu().numpy() for name in _TENSOR_FIELDS}
        fam = self.layouts.get("ROF_v2")
        choices = json.dumps(fam.choices() if fam is not None else {})
        np.savez(path, partSize=np.int64(self.partSize), warpPerBlock=np.int64(self.warpPerBlock),
                 layout_choices=np.array(choices), **arrays)

    @classmethod
    def load(cls, path, device="cuda", autotune=None, **layout_opts):
        """Inverse of save(); rebuilds the device layout from the stored v2 arrays without a plan search.  Width
        classes whose layout was chosen by timing before the save are rebuilt as chosen; `autotune` applies to the
        others."""
        z = np.load(path if str(path).endswith(".npz") else str(path) + ".npz")
        t = {name: torch.from_numpy(z[name]).to(device) for name in _TENSOR_FIELDS}
        info = cls(t["row_pointers"], t["column_index"], t["degrees"], t["part_pointers"], t["part2Node"],
                   int(z["partSize"]), int(z["warpPerBlock"]), t["part_cache_flagindex"], t["part_pointers_cache"],
                   t["column_index_cache"], t["uniqpart_column_index"], t["uniqpart_pointers"], t["part2Node_ptr"],
                   t["part2Node_col"])
        if torch.device(device).type == "cuda":
            n, ps = len(z["row_pointers"]) - 1, int(z["partSize"])
            v2 = tuple(np.array(z[k]) for k in ("uniqpart_column_index", "uniqpart_pointers", "part2Node_ptr",
                                                 "part2Node_col"))
            choices = json.loads(str(z["layout_choices"])) if "layout_choices" in z.files else {}
            info.layouts["ROF_v2"] = LayoutFamily(lambda lpr, eb, rb=0, **kw: Layout.from_v2(
                *v2, n, ps, lanes_per_row=lpr, elem_bytes=eb, row_bytes=rb, **{**layout_opts, **kw}),
                autotune=autotune, choices=choices)
        return info

    def __getstate__(self):
        d = dict(self.__dict__)
        d["layouts"] = {}   # device handles are rebuilt on demand
        return d

    def __repr__(self):
        shapes = ", ".join(f"{n}={tuple(getattr(self, n).shape)}" for n in _TENSOR_FIELDS
                           if isinstance(getattr(self, n), torch.Tensor))
        return f"ROF_inputInfo(partSize={self.partSize}, warpPerBlock={self.warpPerBlock}, {shapes})"


def build_input_info(indptr, indices, part_size=3, device="cuda", warps_per_block=4, plan=None, search="upstream",
                     hubs=16384, autotune=None, **layout_opts):
    """CSR (symmetric graph, in-neighbours = out-neighbours) -> ROF_inputInfo, following the glue of
    ROF_main.py:71-178: plan on the CPU, arrays cast to int32, degrees = diff(indptr) as float32.
    `layout_opts` (min_consumers, disable_reuse, hub_split, segment) go to the device layout; `autotune=True` lets
    the layout family choose the cut of long rows and the launch settings of every width class by timing candidates
    on the GPU at first use (LayoutFamily; None: the environment variable ROF_AUTOTUNE).
    search="hub_patterns" (not upstream) fills the v2 tensors from reuse_search_ext.hub_pattern_plan with
    `hubs` hubs in blocks of `part_size`, search="dynamic_greedy" from reuse_search_ext.dynamic_greedy_plan; the
    GNNA / v1 tensors then describe the graph without reuse."""
    indptr = np.asarray(indptr)
    indices = np.asarray(indices)
    if search not in ("upstream", "hub_patterns", "dynamic_greedy"):
        raise ValueError("search must be 'upstream', 'hub_patterns' or 'dynamic_greedy'")
    if plan is None and search != "upstream":
        plan = (reuse_search_ext.hub_pattern_plan(indptr, indices, hubs, part_size) if search == "hub_patterns"
                else reuse_search_ext.dynamic_greedy_plan(indptr, indices, part_size))
        empty = np.zeros(0, np.uint32)
        ptr, p2n, _ = reuse_search_ext.py_split_part(empty, empty, indptr, part_size)
        plan.update(new_indices_src=np.asarray(indices), part_ptr=ptr, part2Node=p2n,
                    part_cache_flagindex=np.zeros(len(p2n), np.uint32), part_pointers_cache=np.zeros(1, np.uint32),
                    column_index_cache=np.zeros(0, np.uint32))
    elif plan is None:
        plan = reuse_search_ext.build_plan(indptr, indices, part_size)
    n = len(indptr) - 1

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(np.asarray(a).astype(np.int32))).to(device)

    degree_in = np.diff(indptr.astype(np.int64)).astype(np.float32)
    info = ROF_inputInfo(t(indptr), t(plan["new_indices_src"]), torch.from_numpy(degree_in).to(device),
                         t(plan["part_ptr"]), t(plan["part2Node"]), int(part_size), int(warps_per_block),
                         t(plan["part_cache_flagindex"]), t(plan["part_pointers_cache"]),
                         t(plan["column_index_cache"]), t(plan["uniqpart_column_index"]), t(plan["uniqpart_pointers"]),
                         t(plan["part2Node_ptr"]), t(plan["part2Node_col"]))
    if torch.device(device).type == "cuda":
        info.layouts["ROF_v2"] = LayoutFamily(lambda lpr, eb, rb=0, **kw: Layout.from_v2(
            plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"], plan["part2Node_col"], n,
            part_size, lanes_per_row=lpr, elem_bytes=eb, row_bytes=rb, **{**layout_opts, **kw}), autotune=autotune)
    info.plan = plan
    return info


def _layout_arg(layout):
    """The prebuilt layout of a plan container as a keyword argument, when there is one: upstream's signature has no
    such argument, and an operator module without it (the compiled one) re-lays the plan tensors out itself."""
    return {} if layout is None else {"layout": layout}


class ROF_GCNConvFunc(torch.autograd.Function):
    """reuse_conv.py:30-92: dispatch on kernel_type, same plan forward and backward, five gradients."""

    @staticmethod
    def forward(ctx, x, weight, inputInfo, add_self_loops=False, kernel_type="ROF_v1"):
        ii = inputInfo
        ctx.save_for_backward(x, weight, ii.column_index, ii.degrees, ii.part_pointers, ii.part2Node,
                              ii.part_result_cache, ii.part_cache_flagindex, ii.part_pointers_cache,
                              ii.column_index_cache, ii.uniqpart_column_index, ii.uniqpart_pointers, ii.part2Node_ptr,
                              ii.part2Node_col)
        ctx.partSize = ii.partSize
        ctx.dimWorker = ii.dimWorker
        ctx.warpPerBlock = ii.warpPerBlock
        ctx.kernel_type = kernel_type
        ctx.layout = getattr(ii, "layouts", {}).get(kernel_type)
        if add_self_loops:
            raise NotImplementedError   # reuse_conv.py:72-73
        if kernel_type == "GNNA":
            return ROF.GNNA_forward(x, weight, ii.column_index, ii.degrees, ii.part_pointers, ii.part2Node,
                                    ii.partSize, ii.dimWorker, ii.warpPerBlock)[0]
        if kernel_type == "ROF_v1":
            return ROF.reuse_forward_v1(x, weight, ii.column_index, ii.degrees, ii.part_pointers, ii.part2Node,
                                        ii.partSize, ii.dimWorker, ii.warpPerBlock, ii.part_result_cache,
                                        ii.part_cache_flagindex, ii.part_pointers_cache, ii.column_index_cache)[0]
        if kernel_type == "ROF_v2":
            return ROF.reuse_forward_v2(x, weight, ii.uniqpart_column_index, ii.degrees, ii.uniqpart_pointers,
                                        ii.part2Node_ptr, ii.part2Node_col, ii.partSize, ii.dimWorker,
                                        ii.warpPerBlock, **_layout_arg(ctx.layout))[0]
        raise NotImplementedError

    @staticmethod
    def backward(ctx, grad_output):
        (x, weight, column_index, degrees, part_pointers, part2Node, part_result_cache, part_cache_flagindex,
         part_pointers_cache, column_index_cache) = ctx.saved_tensors[:-4]
        uniqpart_column_index, uniqpart_pointers, part2Node_ptr, part2Node_col = ctx.saved_tensors[-4:]
        ps, dw, wpb = ctx.partSize, ctx.dimWorker, ctx.warpPerBlock
        grad_output = grad_output.contiguous()
        if ctx.kernel_type == "GNNA":
            d_input, d_weight = ROF.GNNA_backward(grad_output, x, weight, column_index, degrees, part_pointers,
                                                  part2Node, ps, dw, wpb)
        elif ctx.kernel_type == "ROF_v1":
            d_input, d_weight = ROF.reuse_backward_v1(grad_output, x, weight, column_index, degrees, part_pointers,
                                                      part2Node, ps, dw, wpb, part_result_cache, part_cache_flagindex,
                                                      part_pointers_cache, column_index_cache)
        elif ctx.kernel_type == "ROF_v2":
            d_input, d_weight = ROF.reuse_backward_v2(grad_output, x, weight, uniqpart_column_index, degrees,
                                                      uniqpart_pointers, part2Node_ptr, part2Node_col, ps, dw, wpb,
                                                      **_layout_arg(ctx.layout))
        else:
            raise NotImplementedError
        return d_input, d_weight, None, None, None


def _family(ii, kernel_type, num_nodes):
    """LayoutFamily for a plan container: the one built with it, else from its device tensors."""
    fam = getattr(ii, "layouts", {}).get(kernel_type)
    if fam is not None:
        return fam
    if kernel_type == "GNNA":
        return ROF._layout_parts(ii.column_index, ii.part_pointers, ii.part2Node, num_nodes, ii.partSize)
    if kernel_type == "ROF_v1":
        return ROF._layout_v1(ii.column_index, ii.part_pointers, ii.part2Node, ii.part_cache_flagindex,
                              ii.part_pointers_cache, ii.column_index_cache, num_nodes, ii.partSize)
    if kernel_type == "ROF_v2":
        return ROF._layout_v2(ii.uniqpart_column_index, ii.uniqpart_pointers, ii.part2Node_ptr, ii.part2Node_col,
                              num_nodes, ii.partSize)
    raise NotImplementedError


def _bf16_rows(t):
    """`t` as bfloat16 rows that start on 16-byte boundaries (row stride a multiple of 8 elements), so that the
    kernels gather them with 16-byte loads; one pass at most (the cast writes straight into the padded buffer)."""
    if t.dtype == torch.bfloat16 and t.stride(1) == 1 and t.stride(0) % 8 == 0:
        return t
    f = t.shape[1]
    buf = torch.empty((t.shape[0], f + (-f) % 8), dtype=torch.bfloat16, device=t.device)
    view = buf[:, :f]
    view.copy_(t)
    return view


class ROF_GCNLayerFunc(torch.autograd.Function):
    """Whole GCN layer  act(A_hat (x W) + b)  as one autograd node (not upstream, which runs the bias and the
    activation as separate passes over the output: reuse_conv.py:147-150, ROF_main.py:181).

    update-first (upstream's order, reuse_conv_kernel.cu:971-1000): bias and ReLU are applied by the
    aggregation kernel as it stores each output row.  aggregate-first evaluates (A_hat x) W instead, which
    gathers rows of width in_channels; it is the cheaper order when in_channels < out_channels.  Both orders
    give the same layer up to fp32 re-association.  Backward: with g = grad * (out > 0),
    update-first  dT = A_hat g, dX = dT W^T, dW = x^T dT;  aggregate-first  dW = (A_hat x)^T g, dX = A_hat (g W^T);
    db = column sums of g.  A_hat is symmetric, as upstream assumes (reuse_conv_kernel.cu:1021-1041).

    bf16=True is the mixed-precision form: every gathered row and every GEMM operand is bfloat16 (x may already
    be), every neighbour sum is accumulated in fp32, parameters and their gradients stay fp32.  out_bf16 makes
    the layer's output bfloat16 as well (rounded once, in the aggregation store), which is what the next such
    layer consumes."""

    @staticmethod
    def forward(ctx, x, weight, bias, inputInfo, kernel_type, relu, aggregate_first, bf16=False, out_bf16=False):
        ROF._check(input=x, weight=weight)
        fam = _family(inputInfo, kernel_type, x.shape[0])
        deg = inputInfo.degrees
        ctx.fam, ctx.deg, ctx.relu, ctx.aggregate_first, ctx.bf16 = fam, deg, bool(relu), bool(aggregate_first), bool(bf16)
        ctx.has_bias = bias is not None
        ctx.x_dtype = x.dtype
        b = None if bias is None else bias.detach().contiguous()
        half = torch.bfloat16
        odt = half if (bf16 and out_bf16) else torch.float32
        if bf16:
            x = _bf16_rows(x)
            wb = weight.detach().to(half)
        elif x.dtype != torch.float32:
            raise RuntimeError("input must be float32 (or bfloat16 with compute_dtype='bf16')")
        if aggregate_first:
            f = x.shape[1]
            lay = fam.get(f, bf16)
            lay.set_degrees(deg)
            h = lay.aggregate(x, normalized=True, feat_dim=f, out_dtype=half if bf16 else None)
            if bf16:
                out = torch.mm(h, wb)
                out = out.to(odt) if b is None else (out.float() + b).to(odt)
            else:
                out = torch.mm(h, weight) if b is None else torch.addmm(b, h, weight)
            if relu:
                out.relu_()
            ctx.save_for_backward(h, weight, out if relu else None)
        else:
            if bf16:
                f = weight.shape[1]
                pad = (-f) % 8                        # rows of the update are gathered 8 bf16 at a time
                tmp = torch.mm(x, wb if pad == 0 else torch.cat([wb, wb.new_zeros(wb.shape[0], pad)], dim=1))
            else:
                tmp, f = ROF._update(x, weight)
            lay = fam.get(f, bf16)
            lay.set_degrees(deg)
            out = lay.aggregate(tmp, normalized=True, feat_dim=f, bias=b, relu=relu, out_dtype=odt)
            ctx.save_for_backward(x, weight, out if relu else None)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        saved, weight, out = ctx.saved_tensors
        g = grad_output.contiguous()
        if ctx.relu:
            f = g.shape[1]
            if not ctx.bf16 and f % 4:
                # the masked gradient is a new tensor anyway: give it 16-byte rows, which the backward
                # aggregation gathers ~12 % faster than packed ones
                masked = g.new_empty((g.shape[0], f + (-f) % 4))[:, :f]
                torch.mul(g, out > 0, out=masked)
                g = masked
            else:
                g = g * (out > 0)
        d_bias = column_sums(g) if ctx.has_bias and ctx.needs_input_grad[2] else None
        d_x = d_w = None
        half = torch.bfloat16
        if ctx.bf16:
            g = _bf16_rows(g)
            wb = weight.to(half)
        else:
            wb = weight
        gdt = half if ctx.bf16 else None
        if ctx.aggregate_first:
            if ctx.needs_input_grad[1]:
                d_w = ROF._weight_grad(saved, g)
            if ctx.needs_input_grad[0]:
                dh = torch.mm(g, wb.transpose(0, 1))
                dh = _bf16_rows(dh) if ctx.bf16 else dh
                lay = ctx.fam.get(dh.shape[1], ctx.bf16)
                lay.set_degrees(ctx.deg)
                d_x = lay.aggregate(dh, normalized=True, feat_dim=dh.shape[1], out_dtype=gdt).to(ctx.x_dtype)
        elif ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            lay = ctx.fam.get(g.shape[1], ctx.bf16)
            lay.set_degrees(ctx.deg)
            dt = lay.aggregate(g, normalized=True, feat_dim=g.shape[1], out_dtype=gdt, pad_columns=True)   # internal: rows may keep the padded stride
            if ctx.needs_input_grad[0]:
                d_x = torch.mm(dt, wb.transpose(0, 1)).to(ctx.x_dtype)
            if ctx.needs_input_grad[1]:
                d_w = ROF._weight_grad(saved, dt)
        return d_x, d_w, d_bias, None, None, None, None, None, None


class ROF_GCNConv(torch.nn.Module):
    """reuse_conv.py:96-150.  Note the upstream default add_self_loops=True raises at call time
    (reuse_conv.py:102 with :72-73); pass add_self_loops=False as the upstream drivers do.

    Keyword arguments beyond upstream's (all optional; the defaults reproduce upstream's arithmetic):
      fuse_epilogue (default True)  add the bias inside the aggregation kernel instead of a separate pass
                                    (same bits); False runs upstream's literal sequence
      activation   None | "relu"    also apply ReLU there, so the layer returns relu(A_hat x W + b)
      order  "update_first" (default, upstream) | "aggregate_first" | "auto" (aggregate first when
             in_channels < out_channels)
      compute_dtype  None | "bf16"  gather bfloat16 rows and run the GEMMs on bfloat16 operands; sums are
                                    accumulated in fp32, parameters stay fp32
      out_dtype      None | "bf16"  with compute_dtype="bf16": return bfloat16 (rounded once, as rows are stored)"""

    def __init__(self, in_channels, out_channels, bias=True, **kwargs):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kwargs = kwargs
        self.add_self_loops = kwargs.get("add_self_loops", True)
        self.kernel_type = kwargs.get("kernel_type", "ROF_v1")
        self.weight = torch.nn.Parameter(torch.empty(in_channels, out_channels))
        if bias:
            self.bias = torch.nn.Parameter(torch.empty(out_channels))
        else:
            self.register_parameter("bias", None)
        self.reuse_size = kwargs.get("reuse_size", 0)
        # scratch of the v1 kernels; a plain Parameter upstream (reuse_conv.py:113), so it is one here: it shows
        # up in state_dict() and in parameters() (an optimizer skips it, it never receives a gradient)
        self.part_result_cache = torch.nn.Parameter(torch.empty(max(self.reuse_size, 0), out_channels + 1))
        self.dimWorker = kwargs.get("dimWorker", 0)
        if self.dimWorker == 0:
            self.dimWorker = 32 if out_channels > 32 else out_channels   # reuse_conv.py:115-120
        self.fuse_epilogue = bool(kwargs.get("fuse_epilogue", True))
        self.activation = kwargs.get("activation", None)
        if self.activation not in (None, "relu"):
            raise NotImplementedError("activation must be None or 'relu'")
        order = kwargs.get("order", "update_first")
        if order not in ("update_first", "aggregate_first", "auto"):
            raise ValueError("order must be 'update_first', 'aggregate_first' or 'auto'")
        self.aggregate_first = order == "aggregate_first" or (order == "auto" and in_channels < out_channels)
        self.bf16 = kwargs.get("compute_dtype", None) in ("bf16", torch.bfloat16)
        if kwargs.get("compute_dtype", None) not in (None, "bf16", torch.bfloat16, "fp32", torch.float32):
            raise ValueError("compute_dtype must be None or 'bf16'")
        self.out_bf16 = self.bf16 and kwargs.get("out_dtype", None) in ("bf16", torch.bfloat16)
        if self.kernel_type == "ROF_v1" and not self.bf16 and (self.aggregate_first or "fuse_epilogue" in kwargs):
            # only upstream's literal sequence fills the caller's part_result_cache, so that is what ROF_v1 runs
            import warnings

            warnings.warn("ROF_GCNConv(kernel_type='ROF_v1') always runs upstream's sequence (update, aggregate, "
                          "bias pass): `order` and `fuse_epilogue` have no effect; use kernel_type='ROF_v2' for them")
        self.reset_parameters()

    def reset_parameters(self):
        init = self.kwargs.get("weight_initializer", "glorot")
        if init == "glorot":
            torch.nn.init.xavier_uniform_(self.weight)
        elif init == "uniform":
            bound = 1.0 / math.sqrt(self.in_channels)
            torch.nn.init.uniform_(self.weight.data, -bound, bound)
        elif init == "he":
            bound = math.sqrt(6 / ((1 + 5) * self.in_channels))   # a = sqrt(5): reuse_conv.py:131-136
            self.weight.data.uniform_(-bound, bound)
        else:
            raise NotImplementedError
        if self.bias is not None:
            torch.nn.init.zeros_(self.bias)
        with torch.no_grad():
            self.part_result_cache.zero_()

    def forward(self, x, inputInfo):
        inputInfo.part_result_cache = self.part_result_cache
        inputInfo.dimWorker = self.dimWorker
        plain = (self.activation is None and not self.aggregate_first and not self.bf16
                 and (self.bias is None or not self.fuse_epilogue))
        if plain or (self.kernel_type == "ROF_v1" and not self.bf16):
            # upstream's sequence; the v1 entry points also fill the caller's cache (reuse_conv_kernel.cu:476-485)
            out = ROF_GCNConvFunc.apply(x, self.weight, inputInfo, self.add_self_loops, self.kernel_type)
            out = out if self.bias is None else out + self.bias
            return torch.relu(out) if self.activation == "relu" else out
        if self.add_self_loops:
            raise NotImplementedError   # reuse_conv.py:72-73
        return ROF_GCNLayerFunc.apply(x, self.weight, self.bias, inputInfo, self.kernel_type,
                                      self.activation == "relu", self.aggregate_first, self.bf16, self.out_bf16)


class _SumAggregate(torch.autograd.Function):
    """self_weight * x_v + unnormalised neighbour sum through the reuse plan, the own row added as the sum is
    stored; the backward pass is the same operator on the gradient because the graphs are symmetric (the
    assumption upstream makes for GCN as well)."""

    @staticmethod
    def forward(ctx, x, family, self_weight):
        ctx.family, ctx.self_weight = family, float(self_weight)
        return family.get(x.shape[1]).aggregate(x.contiguous(), normalized=False, feat_dim=x.shape[1],
                                                self_weight=ctx.self_weight)

    @staticmethod
    def backward(ctx, grad):
        g = grad.contiguous()
        return ctx.family.get(g.shape[1]).aggregate(g, normalized=False, feat_dim=g.shape[1],
                                                    self_weight=ctx.self_weight), None, None


class ROF_GINConv(torch.nn.Module):
    """GIN layer: mlp((1 + eps) * x + sum_{u in N(v)} x_u), the sum evaluated through the reuse plan."""

    def __init__(self, in_channels, out_channels, eps=0.0, kernel_type="ROF_v2"):
        super().__init__()
        self.eps = float(eps)
        self.kernel_type = kernel_type
        self.mlp = torch.nn.Linear(in_channels, out_channels)

    def forward(self, x, inputInfo):
        return self.mlp(_SumAggregate.apply(x, _family(inputInfo, self.kernel_type, x.shape[0]), 1.0 + self.eps))
