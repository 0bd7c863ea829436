"""Drop-in for the upstream `ROF` extension module (ROF/reuse_conv/reuse_conv.cpp:353-365).

Same seven functions, positional signatures, dtypes and return shapes.  Each call
  1. checks its tensors the way upstream's CHECK_INPUT does (reuse_conv.cpp:121-123): RuntimeError
     "<name> must be a CUDA tensor" / "<name> must be contiguous";
  2. runs the dense update with torch.mm exactly where upstream does (reuse_conv_kernel.cu:302, 382-383);
  3. runs the aggregation through librof.so's gfx950 kernels on PyTorch's current stream.

The plan tensors are re-laid out into the device layout on first use and cached by their storage
addresses (upstream treats them as immutable and shares them across layers and passes:
reuse_conv.py:40-43).  `partSize` keeps its meaning; `dimWorker` and `warpPerBlock` are tuning
hints of the upstream warp-per-part scheme and are accepted but unused.
"""
from __future__ import annotations

from collections import OrderedDict

import torch

from .layout import Layout, LayoutFamily

__all__ = ["SAG", "GNNA_forward", "GNNA_backward", "reuse_forward_v1", "reuse_backward_v1", "reuse_forward_v2",
           "reuse_backward_v2", "clear_layout_cache"]

_CACHE: "OrderedDict[tuple, LayoutFamily]" = OrderedDict()
_CACHE_MAX = 32


def clear_layout_cache():
    for lay in _CACHE.values():
        lay.close()
    _CACHE.clear()


def _check(**tensors):
    for name, t in tensors.items():
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a CUDA tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")


def _key(kind, part_size, *tensors):
    return (kind, int(part_size)) + tuple((t.data_ptr(), t.numel(), t._version) for t in tensors)


def _cached(key, build, keep):
    lay = _CACHE.get(key)
    if lay is None:
        lay = build()
        lay._keep = keep   # the key holds raw addresses: keep their owners alive
        _CACHE[key] = lay
        while len(_CACHE) > _CACHE_MAX:
            _, old = _CACHE.popitem(last=False)
            old.close()
    else:
        _CACHE.move_to_end(key)
    return lay


def _host(*tensors):
    for t in tensors:
        if t.dtype != torch.int32:
            raise RuntimeError("plan tensors must be int32")
    return [t.detach().cpu().numpy() for t in tensors]


def _layout_parts(column_index, part_pointers, part2Node, num_nodes, part_size):
    key = _key("parts", part_size, column_index, part_pointers, part2Node)

    def build():
        host = _host(column_index, part_pointers, part2Node)
        return LayoutFamily(lambda lpr, eb, rb=0, **kw: Layout.from_parts(*host, num_nodes, part_size, lanes_per_row=lpr,
                                                                          elem_bytes=eb, row_bytes=rb, **kw))

    return _cached(key, build, (column_index, part_pointers, part2Node))


def _layout_v1(column_index, part_pointers, part2Node, flag, cache_ptr, cache_col, num_nodes, part_size):
    key = _key("v1", part_size, column_index, part_pointers, part2Node, flag, cache_ptr, cache_col)

    def build():
        host = _host(column_index, part_pointers, part2Node, flag, cache_ptr, cache_col)
        # every cache row is materialised (min_consumers=-1) so that slot g of the workspace is cache row g
        return LayoutFamily(lambda lpr, eb, rb=0, **kw: Layout.from_v1(*host, num_nodes, part_size, min_consumers=-1,
                                                                       lanes_per_row=lpr, elem_bytes=eb, row_bytes=rb,
                                                                       **kw))

    return _cached(key, build, (column_index, part_pointers, part2Node, flag, cache_ptr, cache_col))


def _layout_v2(ucol, uptr, dptr, dcol, num_nodes, part_size):
    key = _key("v2", part_size, ucol, uptr, dptr, dcol)

    def build():
        host = _host(ucol, uptr, dptr, dcol)
        return LayoutFamily(lambda lpr, eb, rb=0, **kw: Layout.from_v2(*host, num_nodes, part_size, lanes_per_row=lpr,
                                                                       elem_bytes=eb, row_bytes=rb, **kw))

    return _cached(key, build, (ucol, uptr, dptr, dcol))


def _update(x, weight):
    """tmp = x @ weight (reuse_conv_kernel.cu:302), produced with a row stride that is a multiple of
    four floats so rows can be gathered with 16-byte loads.  Returns (buffer, width)."""
    f = weight.shape[1]
    pad = (-f) % 4
    if pad == 0:
        return torch.mm(x, weight), f
    wpad = torch.cat([weight, weight.new_zeros(weight.shape[0], pad)], dim=1)
    return torch.mm(x, wpad), f


def _weight_grad(x, d):
    """x^T @ d in float32 for tall operands ([N, in]^T [N, out], N in the millions): the product has only
    in * out outputs, far too few tiles to fill the GPU, and a single GEMM call runs at a tenth of the memory
    rate (measured 3.85 ms for 2.4 M x 100 x 47).  The rows are cut into slabs of ~4096, every slab is one
    member of a batched GEMM, and the slab products are added in float32 (0.41 ms for the same shape)."""
    n = x.shape[0]
    slabs = min(1024, n // 4096)
    if slabs < 4:
        return torch.mm(x.transpose(0, 1), d).float()
    m = n // slabs
    a = x[: m * slabs].unflatten(0, (slabs, m))
    b = d[: m * slabs].unflatten(0, (slabs, m))
    out = torch.bmm(a.transpose(1, 2), b).sum(0, dtype=torch.float32)
    if m * slabs < n:
        out += torch.mm(x[m * slabs:].transpose(0, 1), d[m * slabs:]).float()
    return out


def _forward(family, x, weight, degrees):
    tmp, f = _update(x, weight)
    layout = family.get(f)
    layout.set_degrees(degrees)
    return layout.aggregate(tmp, normalized=True, feat_dim=f), layout


def _backward(family, d_output, X, W, degrees):
    # upstream aggregates d_output with the same un-transposed plan (reuse_conv_kernel.cu:353-373,
    # 743-808, 1021-1041), then the two GEMMs (cu:382-383)
    f = d_output.shape[1]
    layout = family.get(f)
    layout.set_degrees(degrees)
    # the packed gradient is gathered in place (16-byte loads at any 4-byte boundary); the result is an
    # intermediate and keeps rows of the padded stride
    d_input_prime = layout.aggregate(d_output, normalized=True, feat_dim=f, pad_columns=True)
    d_input = torch.mm(d_input_prime, W.transpose(0, 1))
    d_weight = _weight_grad(X, d_input_prime)
    return [d_input, d_weight], layout


def SAG(input, row_pointers, column_index, degrees, part_pointers, part2Node, partSize, dimWorker, warpPerBlock):
    """Unnormalised sum aggregation of `input` itself (reuse_conv.cpp:132-155, kernel cu:123-196)."""
    _check(input=input, row_pointers=row_pointers, column_index=column_index, degrees=degrees,
           part_pointers=part_pointers, part2Node=part2Node)
    fam = _layout_parts(column_index, part_pointers, part2Node, input.shape[0], partSize)
    return fam.get(input.shape[1]).aggregate(input, normalized=False, feat_dim=input.shape[1])


def GNNA_forward(input, weight, column_index, degrees, part_pointers, part2Node, partSize, dimWorker, warpPerBlock):
    """reuse_conv.cpp:158-176 -> [output]."""
    _check(input=input, weight=weight, column_index=column_index, degrees=degrees, part_pointers=part_pointers,
           part2Node=part2Node)
    fam = _layout_parts(column_index, part_pointers, part2Node, input.shape[0], partSize)
    return [_forward(fam, input, weight, degrees)[0]]


def GNNA_backward(d_output, X, W, column_index, degrees, part_pointers, part2Node, partSize, dimWorker, warpPerBlock):
    """reuse_conv.cpp:179-196 -> [d_input, d_weight]."""
    _check(d_output=d_output, X=X, W=W, column_index=column_index, degrees=degrees, part_pointers=part_pointers,
           part2Node=part2Node)
    fam = _layout_parts(column_index, part_pointers, part2Node, X.shape[0], partSize)
    return _backward(fam, d_output, X, W, degrees)[0]


def _fill_cache(lay, part_result_cache, f):
    """Upstream's caching kernel leaves the group sums and a ready flag of 1 in the caller's scratch
    (reuse_conv_kernel.cu:476-485); mirror that side effect."""
    p = part_result_cache.shape[0]
    if p == 0 or part_result_cache.shape[1] != f + 1:
        return
    ld = (f + 7) // 8 * 8
    ws = lay._workspace[: p * ld].view(p, ld)
    with torch.no_grad():
        part_result_cache[:, :f].copy_(ws[:, :f])
        part_result_cache[:, f].fill_(1.0)


def reuse_forward_v1(input, weight, column_index, degrees, part_pointers, part2Node, partSize, dimWorker, warpPerBlock,
                     part_result_cache, part_cache_flagindex, part_pointers_cache, column_index_cache):
    """reuse_conv.cpp:199-240 -> [output]."""
    _check(input=input, weight=weight, column_index=column_index, degrees=degrees, part_pointers=part_pointers,
           part2Node=part2Node, part_result_cache=part_result_cache, part_cache_flagindex=part_cache_flagindex,
           part_pointers_cache=part_pointers_cache, column_index_cache=column_index_cache)
    fam = _layout_v1(column_index, part_pointers, part2Node, part_cache_flagindex, part_pointers_cache,
                     column_index_cache, input.shape[0], partSize)
    out, lay = _forward(fam, input, weight, degrees)
    _fill_cache(lay, part_result_cache, weight.shape[1])
    return [out]


def reuse_backward_v1(d_output, X, W, column_index, degrees, part_pointers, part2Node, partSize, dimWorker,
                      warpPerBlock, part_result_cache, part_cache_flagindex, part_pointers_cache, column_index_cache):
    """reuse_conv.cpp:243-285 -> [d_input, d_weight]."""
    _check(d_output=d_output, X=X, W=W, column_index=column_index, degrees=degrees, part_pointers=part_pointers,
           part2Node=part2Node, part_result_cache=part_result_cache, part_cache_flagindex=part_cache_flagindex,
           part_pointers_cache=part_pointers_cache, column_index_cache=column_index_cache)
    fam = _layout_v1(column_index, part_pointers, part2Node, part_cache_flagindex, part_pointers_cache,
                     column_index_cache, X.shape[0], partSize)
    res, lay = _backward(fam, d_output, X, W, degrees)
    _fill_cache(lay, part_result_cache, d_output.shape[1])
    return res


def reuse_forward_v2(input, weight, uniqpart_column_index, degrees, uniqpart_pointers, part2Node_ptr, part2Node_col,
                     partSize, dimWorker, warpPerBlock, layout=None):
    """reuse_conv.cpp:288-314 -> [output].  `layout` (optional, not upstream): a LayoutFamily built from
    host arrays, which skips the cache lookup and the device-to-host copy of the plan tensors."""
    _check(input=input, weight=weight, uniqpart_column_index=uniqpart_column_index, degrees=degrees,
           uniqpart_pointers=uniqpart_pointers, part2Node_ptr=part2Node_ptr, part2Node_col=part2Node_col)
    fam = layout or _layout_v2(uniqpart_column_index, uniqpart_pointers, part2Node_ptr, part2Node_col, input.shape[0],
                               partSize)
    return [_forward(fam, input, weight, degrees)[0]]


def reuse_backward_v2(d_output, X, W, uniqpart_column_index, degrees, uniqpart_pointers, part2Node_ptr, part2Node_col,
                      partSize, dimWorker, warpPerBlock, layout=None):
    """reuse_conv.cpp:317-346 -> [d_input, d_weight]."""
    _check(d_output=d_output, X=X, W=W, uniqpart_column_index=uniqpart_column_index, degrees=degrees,
           uniqpart_pointers=uniqpart_pointers, part2Node_ptr=part2Node_ptr, part2Node_col=part2Node_col)
    fam = layout or _layout_v2(uniqpart_column_index, uniqpart_pointers, part2Node_ptr, part2Node_col, X.shape[0],
                               partSize)
    return _backward(fam, d_output, X, W, degrees)[0]
