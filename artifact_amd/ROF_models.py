"""Models on top of the reuse-aware layers: counterpart of the upstream `ROF_models` module, which its
drivers import (`from ROF_models import ROF_GCN, ROF_inputInfo`, ROF_evaluation/ROF_main.py:31) but which is
not part of the upstream tree.  The constructor and call conventions are the ones the call sites fix:

    ROF_GCN(in_feats, n_hidden, n_classes, n_layers, activation, dropout, add_self_loops, reuse_size, kernel_type)
        (ROF_main.py:192-200, cuda/middle-rof.py:474-482)
    model(features, inputInfo)                (ROF_main.py:230)
    model(features, edge_index, inputInfo)    (cuda/middle-rof.py:496; edge_index is unused by the layers)

`n_layers` hidden convolutions plus the output convolution, i.e. n_layers + 1 layers (ROF_main.py:256 reports
"layers": n_layers + 1), activation between them, dropout on the input of every layer but the first.
"""
from __future__ import annotations

import torch

from .reuse_conv import ROF_GCNConv, ROF_GINConv, ROF_inputInfo  # noqa: F401  (re-exported like upstream)

__all__ = ["ROF_GCN", "ROF_GIN", "ROF_inputInfo"]


class ROF_GCN(torch.nn.Module):
    def __init__(self, in_feats, n_hidden, n_classes, n_layers, activation, dropout, add_self_loops=False,
                 reuse_size=0, kernel_type="ROF_v1", bias=True, order="update_first", fuse_epilogue=True,
                 compute_dtype=None):
        """`order`, `fuse_epilogue` and `compute_dtype` are passed to every ROF_GCNConv (not upstream).  A ReLU
        activation is then applied by the aggregation kernel of each hidden layer rather than as a pass of its
        own.  compute_dtype="bf16": bfloat16 rows and GEMM operands, fp32 sums and parameters; hidden layers hand
        bfloat16 to each other, the last layer returns float32."""
        super().__init__()
        dims = [in_feats] + [n_hidden] * n_layers + [n_classes]
        last = len(dims) - 2
        bf16 = compute_dtype in ("bf16", torch.bfloat16)
        self._fused_act = bool(fuse_epilogue) and (kernel_type != "ROF_v1" or bf16) and activation in (
            torch.relu, torch.nn.functional.relu)
        self.layers = torch.nn.ModuleList(
            ROF_GCNConv(dims[i], dims[i + 1], bias=bias, add_self_loops=add_self_loops, reuse_size=reuse_size,
                        kernel_type=kernel_type, order=order, fuse_epilogue=fuse_epilogue,
                        activation="relu" if self._fused_act and i != last else None, compute_dtype=compute_dtype,
                        out_dtype="bf16" if bf16 and i != last else None)
            for i in range(len(dims) - 1))
        self.activation = activation
        self.dropout = torch.nn.Dropout(p=dropout)

    def forward(self, features, *args):
        inputInfo = args[-1]
        h = features
        last = len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            if i != 0:
                h = self.dropout(h)
            h = layer(h, inputInfo)
            if i != last and self.activation is not None and not self._fused_act:
                h = self.activation(h)
        return h


class ROF_GIN(torch.nn.Module):
    """GIN with sum aggregation (eps fixed) and one linear map per layer, e.g. 3 x (64 -> 64)."""

    def __init__(self, in_feats, n_hidden, n_classes, n_layers, activation=torch.relu, dropout=0.0, eps=0.0,
                 kernel_type="ROF_v2"):
        super().__init__()
        dims = [in_feats] + [n_hidden] * (n_layers - 1) + [n_classes]
        self.layers = torch.nn.ModuleList(ROF_GINConv(dims[i], dims[i + 1], eps=eps, kernel_type=kernel_type)
                                          for i in range(len(dims) - 1))
        self.activation = activation
        self.dropout = torch.nn.Dropout(p=dropout)

    def forward(self, features, *args):
        inputInfo = args[-1]
        h = features
        last = len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            if i != 0:
                h = self.dropout(h)
            h = layer(h, inputInfo)
            if i != last and self.activation is not None:
                h = self.activation(h)
        return h
