"""Training harness: counterpart of the loop in ROF_evaluation/ROF_main.py:201-249 (Adam, cross entropy on a
training mask, accuracy on a validation mask) on the synthetic workloads, since the upstream data loader
(`data_prepare.load_graph`) and its datasets are not available.

    python -m artifact_amd.train --workload c1 --epochs 50 --kernel_type ROF_v2
"""
from __future__ import annotations

import argparse
import time

import numpy as np
import torch
import torch.nn.functional as F

from .graphgen import features as make_features
from .graphgen import make_workload
from .ROF_models import ROF_GCN
from .reuse_conv import build_input_info


def synthetic_labels(indptr, indices, x, n_classes, seed):
    """Learnable labels: argmax of a random linear teacher applied to mean-aggregated features."""
    import scipy.sparse as sp

    n = len(indptr) - 1
    a = sp.csr_matrix((np.ones(len(indices), dtype=np.float32), indices, indptr), shape=(n, n))
    deg = np.maximum(np.diff(indptr), 1).astype(np.float32)
    h = (a @ x) / deg[:, None] + x
    rng = np.random.Generator(np.random.PCG64(seed))
    teacher = rng.standard_normal((x.shape[1], n_classes)).astype(np.float32)
    return np.argmax(h @ teacher, axis=1).astype(np.int64)


def evaluate(model, feats, info, labels, mask):
    """ROF_main.py:208-216."""
    model.eval()
    with torch.no_grad():
        logits = model(feats, info)[mask]
        return float((logits.argmax(dim=1) == labels[mask]).sum().item()) / max(1, int(mask.sum().item()))


def train(model, feats, info, labels, train_mask, val_mask, epochs, lr=1e-2, weight_decay=5e-4, log_every=0):
    """ROF_main.py:201-243.  Returns (losses, validation accuracies, seconds per epoch)."""
    loss_fcn = torch.nn.CrossEntropyLoss()
    opt = torch.optim.Adam(model.parameters(), lr=lr, weight_decay=weight_decay)
    losses, accs, dur = [], [], []
    for epoch in range(epochs):
        model.train()
        if feats.is_cuda:
            torch.cuda.synchronize()
        t0 = time.time()
        opt.zero_grad()
        loss = loss_fcn(model(feats, info)[train_mask], labels[train_mask])
        loss.backward()
        opt.step()
        if feats.is_cuda:
            torch.cuda.synchronize()
        dur.append(time.time() - t0)
        losses.append(float(loss.item()))
        accs.append(evaluate(model, feats, info, labels, val_mask))
        if log_every and epoch % log_every == 0:
            print(f"Epoch {epoch:05d} | Time(s) {dur[-1]:.4f} | Loss {losses[-1]:.4f} | Accuracy {accs[-1]:.4f}")
    return losses, accs, dur


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="c1")
    ap.add_argument("--scale-down", type=int, default=0)
    ap.add_argument("--kernel_type", "-kt", default="ROF_v2", choices=["GNNA", "ROF_v1", "ROF_v2"])
    ap.add_argument("--n_hidden", "-nh", type=int, default=16)
    ap.add_argument("--n_layers", type=int, default=1)
    ap.add_argument("--part_size", type=int, default=3)
    ap.add_argument("--epochs", type=int, default=50)
    ap.add_argument("--dim_input", type=int, default=32)
    ap.add_argument("--n_classes", type=int, default=8)
    args = ap.parse_args()
    dev = torch.device("cuda")
    indptr, indices = make_workload(args.workload, args.scale_down)
    n = len(indptr) - 1
    x = make_features(n, args.dim_input, seed=2100)
    y = synthetic_labels(indptr, indices, x, args.n_classes, seed=2200)
    rng = np.random.Generator(np.random.PCG64(2300))
    split = rng.random(n)
    info = build_input_info(indptr, indices, args.part_size, device=dev)
    model = ROF_GCN(args.dim_input, args.n_hidden, args.n_classes, args.n_layers, F.relu, 0.5, add_self_loops=False,
                    reuse_size=info.reuse_size, kernel_type=args.kernel_type).to(dev)
    feats, labels = torch.from_numpy(x).to(dev), torch.from_numpy(y).to(dev)
    tm, vm, sm = (torch.from_numpy(m).to(dev) for m in (split < 0.6, (split >= 0.6) & (split < 0.8), split >= 0.8))
    losses, accs, dur = train(model, feats, info, labels, tm, vm, args.epochs, log_every=max(1, args.epochs // 10))
    print(f"nodes {n} edges {len(indices)} | mean epoch {np.mean(dur[3:]) * 1e3:.3f} ms | final loss {losses[-1]:.4f} | "
          f"val acc {accs[-1]:.4f} | test acc {evaluate(model, feats, info, labels, sm):.4f}")


if __name__ == "__main__":
    main()
