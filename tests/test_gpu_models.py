"""The model and training harness on top of the layers (counterpart of the loop in
ROF_evaluation/ROF_main.py:180-249): one training step against a dense float64 reference, a short run that
must learn, and the on-disk plan container."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

import torch.nn.functional as F                                         # noqa: E402

from artifact_amd.graphgen import features, make_workload               # noqa: E402
from artifact_amd.reuse_conv import ROF_GCNConv, ROF_inputInfo, build_input_info  # noqa: E402
from artifact_amd.ROF_models import ROF_GCN, ROF_GIN                    # noqa: E402
from artifact_amd.train import synthetic_labels, train                  # noqa: E402

DEV = "cuda"


def _dense_norm_adj(ip, ix):
    n = len(ip) - 1
    a = torch.zeros((n, n), dtype=torch.float64)
    rows = np.repeat(np.arange(n), np.diff(ip))
    a[torch.from_numpy(rows), torch.from_numpy(ix.astype(np.int64))] = 1.0
    r = torch.from_numpy(1.0 / np.sqrt(np.maximum(np.diff(ip), 1).astype(np.float64)))
    return r[:, None] * a * r[None, :]


@pytest.mark.parametrize("kernel_type", ["GNNA", "ROF_v1", "ROF_v2"])
def test_one_training_step_matches_dense_float64_reference(kernel_type):
    ip, ix = make_workload("c1", 5)                                      # 512 nodes, self loops: every degree >= 1
    n = len(ip) - 1
    info = build_input_info(ip, ix, 3, device=DEV, min_consumers=2)
    x = features(n, 24, seed=41)
    y = synthetic_labels(ip, ix, x, 5, seed=42)
    model = ROF_GCN(24, 16, 5, 1, F.relu, 0.0, add_self_loops=False, reuse_size=info.reuse_size,
                    kernel_type=kernel_type).to(DEV)
    assert len(model.layers) == 2                                        # n_layers + 1 (ROF_main.py:256)
    xt, yt = torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV)
    loss = F.cross_entropy(model(xt, info), yt)
    loss.backward()
    # dense reference with the same parameters
    a = _dense_norm_adj(ip, ix)
    w1 = model.layers[0].weight.detach().cpu().double().requires_grad_(True)
    w2 = model.layers[1].weight.detach().cpu().double().requires_grad_(True)
    b1 = model.layers[0].bias.detach().cpu().double()
    b2 = model.layers[1].bias.detach().cpu().double()
    h = torch.relu(a @ (torch.from_numpy(x).double() @ w1) + b1)
    ref = F.cross_entropy(a @ (h @ w2) + b2, torch.from_numpy(y))
    ref.backward()
    assert abs(loss.item() - ref.item()) < 1e-5 * max(1.0, abs(ref.item()))
    assert torch.allclose(model.layers[0].weight.grad.cpu().double(), w1.grad, rtol=1e-3, atol=1e-6)
    assert torch.allclose(model.layers[1].weight.grad.cpu().double(), w2.grad, rtol=1e-3, atol=1e-6)
    # both upstream call conventions
    out3 = model(xt, None, info)
    assert out3.shape == (n, 5)


def _bf(t):
    """Round to bfloat16 and come back to float64: the roundings of the mixed-precision layer, restated."""
    return t.to(torch.float32).to(torch.bfloat16).double()


def test_bf16_training_step_matches_float64_with_the_same_roundings():
    """The mixed-precision step of the bf16 workload in miniature: bfloat16 features, gathered rows and GEMM
    operands, fp32 sums and parameters.  Checked twice: tightly (2e-3 in the Frobenius norm) against a float64
    evaluation that rounds to bfloat16 at exactly the points the layer does -- operands of every GEMM, the
    update before it is gathered, the hidden activation and the gradients handed from layer to layer -- and
    loosely (1e-2 logits and loss, 2e-2 gradients) against plain float64 on the bf16-rounded features."""
    ip, ix = make_workload("c5", 10)                                     # 4096 nodes, self loops
    n = len(ip) - 1
    info = build_input_info(ip, ix, 3, device=DEV, min_consumers=2)
    x = torch.from_numpy(features(n, 64, seed=45, kind="uniform")).to(torch.bfloat16)
    y = torch.from_numpy(synthetic_labels(ip, ix, x.float().numpy(), 7, seed=46))
    torch.manual_seed(7)
    model = ROF_GCN(64, 48, 7, 1, F.relu, 0.0, add_self_loops=False, reuse_size=info.reuse_size,
                    kernel_type="ROF_v2", compute_dtype="bf16").to(DEV)
    with torch.no_grad():
        model.layers[0].bias.uniform_(-0.1, 0.1)
        model.layers[1].bias.uniform_(-0.1, 0.1)
    hidden = model.layers[0](x.to(DEV), info)
    assert hidden.dtype == torch.bfloat16 and (hidden >= 0).all()       # ReLU applied in the store, bf16 hand-over
    logits = model(x.to(DEV), info)
    assert logits.dtype == torch.float32
    loss = F.cross_entropy(logits, y.to(DEV))
    loss.backward()
    assert model.layers[0].weight.grad.dtype == torch.float32

    a = _dense_norm_adj(ip, ix)
    w1, w2 = (l.weight.detach().cpu().double() for l in model.layers)
    b1, b2 = (l.bias.detach().cpu().double() for l in model.layers)
    xd = x.double()

    # (1) float64 with the layer's roundings, forward and backward written out
    h = _bf(torch.relu(a @ _bf(xd @ _bf(w1)) + b1))
    lg = (a @ _bf(h @ _bf(w2)) + b2).requires_grad_(True)
    F.cross_entropy(lg, y).backward()
    g2 = lg.grad
    dt2 = _bf(a @ _bf(g2))
    want = {"logits": lg.detach(), "db2": g2.sum(0), "dW2": h.T @ dt2}
    g1 = _bf(dt2 @ _bf(w2).T) * (h > 0)
    dt1 = _bf(a @ g1)
    want.update(db1=g1.sum(0), dW1=xd.T @ dt1)
    got = {"logits": logits, "dW1": model.layers[0].weight.grad, "db1": model.layers[0].bias.grad,
           "dW2": model.layers[1].weight.grad, "db2": model.layers[1].bias.grad}
    for k, w in want.items():
        diff = (got[k].detach().cpu().double() - w).norm().item()
        assert diff <= 2e-3 * w.norm().item(), f"{k} against the rounded evaluation: {diff / w.norm().item():.2e}"

    # (2) plain float64: what the roundings cost
    w1r, w2r, b1r, b2r = (t.clone().requires_grad_(True) for t in (w1, w2, b1, b2))
    ref_logits = a @ (torch.relu(a @ (xd @ w1r) + b1r) @ w2r) + b2r
    ref = F.cross_entropy(ref_logits, y)
    ref.backward()
    assert abs(loss.item() - ref.item()) < 1e-2 * ref.item()
    for k, w, rel in (("logits", ref_logits.detach(), 1e-2), ("dW1", w1r.grad, 2e-2), ("db1", b1r.grad, 2e-2),
                      ("dW2", w2r.grad, 2e-2), ("db2", b2r.grad, 2e-2)):
        diff = (got[k].detach().cpu().double() - w).norm().item()
        assert diff <= rel * w.norm().item(), f"{k} against plain float64: {diff / w.norm().item():.2e}"


def test_bf16_layer_orders_agree():
    """aggregate-first in bfloat16 (the sum is rounded before the GEMM instead of after) stays within 1e-2 of
    update-first on the outputs and 3e-2 on the gradients (Frobenius norm)."""
    ip, ix = make_workload("c5", 10)
    n = len(ip) - 1
    info = build_input_info(ip, ix, 3, device=DEV, min_consumers=2)
    x = torch.from_numpy(features(n, 40, seed=47, kind="uniform")).to(torch.bfloat16).to(DEV)
    coef = torch.from_numpy(features(n, 56, seed=48)).to(DEV)
    res = {}
    for order in ("update_first", "aggregate_first"):
        torch.manual_seed(11)
        conv = ROF_GCNConv(40, 56, add_self_loops=False, kernel_type="ROF_v2", compute_dtype="bf16", order=order,
                           activation="relu").to(DEV)
        xg = x.clone().requires_grad_(True)
        out = conv(xg, info)
        assert out.dtype == torch.float32
        (out * coef).sum().backward()
        res[order] = (out.detach(), xg.grad.float(), conv.weight.grad, conv.bias.grad)
    # the outputs differ by bf16 roundings; the gradients also by the few ReLU masks those roundings flip
    for u, v, what, rel in zip(res["update_first"], res["aggregate_first"], ("out", "dX", "dW", "db"),
                               (1e-2, 3e-2, 3e-2, 3e-2)):
        assert (u - v).norm().item() <= rel * u.norm().item(), what


def test_training_learns_and_gin_runs():
    ip, ix = make_workload("c1", 3)
    n = len(ip) - 1
    info = build_input_info(ip, ix, 3, device=DEV, min_consumers=2)
    x = features(n, 16, seed=51)
    y = synthetic_labels(ip, ix, x, 4, seed=52)
    torch.manual_seed(0)
    model = ROF_GCN(16, 32, 4, 1, F.relu, 0.1, add_self_loops=False, reuse_size=info.reuse_size,
                    kernel_type="ROF_v2").to(DEV)
    xt, yt = torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV)
    mask = torch.ones(n, dtype=torch.bool, device=DEV)
    losses, accs, _ = train(model, xt, info, yt, mask, mask, epochs=60, lr=2e-2, weight_decay=0.0)
    assert losses[-1] < 0.7 * losses[0] and accs[-1] > 0.5
    gin = ROF_GIN(16, 64, 4, 3).to(DEV)
    out = gin(xt, info)
    out.sum().backward()
    assert out.shape == (n, 4) and all(p.grad is not None for p in gin.parameters())


def test_three_layer_gin_matches_a_dense_float64_model():
    """The block-structured workload's model (3 x GIN 64 -> 64, sum aggregation, eps = 0, ReLU between) on a
    scaled-down graph of the same generator: forward, input gradient and every parameter gradient against the
    same model written with a dense float64 adjacency."""
    ip, ix = make_workload("c3", 6)                                      # SBM, 4 blocks of 4096 nodes
    n = len(ip) - 1
    info = build_input_info(ip, ix, 3, device=DEV, min_consumers=2)
    torch.manual_seed(5)
    gin = ROF_GIN(64, 64, 64, 3, activation=torch.relu, eps=0.0).to(DEV)
    x = torch.from_numpy(features(n, 64, seed=71)).to(DEV).requires_grad_(True)
    coef = torch.from_numpy(features(n, 64, seed=72)).to(DEV)
    out = gin(x, info)
    (out * coef).sum().backward()
    # dense float64 model: h <- W_l ((1 + eps) h + A h) + b_l
    rows = np.repeat(np.arange(n), np.diff(ip))
    a = torch.sparse_coo_tensor(np.stack([rows, ix.astype(np.int64)]), np.ones(len(ix)), (n, n)).coalesce()
    ws = [(l.mlp.weight.detach().cpu().double().requires_grad_(True), l.mlp.bias.detach().cpu().double().requires_grad_(True))
          for l in gin.layers]
    xd = x.detach().cpu().double().requires_grad_(True)
    h = xd
    for i, (w, b) in enumerate(ws):
        h = (h + torch.sparse.mm(a, h)) @ w.t() + b
        if i != 2:
            h = torch.relu(h)
    (h * coef.cpu().double()).sum().backward()
    # three sums over ~27 neighbours each compound the fp32 round-off: relative to the size of the whole result
    def rel(got, want):
        return ((got.detach().cpu().double() - want.detach()).norm() / want.detach().norm()).item()
    assert rel(out, h) < 2e-6
    assert rel(x.grad, xd.grad) < 5e-6
    for layer, (w, b) in zip(gin.layers, ws):
        assert rel(layer.mlp.weight.grad, w.grad) < 5e-6 and rel(layer.mlp.bias.grad, b.grad) < 5e-6
    # element-wise at the stated bar, widened by the magnitude of the result (sums of sums: no per-term bound here)
    scale = h.detach().abs().max().item()
    assert (out.detach().cpu().double() - h.detach()).abs().max().item() <= 1e-5 * scale


@pytest.mark.parametrize("fused", [False, True])
def test_loss_curve_follows_a_dense_float64_model(fused):
    """Forty Adam steps of the two-layer GCN (no dropout) against the same model written with a dense float64
    adjacency and trained by the same optimizer from the same parameters: the loss curves must stay together
    (fp32 round-off only), and so must the trained weights."""
    ip, ix = make_workload("c1", 4)                                      # 1024 nodes
    n = len(ip) - 1
    info = build_input_info(ip, ix, 3, device=DEV, min_consumers=2)
    x = features(n, 20, seed=61)
    y = synthetic_labels(ip, ix, x, 6, seed=62)
    torch.manual_seed(3)
    model = ROF_GCN(20, 24, 6, 1, F.relu, 0.0, add_self_loops=False, reuse_size=info.reuse_size,
                    kernel_type="ROF_v2", fuse_epilogue=fused).to(DEV)
    params = [(l.weight.detach().cpu().double().clone().requires_grad_(True),
               l.bias.detach().cpu().double().clone().requires_grad_(True)) for l in model.layers]
    xt, yt = torch.from_numpy(x).to(DEV), torch.from_numpy(y).to(DEV)
    mask = torch.ones(n, dtype=torch.bool, device=DEV)
    losses, _, _ = train(model, xt, info, yt, mask, mask, epochs=40, lr=1e-2, weight_decay=5e-4)
    a, xd, yd = _dense_norm_adj(ip, ix), torch.from_numpy(x).double(), torch.from_numpy(y)
    opt = torch.optim.Adam([t for wb in params for t in wb], lr=1e-2, weight_decay=5e-4)
    want = []
    for _ in range(40):
        opt.zero_grad()
        (w1, b1), (w2, b2) = params
        loss = F.cross_entropy(a @ (torch.relu(a @ (xd @ w1) + b1) @ w2) + b2, yd)
        loss.backward()
        opt.step()
        want.append(float(loss.detach()))
    assert want[-1] < 0.9 * want[0]                                      # the reference itself learns
    assert np.allclose(losses, want, rtol=2e-4, atol=1e-5), np.abs(np.array(losses) - np.array(want)).max()
    for layer, (w, b) in zip(model.layers, params):
        assert torch.allclose(layer.weight.detach().cpu().double(), w.detach(), rtol=0, atol=2e-4)
        assert torch.allclose(layer.bias.detach().cpu().double(), b.detach(), rtol=0, atol=2e-4)


def test_plan_container_round_trips_through_disk(tmp_path):
    ip, ix = make_workload("c1", 4)
    n = len(ip) - 1
    info = build_input_info(ip, ix, 3, device=DEV, min_consumers=2)
    path = str(tmp_path / "plan.npz")
    info.save(path)
    back = ROF_inputInfo.load(path, device=DEV, min_consumers=2)
    for name in ("uniqpart_column_index", "part_cache_flagindex", "column_index", "degrees"):
        assert torch.equal(getattr(info, name), getattr(back, name))
    x = torch.from_numpy(features(n, 12, seed=61)).to(DEV)
    w = torch.from_numpy(features(12, 8, seed=62)).to(DEV)
    from artifact_amd.reuse_conv import ROF_GCNConvFunc
    info.part_result_cache = back.part_result_cache = torch.zeros((info.reuse_size, 9), device=DEV)
    a = ROF_GCNConvFunc.apply(x, w, info, False, "ROF_v2")
    b = ROF_GCNConvFunc.apply(x, w, back, False, "ROF_v2")
    assert torch.equal(a, b)


def test_timed_layout_choices_are_saved_with_the_plan(tmp_path):
    """What an autotuning family chose by timing is written with the plan and replayed after a load: no timing, the
    same cut and launch settings, the same bits."""
    from artifact_amd.reuse_conv import ROF_GCNConvFunc
    ip, ix = make_workload("c4", 6)
    n = len(ip) - 1
    info = build_input_info(ip, ix, 3, device=DEV, autotune=True)
    x = torch.from_numpy(features(n, 20, seed=63)).to(DEV)
    w = torch.from_numpy(features(20, 47, seed=64)).to(DEV)
    a = ROF_GCNConvFunc.apply(x, w, info, False, "ROF_v2")
    chosen = info.layouts["ROF_v2"].choices()
    assert chosen and all(set(v) == {"cut", "segment", "tuning"} for v in chosen.values())
    path = str(tmp_path / "plan.npz")
    info.save(path)
    back = ROF_inputInfo.load(path, device=DEV)
    b = ROF_GCNConvFunc.apply(x, w, back, False, "ROF_v2")
    fam = back.layouts["ROF_v2"]
    assert fam.choices() == chosen and all(v.get("replayed") for v in fam.chosen.values()) and not fam.autotune
    assert torch.equal(a, b)
