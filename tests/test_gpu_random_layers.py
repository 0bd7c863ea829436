"""Randomised parity of the layer (ROF_GCNConv with autograd) against a dense float64 statement of
    y = act( A_hat (x W) + b ),  A_hat = D^-1/2 A D^-1/2          (reuse_conv.py:144-150, reuse_conv_kernel.cu:254-276)
and of its gradients  dX = A_hat dY W^T,  dW = X^T A_hat dY,  db = column sums of dY  (reuse_conv.py:76-92),
over random symmetric graphs, widths (odd ones included), kernel types, layer orders and the fused / unfused
epilogue.  fp32 bar: 1e-5 relative to the magnitude of the summed terms, times the inner width of the GEMMs
(rocBLAS sums in fp32)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from artifact_amd.reuse_conv import ROF_GCNConv, build_input_info   # noqa: E402


def random_symmetric_csr(rng, n):
    """Symmetric, self loops (every degree >= 1), a few hubs, some triples of neighbours shared by many rows."""
    m = int(n * rng.integers(2, 12))
    a, b = rng.integers(0, n, m), rng.integers(0, n, m)
    hub = rng.choice(n, max(1, n // 100), replace=False)
    a = np.r_[a, np.repeat(hub, n // 3)]
    b = np.r_[b, rng.integers(0, n, len(hub) * (n // 3))]
    anchors = rng.choice(n, 3, replace=False)
    fans = rng.choice(n, n // 4, replace=False)
    a = np.r_[a, np.repeat(fans, 3)]
    b = np.r_[b, np.tile(anchors, len(fans))]
    rows = np.r_[a, b, np.arange(n)]
    cols = np.r_[b, a, np.arange(n)]
    key = np.unique(rows.astype(np.int64) * n + cols)
    rows, cols = key // n, key % n
    ip = np.r_[0, np.cumsum(np.bincount(rows, minlength=n))].astype(np.int32)
    return ip, cols.astype(np.int32)


@pytest.mark.parametrize("block", range(6))
def test_random_layers_match_the_dense_float64_layer(block):
    for case in range(6):
        seed = 100 * block + case
        rng = np.random.default_rng(seed)
        n = int(rng.integers(40, 1500))
        ip, ix = random_symmetric_csr(rng, n)
        ps = int(rng.integers(2, 5))
        fin, fout = (int(rng.choice([1, 3, 5, 16, 33, 47, 64, 100, 130])) for _ in range(2))
        kernel_type = str(rng.choice(["GNNA", "ROF_v1", "ROF_v2"]))
        order = str(rng.choice(["update_first", "aggregate_first", "auto"]))
        fused, bias, relu = rng.random() < 0.6, rng.random() < 0.7, rng.random() < 0.5
        needs_dx = rng.random() < 0.8
        what = (f"seed {seed}: n {n} edges {len(ix)} ps {ps} {fin}->{fout} {kernel_type} {order} fused {fused} "
                f"bias {bias} relu {relu} dx {needs_dx}")
        print(what, flush=True)
        info = build_input_info(ip, ix, ps, device="cuda", min_consumers=int(rng.choice([0, 2])),
                                hub_split=int(rng.choice([0, 16, 100])))
        torch.manual_seed(seed)
        layer = ROF_GCNConv(fin, fout, bias=bias, add_self_loops=False, kernel_type=kernel_type,
                            reuse_size=info.reuse_size, order=order, fuse_epilogue=fused,
                            activation="relu" if relu else None).cuda()
        if bias:
            with torch.no_grad():
                layer.bias.copy_(torch.from_numpy(rng.standard_normal(fout).astype(np.float32)))
        x = torch.from_numpy(rng.standard_normal((n, fin)).astype(np.float32)).cuda().requires_grad_(needs_dx)
        gy = torch.from_numpy(rng.standard_normal((n, fout)).astype(np.float32))

        a = torch.zeros((n, n), dtype=torch.float64)
        a[torch.from_numpy(np.repeat(np.arange(n), np.diff(ip))), torch.from_numpy(ix.astype(np.int64))] = 1.0
        r = torch.from_numpy(1.0 / np.sqrt(np.diff(ip).astype(np.float64)))
        a = r[:, None] * a * r[None, :]
        xd = x.detach().cpu().double().requires_grad_(True)
        wd = layer.weight.detach().cpu().double().requires_grad_(True)
        bd = layer.bias.detach().cpu().double().requires_grad_(True) if bias else None
        pre = a @ (xd @ wd) + (bd if bias else 0.0)
        yd = torch.relu(pre) if relu else pre
        # magnitude of the summed terms, for the fp32 summation bound
        mag_y = a @ (xd.detach().abs() @ wd.detach().abs()) + (bd.detach().abs() if bias else 0.0)
        tol = 1e-5 * (fin + 8)
        # a ReLU input that rounds to the other side of zero flips its gradient mask: such outputs get no
        # upstream gradient and are not compared
        live = (pre.detach().abs() > tol * mag_y + 1e-6) if relu else torch.ones_like(pre, dtype=torch.bool)
        gy = gy * live
        yd.backward(gy.double())

        y = layer(x, info)
        y.backward(gy.cuda())

        def check(name, got, want, mag):
            err = (got.detach().cpu().double() - want).abs()
            bound = 1e-6 + tol * mag
            assert bool((err <= bound).all()), f"{what}: {name} off by {float((err - bound).max()):.3e}"

        check("y", torch.where(live.cuda(), y, torch.zeros_like(y)), torch.where(live, yd.detach(), torch.zeros_like(yd)),
              mag_y)
        g_eff = gy.double().abs() * ((pre.detach() > 0) if relu else 1.0)
        rows = (n / 64 + 8) / (fin + 8)                      # dW and db sum over the n rows instead of over fin
        if needs_dx:
            check("dX", x.grad, xd.grad, (a @ g_eff) @ wd.detach().abs().T * (fout + 8) / (fin + 8))
        else:
            assert x.grad is None
        check("dW", layer.weight.grad, wd.grad, xd.detach().abs().T @ (a @ g_eff) * rows)
        if bias:
            check("db", layer.bias.grad, bd.grad, g_eff.sum(0) * rows)
