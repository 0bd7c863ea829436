"""The remaining workloads at their full sizes.

* 2^18-node R-MAT (3.7 M edges) at widths 256 and 40 and the 2^20-node block model (27 M edges, unnormalised
  sums, width 64): small enough for the float64 closed form of the whole layer, so every element is compared.
* 2^22-node R-MAT (133 M edges) with bfloat16 rows of width 256 -- a 2.1 GB feature matrix, a partial-sum
  workspace above 1 GB, more than a million segments: checked through properties that need no oracle run of that
  size (exact integer sums, a float64 checksum of checksums, reuse == reuse-disabled, linearity in exactly
  representable inputs, sampled rows in float64)."""
import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from artifact_amd import reuse_search_ext as R                     # noqa: E402
from artifact_amd.graphgen import features, make_workload          # noqa: E402
from artifact_amd.layout import Layout, lanes_per_row               # noqa: E402
from helpers import close_fp32                                      # noqa: E402

DEV = "cuda"


def _layouts(ip, ix, ps, feat, bf16=False):
    plan = R.build_plan(ip, ix, ps)
    n = len(ip) - 1
    args = (plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"], plan["part2Node_col"], n, ps)
    opts = dict(lanes_per_row=lanes_per_row(feat, bf16), elem_bytes=2 if bf16 else 4)
    return {"default": Layout.from_v2(*args, **opts), "shared": Layout.from_v2(*args, min_consumers=3, **opts),
            "disabled": Layout.from_v2(*args, disable_reuse=True, **opts)}


def _closed_form64(ip, ix, x64, normalized):
    n = len(ip) - 1
    a = sp.csr_matrix((np.ones(len(ix)), ix, ip), shape=(n, n))
    if not normalized:
        return a @ x64, a @ np.abs(x64)
    r = 1.0 / np.sqrt(np.maximum(np.diff(ip), 1).astype(np.float64))
    # the kernels use rsqrt correctly rounded to float32 (reuse_conv_kernel.cu:254,276)
    r = r.astype(np.float32).astype(np.float64)
    return r[:, None] * (a @ (r[:, None] * x64)), r[:, None] * (a @ (r[:, None] * np.abs(x64)))


@pytest.fixture(scope="module")
def c2():
    ip, ix = make_workload("c2")
    return ip, ix


@pytest.mark.parametrize("feat", [256, 40])
def test_c2_full_size_against_the_closed_form(c2, feat):
    ip, ix = c2
    n = len(ip) - 1
    lays = _layouts(ip, ix, 3, feat)
    x = features(n, feat, seed=2002)
    want, mag = _closed_form64(ip, ix, x.astype(np.float64), True)
    xt = torch.from_numpy(x).to(DEV)
    deg = torch.from_numpy(np.diff(ip).astype(np.float32)).to(DEV)
    outs = {}
    for name, lay in lays.items():
        lay.set_degrees(deg)
        out = torch.full((n, feat), float("nan"), device=DEV)
        lay.aggregate(xt, normalized=True, out=out)
        outs[name] = out
        close_fp32(out.cpu().numpy(), want, mag, what=f"c2 F={feat} {name}")
    assert lays["shared"].stats()["materialised_groups"] > 0
    assert torch.equal(outs["default"], outs["disabled"])      # the cost model folds this plan: same schedule
    assert torch.allclose(outs["shared"], outs["disabled"], rtol=1e-5, atol=2e-6)
    # the backward pass aggregates a packed gradient with the same plan and keeps padded rows for the GEMMs
    g = torch.from_numpy(features(n, feat, seed=7)).to(DEV)
    gw, gm = _closed_form64(ip, ix, g.cpu().numpy().astype(np.float64), True)
    back = lays["default"].aggregate(g, normalized=True, pad_columns=True)
    close_fp32(back.cpu().numpy(), gw, gm, what=f"c2 F={feat} backward")
    for lay in lays.values():
        lay.close()


def test_c3_full_size_sum_aggregation_against_the_closed_form():
    ip, ix = make_workload("c3")
    n = len(ip) - 1
    assert n == 1 << 20
    lays = _layouts(ip, ix, 3, 64)
    x = features(n, 64, seed=2003)
    want, mag = _closed_form64(ip, ix, x.astype(np.float64), False)
    xt = torch.from_numpy(x).to(DEV)
    outs = {}
    for name, lay in lays.items():
        out = torch.full((n, 64), float("nan"), device=DEV)
        lay.aggregate(xt, normalized=False, out=out)
        outs[name] = out
        close_fp32(out.cpu().numpy(), want, mag, what=f"c3 {name}")
    assert torch.allclose(outs["shared"], outs["disabled"], rtol=1e-5, atol=2e-6)
    # the GIN layer's own-row term, added as the row is stored: (1 + eps) x_v + sum
    own = lays["default"].aggregate(xt, normalized=False, self_weight=1.0)
    close_fp32(own.cpu().numpy(), want + x, mag + np.abs(x), what="c3 own row")
    # all-ones features: the sums are the in-degrees, exactly
    ones = torch.ones((n, 8), device=DEV)
    got = lays["default"].aggregate(ones, normalized=False).cpu().numpy()
    assert np.array_equal(got, np.repeat(np.diff(ip).astype(np.float32)[:, None], 8, axis=1))
    for lay in lays.values():
        lay.close()


@pytest.fixture(scope="module")
def c5():
    ip, ix = make_workload("c5")
    n = len(ip) - 1
    return ip, ix, n, _layouts(ip, ix, 3, 256, bf16=True)


def test_c5_full_size_bf16_rows(c5):
    ip, ix, n, lays = c5
    assert n == 1 << 22
    deg = np.diff(ip).astype(np.float32)
    degt = torch.from_numpy(deg).to(DEV)
    reuse, shared, plain = lays["default"], lays["shared"], lays["disabled"]
    st = reuse.stats()
    assert st["hub_segments"] > 1_000_000 and reuse.workspace_bytes(256) > (1 << 30)
    # (1) all-ones bf16 rows, unnormalised: the sums are the in-degrees, exactly (fp32 accumulation of integers)
    ones = torch.ones((n, 16), dtype=torch.bfloat16, device=DEV)
    for lay in (reuse, shared):
        got = lay.aggregate(ones, normalized=False)
        assert torch.equal(got[:, 0].cpu(), torch.from_numpy(deg)) and bool((got == got[:, :1]).all())
    del ones, got
    # (2) checksum of checksums on random bf16 rows: sum_v out[v] = sum_u deg(u) x[u] (symmetric graph)
    g = torch.Generator(device=DEV).manual_seed(55)
    x = (torch.rand((n, 256), device=DEV, generator=g) * 2 - 1).to(torch.bfloat16)
    out = reuse.aggregate(x, normalized=False)
    lhs = out.double().sum(0).cpu().numpy()
    rhs = (x.double() * degt.double()[:, None]).sum(0).cpu().numpy()
    assert np.allclose(lhs, rhs, rtol=1e-6, atol=0.5)       # one lost or doubled edge of a hub would move a sum by ~1
    del out
    # (3) the normalised layer: default == reuse-disabled bit for bit (folded plan), forced sharing to round-off
    for lay in (reuse, shared, plain):
        lay.set_degrees(degt)
    a = reuse.aggregate(x, normalized=True)
    b = plain.aggregate(x, normalized=True)
    assert torch.equal(a, b)
    c = shared.aggregate(x, normalized=True, out=b)
    assert torch.allclose(a, c, rtol=1e-5, atol=2e-6)
    del b, c
    # (4) sampled rows against float64 on the bf16-rounded inputs: the stated bar (rel 1e-2) and the fp32 bar
    rows = np.random.default_rng(2).integers(0, n, 300)
    rows = np.concatenate([rows, np.argsort(deg)[-3:]])     # and the three longest rows (hundreds of segments)
    r = 1.0 / np.sqrt(np.maximum(deg, 1).astype(np.float64))
    r = r.astype(np.float32).astype(np.float64)
    ah = a[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    for i, v in enumerate(rows):
        nb = ix[ip[v]:ip[v + 1]]
        xn = x[torch.from_numpy(nb.astype(np.int64)).to(DEV)].double().cpu().numpy()
        want = r[v] * (xn * r[nb, None]).sum(0)
        mag = r[v] * (np.abs(xn) * r[nb, None]).sum(0)
        assert (np.abs(ah[i] - want) <= 1e-6 + 1e-2 * np.abs(want) + 1e-2 * mag).all(), v
        close_fp32(ah[i], want, mag, what=f"c5 row {v}")
    # (5) fused store at this size: bias + ReLU + bf16 rounding == separate passes, bit for bit
    bias = torch.randn(256, device=DEV, generator=g)
    fused = reuse.aggregate(x, normalized=True, bias=bias, relu=True, out_dtype=torch.bfloat16)
    assert torch.equal(fused.view(torch.int16), torch.relu(a + bias).to(torch.bfloat16).view(torch.int16))
