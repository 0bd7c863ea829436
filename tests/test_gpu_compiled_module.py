"""The compiled operator module (artifact_amd/_ROF*.so, csrc/rof_torch.cpp: upstream's seven `ROF` functions as a
C++ extension over the C ABI) against the fp32 restatements of the upstream kernels, the float64 closed form, and
bit for bit against the Python form of the same interface (artifact_amd/ROF.py)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from artifact_amd import ROF as ROF_py                                     # noqa: E402
from artifact_amd import rof_module                                        # noqa: E402
from artifact_amd.graphgen import features, glorot, make_workload          # noqa: E402
from artifact_amd.reuse_conv import build_input_info                       # noqa: E402
from helpers import close_fp32                                             # noqa: E402

DEV = "cuda"


@pytest.fixture(scope="module")
def ROF():
    return rof_module.compiled()


def _setup(ps=3, fin=20, fout=47):
    ip, ix = make_workload("c1", 2)
    n = len(ip) - 1
    info = build_input_info(ip, ix, part_size=ps, device=DEV, min_consumers=2)
    return ip, ix, n, info, features(n, fin, seed=21), glorot(fin, fout, seed=22)


def _call(kind, ii, *lead):
    dw, wpb = 32, ii.warpPerBlock
    if kind == "GNNA":
        return lead + (ii.column_index, ii.degrees, ii.part_pointers, ii.part2Node, ii.partSize, dw, wpb)
    if kind == "v1":
        return lead + (ii.column_index, ii.degrees, ii.part_pointers, ii.part2Node, ii.partSize, dw, wpb,
                       ii.part_result_cache, ii.part_cache_flagindex, ii.part_pointers_cache, ii.column_index_cache)
    return lead + (ii.uniqpart_column_index, ii.degrees, ii.uniqpart_pointers, ii.part2Node_ptr, ii.part2Node_col,
                   ii.partSize, dw, wpb)


@pytest.mark.parametrize("fout", [47, 32, 3, 100, 300])
def test_forward_of_all_three_kernel_types(oracle, ROF, fout):
    ip, ix, n, info, x, w = _setup(fout=fout)
    xt, wt = torch.from_numpy(x).to(DEV), torch.from_numpy(w).to(DEV)
    deg = np.diff(ip).astype(np.float32)
    tmp = x.astype(np.float64) @ w.astype(np.float64)
    want, mag = oracle.closed_form(ip, ix, tmp, deg), oracle.closed_form(ip, ix, np.abs(tmp), deg)
    p = info.plan
    tmp32 = (xt @ wt).cpu().numpy()
    ref_v2 = oracle.agg_v2(tmp32, deg, p["uniqpart_column_index"], p["uniqpart_pointers"], p["part2Node_ptr"],
                           p["part2Node_col"])
    for kind in ("GNNA", "v1", "v2"):
        info.part_result_cache = torch.full((info.reuse_size, fout + 1), float("nan"), device=DEV)
        res = getattr(ROF, {"GNNA": "GNNA_forward", "v1": "reuse_forward_v1", "v2": "reuse_forward_v2"}[kind])(
            *_call(kind, info, xt, wt))
        assert isinstance(res, list) and len(res) == 1
        out = res[0]
        assert out.shape == (n, fout) and out.is_contiguous() and out.dtype == torch.float32
        close_fp32(out.cpu().numpy(), want, mag, rtol=2e-5)
        close_fp32(out.cpu().numpy(), ref_v2.astype(np.float64), mag)
        mine_cache = info.part_result_cache.clone()
        info.part_result_cache = torch.full((info.reuse_size, fout + 1), float("nan"), device=DEV)
        py = getattr(ROF_py, {"GNNA": "GNNA_forward", "v1": "reuse_forward_v1", "v2": "reuse_forward_v2"}[kind])(
            *_call(kind, info, xt, wt))[0]
        assert torch.equal(out, py), kind                      # same library, same schedule: same bits
        if kind == "v1":                                       # the caller's scratch: group sums + ready flags
            assert torch.equal(mine_cache, info.part_result_cache) and (mine_cache[:, -1] == 1.0).all()


@pytest.mark.parametrize("kind", ["GNNA", "v1", "v2"])
def test_backward_functions(oracle, ROF, kind):
    ip, ix, n, info, x, w = _setup(fin=24, fout=47)
    info.part_result_cache = torch.zeros((info.reuse_size, 48), device=DEV)
    xt, wt = torch.from_numpy(x).to(DEV), torch.from_numpy(w).to(DEV)
    g = features(n, 47, seed=23)
    gt = torch.from_numpy(g).to(DEV)
    name = {"GNNA": "GNNA_backward", "v1": "reuse_backward_v1", "v2": "reuse_backward_v2"}[kind]
    d_input, d_weight = getattr(ROF, name)(*_call(kind, info, gt, xt, wt))
    deg = np.diff(ip).astype(np.float32)
    gp = oracle.closed_form(ip, ix, g, deg)                   # same un-transposed plan on d_output (cu:1021-1041)
    assert d_input.shape == (n, 24) and d_weight.shape == (24, 47)
    assert np.allclose(d_input.cpu().numpy(), gp @ w.astype(np.float64).T, rtol=1e-4, atol=1e-5)
    assert np.allclose(d_weight.cpu().numpy(), x.astype(np.float64).T @ gp, rtol=1e-4, atol=1e-3)
    py_in, py_w = getattr(ROF_py, name)(*_call(kind, info, gt, xt, wt))
    assert torch.equal(d_input, py_in) and torch.equal(d_weight, py_w)


def test_sag_and_input_checks(oracle, ROF):
    ip, ix, n, info, x, w = _setup(fin=19)
    xt = torch.from_numpy(x).to(DEV)
    args = (info.row_pointers, info.column_index, info.degrees, info.part_pointers, info.part2Node, info.partSize, 19, 4)
    out = ROF.SAG(xt, *args)
    assert isinstance(out, torch.Tensor) and out.shape == (n, 19)
    close_fp32(out.cpu().numpy(), oracle.closed_form(ip, ix, x, normalized=False),
               oracle.closed_form(ip, ix, np.abs(x), normalized=False))
    assert torch.equal(out, ROF_py.SAG(xt, *args))
    wt = torch.from_numpy(np.ascontiguousarray(w.T)).to(DEV).t()           # right shape, not contiguous
    with pytest.raises(RuntimeError, match="weight must be contiguous"):   # CHECK_INPUT, reuse_conv.cpp:121-123
        ROF.GNNA_forward(*_call("GNNA", info, xt, wt))
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        ROF.GNNA_forward(*_call("GNNA", info, xt.cpu(), torch.from_numpy(w).to(DEV)))
    with pytest.raises(RuntimeError, match="float32"):                      # the double SAG of upstream has no defined result
        ROF.SAG(xt.double(), *args)
    ROF.clear_layout_cache()


def test_upstream_layer_runs_on_the_compiled_module(oracle, ROF, monkeypatch):
    """The layer API with its operator module swapped for the compiled one, the way an upstream script would see
    it after `rof_module.install()`: ROF_GCNConvFunc's forward and 5-tuple backward (reuse_conv.py:30-93)."""
    from artifact_amd import reuse_conv

    ip, ix, n, info, x, w = _setup(fin=16, fout=12)
    monkeypatch.setattr(reuse_conv, "ROF", ROF)
    info.layouts = {}                                        # no prebuilt layouts: the module re-lays the tensors out
    xt = torch.from_numpy(x).to(DEV).requires_grad_(True)
    wt = torch.from_numpy(w).to(DEV).requires_grad_(True)
    out = reuse_conv.ROF_GCNConvFunc.apply(xt, wt, info, False, "ROF_v2")
    out.sum().backward()
    deg = np.diff(ip).astype(np.float32)
    tmp = x.astype(np.float64) @ w.astype(np.float64)
    close_fp32(out.detach().cpu().numpy(), oracle.closed_form(ip, ix, tmp, deg),
               oracle.closed_form(ip, ix, np.abs(tmp), deg), rtol=2e-5)
    gp = oracle.closed_form(ip, ix, np.ones((n, 12)), deg)
    assert np.allclose(xt.grad.cpu().numpy(), gp @ w.astype(np.float64).T, rtol=1e-4, atol=1e-5)
    assert np.allclose(wt.grad.cpu().numpy(), x.astype(np.float64).T @ gp, rtol=1e-4, atol=1e-3)


def test_the_compiled_module_chooses_cuts_by_timing_when_asked(oracle, ROF, monkeypatch):
    """ROF_AUTOTUNE=1: the module times the rule's layout against four other cuts of the long rows and calibrates the
    launch settings of the winner (rof_aggregate_timed, rof_layout_calibrate from C++).  Whatever it picks, forward
    and backward give the float64 closed form; with the variable unset the cache holds the rule's layouts again."""
    ip, ix = make_workload("c4", 5)                                      # 75 000 nodes, rows of up to 10 000 entries
    n = len(ip) - 1
    info = build_input_info(ip, ix, part_size=3, device=DEV)
    x, w = features(n, 20, seed=31), glorot(20, 47, seed=32)
    xt, wt = torch.from_numpy(x).to(DEV), torch.from_numpy(w).to(DEV)
    deg = np.diff(ip).astype(np.float32)
    tmp = x.astype(np.float64) @ w.astype(np.float64)
    want, mag = oracle.closed_form(ip, ix, tmp, deg), oracle.closed_form(ip, ix, np.abs(tmp), deg)
    ROF.clear_layout_cache()
    plain = ROF.reuse_forward_v2(*_call("v2", info, xt, wt))[0].clone()
    monkeypatch.setenv("ROF_AUTOTUNE", "1")
    ROF.clear_layout_cache()
    tuned = ROF.reuse_forward_v2(*_call("v2", info, xt, wt))[0]
    close_fp32(tuned.cpu().numpy(), want, mag)
    assert torch.equal(ROF.reuse_forward_v2(*_call("v2", info, xt, wt))[0], tuned)       # timed once, cached
    d_out = torch.from_numpy(features(n, 47, seed=33)).to(DEV)
    d_in, d_w = ROF.reuse_backward_v2(*_call("v2", info, d_out, xt, wt))
    agg = oracle.closed_form(ip, ix, d_out.cpu().numpy().astype(np.float64), deg)
    assert np.allclose(d_in.cpu().numpy(), agg @ w.astype(np.float64).T, rtol=1e-4, atol=1e-4)
    assert np.allclose(d_w.cpu().numpy(), x.astype(np.float64).T @ agg, rtol=1e-4, atol=1e-3)
    monkeypatch.delenv("ROF_AUTOTUNE")
    ROF.clear_layout_cache()
    assert torch.equal(ROF.reuse_forward_v2(*_call("v2", info, xt, wt))[0], plain)
