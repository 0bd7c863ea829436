"""Randomised parity of the aggregation through the C ABI: random graphs (empty rows, hubs), random plans
(upstream's builder or none), random schedule options (cut, segment length, lanes per row, entry order, tile
size), random widths, strides (with and without permission to use the padding), input and output types and
epilogues, each against the float64 closed form
    out[v] = relu( rs(deg v) * sum_u rs(deg u) x[u]  +  self_weight * x[v]  +  bias )
(reuse_conv_kernel.cu:254,276 for the normalisation; reuse_conv.py:147-150 for the bias).  The schedule may
re-bracket the sum in any way, so every case must meet the same bar: fp32 rel 1e-5 (+ the summation bound),
bf16 inputs exact products of the rounded inputs, bf16 outputs one rounding (2^-8 relative) away."""
import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from artifact_amd import reuse_search_ext as R            # noqa: E402
from artifact_amd.layout import Layout                     # noqa: E402
from helpers import close_fp32                             # noqa: E402

LANES = [0, 4, 8, 10, 12, 16, 20, 32, 64]


def random_csr(rng, n, ps):
    """Rows of 0..40 neighbours, a few hubs of up to n, and rows made of one to three of a few shared
    neighbour sets of `ps` ids each (each set inside its own id range, so the sets stay whole when a row is cut
    into parts and the plan builder finds parts to share); columns sorted and unique per row."""
    kind = rng.random(n)
    deg = np.where(kind < 0.15, 0, rng.integers(1, 41, n))
    hubs = rng.choice(n, max(1, n // 200), replace=False)
    deg[hubs] = rng.integers(n // 4, n + 1, len(hubs))
    kind[hubs] = 0.5
    sets = max(1, min(n // (2 * ps), n // 50 + 1))
    width = n // sets
    shared = [j * width + np.sort(rng.choice(width, ps, replace=False)) for j in range(sets)]
    rows = []
    for v in range(n):
        if kind[v] > 0.6:
            rows.append(np.concatenate([shared[j] for j in np.sort(rng.choice(sets, min(sets, int(rng.integers(1, 4))),
                                                                              replace=False))]))
            continue
        rows.append(np.unique(rng.choice(n, min(int(deg[v]), n), replace=False)))
    ip = np.r_[0, np.cumsum([len(r) for r in rows])].astype(np.int32)
    ix = (np.concatenate(rows) if ip[-1] else np.zeros(0)).astype(np.int32)
    return ip, ix


def bf16_round(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float32).numpy()


@pytest.mark.parametrize("block", range(12))
def test_random_schedules_match_the_closed_form(oracle, block):
    for case in range(10):
        seed = 1000 * block + case
        rng = np.random.default_rng(seed)
        n = int(rng.integers(12, 3000))
        ps = int(rng.integers(2, 6))
        ip, ix = random_csr(rng, n, ps)
        opts = dict(hub_split=int(rng.choice([0, 8, 33, 100])), segment=int(rng.choice([0, 1, 5, 16])),
                    lanes_per_row=int(rng.choice(LANES)), entry_order=str(rng.choice(["descending", "plan", "ascending"])),
                    tile_rows=int(rng.choice([0, 64])), elem_bytes=int(rng.choice([0, 2, 4])),
                    local_groups=int(rng.choice([0, 0, 1, 30, -1])))
        use_plan = rng.random() < 0.6
        if use_plan:
            t = sp.csr_matrix((np.ones(len(ix), np.int8), ix, ip), shape=(n, n)).tocsc()   # the graphs are directed
            plan = R.build_plan(ip, ix, ps, t.indptr, t.indices)
            lay = Layout.from_v2(plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"],
                                 plan["part2Node_col"], n, ps, min_consumers=int(rng.choice([0, 2, 3])), **opts)
        else:
            lay = Layout.from_csr(ip, ix, **opts)
        feat = int(rng.choice([1, 2, 3, 5, 8, 17, 32, 47, 64, 100, 129, 256, 300]))
        ld = feat + int(rng.choice([0, 0, 1, 3, 8]))
        bf16_in, bf16_out = rng.random() < 0.35, rng.random() < 0.3
        normalized = rng.random() < 0.6
        bias = rng.standard_normal(feat).astype(np.float32) if rng.random() < 0.5 else None
        relu = rng.random() < 0.5
        self_weight = float(rng.choice([0.0, 0.0, 0.7, -1.25]))
        pad = bool(rng.random() < 0.4)                         # rows taken as whole vectors where the stride allows it
        what = (f"seed {seed}: n {n} edges {len(ix)} ps {ps} plan {use_plan} {opts} feat {feat} ld {ld} "
                f"bf16 in {bf16_in} out {bf16_out} normalized {normalized} bias {bias is not None} relu {relu} "
                f"self {self_weight} pad {pad} stats {lay.stats()}")
        print(what, flush=True)

        x = rng.standard_normal((n, feat)).astype(np.float32)
        if bf16_in:
            x = bf16_round(x)
        deg = rng.integers(1, 50, n).astype(np.float32)        # the degrees are an input of their own (cu:254)
        base = torch.full((n, ld), 3.0, dtype=torch.bfloat16 if bf16_in else torch.float32, device="cuda")   # padding: junk
        base[:, :feat] = torch.from_numpy(x).cuda()
        xt = base[:, :feat]
        if normalized:
            lay.set_degrees(torch.from_numpy(deg).cuda())
        got = lay.aggregate(xt, normalized=normalized, bias=None if bias is None else torch.from_numpy(bias).cuda(),
                            relu=relu, out_dtype=torch.bfloat16 if bf16_out else None, self_weight=self_weight,
                            pad_columns=pad)
        assert got.dtype == (torch.bfloat16 if bf16_out else torch.float32) and got.shape == (n, feat)
        got = got.float().cpu().numpy().astype(np.float64)

        rs = oracle.rsqrt_rn(deg).astype(np.float64) if normalized else np.ones(n)
        x64 = x.astype(np.float64)
        rows = np.repeat(np.arange(n), np.diff(ip))
        want, mag = np.zeros((n, feat)), np.zeros((n, feat))
        np.add.at(want, rows, x64[ix] * rs[ix, None])
        np.add.at(mag, rows, np.abs(x64[ix]) * rs[ix, None])
        want, mag = want * rs[:, None], mag * rs[:, None]
        want, mag = want + self_weight * x64, mag + abs(self_weight) * np.abs(x64)
        if bias is not None:
            want, mag = want + bias, mag + np.abs(bias)
        if relu:
            want = np.maximum(want, 0.0)
        close_fp32(got, want, mag, extra=2.0 ** -8 * np.abs(want) if bf16_out else None, what=what)
