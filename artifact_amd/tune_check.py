"""Held-out check of the launch heuristics: on graphs and widths that were not used to tune them, is the library's
own choice of wavefront cap, XCD run, row gathers in flight and long-row cut within a few per cent of the best of
the alternatives?

    python -m artifact_amd.tune_check [--graphs h1,...,h13] [--out table.md]

For every (graph, width) one aggregation layer (no reuse plan: `Layout.from_csr`) is timed with the default layout
and launch settings and then with one setting changed at a time: wavefronts per SIMD of the destination-row launch
8 / 7 / 6, runs of 4 / 16 / 256 workgroups per XCD, two and four row gathers in flight, and the long-row cut halved,
doubled and quadrupled; and with the layout that `LayoutFamily(autotune=True)` picks by timing.  Prints a markdown table; the last column is the default's time over
the best time of the row.  Needs a GPU; graphs are generated on the host (a few seconds each).
"""
from __future__ import annotations

import argparse
import sys
import time

import numpy as np

from .graphgen import csr_from_pairs, rmat_csr, sbm_csr
from .layout import Layout, LayoutFamily, lanes_per_row


def uniform_degree_csr(num_nodes, degree, seed):
    """Every node draws `degree` / 2 random partners: degrees concentrate around `degree`, no hubs."""
    rng = np.random.Generator(np.random.PCG64(seed))
    u = np.repeat(np.arange(num_nodes, dtype=np.int64), degree // 2)
    v = rng.integers(0, num_nodes, size=len(u))
    return csr_from_pairs(u, v, num_nodes, False)


def grid_csr(rows, cols):
    """4-neighbour grid, ids row-major: every source is 1 or `cols` ids away."""
    ids = np.arange(rows * cols, dtype=np.int64).reshape(rows, cols)
    u = np.concatenate([ids[:, :-1].ravel(), ids[:-1, :].ravel()])
    v = np.concatenate([ids[:, 1:].ravel(), ids[1:, :].ravel()])
    return csr_from_pairs(u, v, rows * cols, False)


def banded_csr(num_nodes, degree, band, seed):
    """`degree` / 2 random partners per node within `band` ids of it (a nearest-neighbour graph of sorted points)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    u = np.repeat(np.arange(num_nodes, dtype=np.int64), degree // 2)
    v = (u + rng.integers(-band, band + 1, size=len(u))) % num_nodes
    return csr_from_pairs(u, v, num_nodes, False)


def bipartite_csr(users, items, per_user, seed):
    """Users (ids 0 .. users-1) each link to `per_user` items (ids users ..), item popularity ~ 1 / rank: two kinds of
    rows, short user rows that gather from a small popular set and long item rows that gather from everywhere."""
    rng = np.random.Generator(np.random.PCG64(seed))
    u = np.repeat(np.arange(users, dtype=np.int64), per_user)
    p = 1.0 / np.arange(1, items + 1)
    v = users + rng.choice(items, size=len(u), p=p / p.sum())
    return csr_from_pairs(u, v, users + items, False)


GRAPHS = {
    "h1": ("R-MAT a=.45 b=c=.22, 2^21 nodes, average degree 8", lambda: rmat_csr(1 << 21, 8, 71, a=0.45, b=0.22, c=0.22)),
    "h2": ("R-MAT a=.65 b=c=.15, 2^20 nodes, average degree 48", lambda: rmat_csr(1 << 20, 48, 72, a=0.65, b=0.15, c=0.15)),
    "h3": ("uniform degrees (16 random partners per node), 2^21 nodes", lambda: uniform_degree_csr(1 << 21, 16, 73)),
    "h4": ("block model, 2048 blocks of 1024 nodes, degree 16 inside + 4 outside", lambda: sbm_csr(2048, 1024, 16, 4, 74)),
    # small launches: bound by their longest chain of dependent gathers, not by the memory side
    "h5": ("R-MAT a=.5 b=c=.2, 2^16 nodes, average degree 24", lambda: rmat_csr(1 << 16, 24, 75, a=0.5, b=0.2, c=0.2)),
    "h6": ("R-MAT a=.62 b=c=.16, 2^15 nodes, average degree 12", lambda: rmat_csr(1 << 15, 12, 76, a=0.62, b=0.16, c=0.16)),
    "h7": ("R-MAT a=.55 b=.25 c=.15, 2^17 nodes, average degree 6", lambda: rmat_csr(1 << 17, 6, 77, a=0.55, b=0.25, c=0.15)),
    # dense graphs: every row is near or beyond the long-row cut
    "h8": ("uniform degrees (600 random partners per node), 2^17 nodes", lambda: uniform_degree_csr(1 << 17, 600, 78)),
    "h9": ("R-MAT a=.5 b=c=.2, 2^16 nodes, average degree 400", lambda: rmat_csr(1 << 16, 400, 79, a=0.5, b=0.2, c=0.2)),
    # very sparse graphs with local structure
    "h10": ("4-neighbour grid 2048 x 2048", lambda: grid_csr(2048, 2048)),
    "h11": ("16 random partners within 32768 ids, 2^21 nodes", lambda: banded_csr(1 << 21, 16, 1 << 15, 80)),
    "h12": ("bipartite: 2^20 users x 16 of 2^15 items, popularity 1 / rank", lambda: bipartite_csr(1 << 20, 1 << 15, 16, 81)),
    # dense without a popular set of sources that one L2 could hold
    "h13": ("R-MAT a=.5 b=c=.2, 233 000 nodes, average degree 435", lambda: rmat_csr(233_000, 480, 91, a=0.5, b=0.2, c=0.2)),
}
WIDTHS = ((24, False), (72, False), (160, False), (128, True))


def time_round_robin(variants, x, feat, out, rounds=3, iters=8):
    """{label: ms}: every variant is timed once per round, in turn, so that warm-up and clock drift hit all alike;
    the figure of a variant is the median of its rounds.  `variants`: label -> (layout, tuning dict)."""
    for lay, tune in variants.values():                     # upload and warm up
        lay.set_tuning(**tune)
        lay.aggregate(x, normalized=False, out=out, feat_dim=feat)
    ms = {k: [] for k in variants}
    for _ in range(rounds):
        for k, (lay, tune) in variants.items():
            lay.set_tuning(**tune)
            ms[k].append(lay.aggregate_timed(x, iters, normalized=False, out=out, feat_dim=feat)[0])
    return {k: float(np.median(v)) for k, v in ms.items()}


def check(name, widths=WIDTHS, log=print):
    import torch

    descr, make = GRAPHS[name]
    t0 = time.time()
    ip, ix = make()
    n, e = len(ip) - 1, len(ix)
    deg = np.diff(ip)
    log(f"[tune_check] {name}: {descr}: {n} nodes, {e} edges ({time.time() - t0:.1f} s)")
    rows = []
    for feat, bf16 in widths:
        lpr, eb = lanes_per_row(feat, bf16), 2 if bf16 else 4
        mult = 8 if bf16 else 4
        ld = -(-feat // mult) * mult
        x = torch.randn((n, ld), device="cuda").to(torch.bfloat16 if bf16 else torch.float32)[:, :feat]
        out = torch.empty((n, feat), device="cuda")
        rb = feat * eb
        base = Layout.from_csr(ip, ix, lanes_per_row=lpr, elem_bytes=eb, row_bytes=rb)
        cut = base.stats()["hub_split"]
        variants = {"default": (base, {})}
        for cap in (0, 7, 6):
            variants[f"waves {cap or 8}"] = (base, dict(wave_cap=cap))
        for run in (4, 16, 256):
            variants[f"xcd run {run}"] = (base, dict(xcd_run_dst=run))
        if not bf16:
            for deep in (0, 1):
                variants[f"in flight {4 if deep else 2}"] = (base, dict(deep=deep))
        others = []
        for factor, label in ((0.5, "cut / 2"), (2.0, "cut x 2"), (4.0, "cut x 4")):
            lay = Layout.from_csr(ip, ix, lanes_per_row=lpr, elem_bytes=eb, row_bytes=rb, hub_split=max(16, int(cut * factor)))
            variants[label] = (lay, {})
            others.append(lay)
        # what a family picks when it times its candidates (cut of long rows, then launch settings)
        fam = LayoutFamily(lambda l, e_, r=0, **kw: Layout.from_csr(ip, ix, lanes_per_row=l, elem_bytes=e_, row_bytes=r, **kw),
                           autotune=True)
        tuned = fam.get(feat, bf16, normalized=False)
        variants["autotuned"] = (tuned, tuned.tuning())
        res = time_round_robin(variants, x, feat, out, iters=8 if n >= 1 << 19 else 40)
        picked = next(iter(fam.chosen.values()))
        fam.close()
        for lay in others + [base]:
            lay.close()
        best = min((k for k in res if k != "autotuned"), key=res.get)
        share = float(deg[deg > cut].sum()) / max(1, e)
        rows.append((name, f"{feat} {'bf16' if bf16 else 'fp32'}", res, best, res["default"] / res[best], cut, share,
                     f"{picked['cut']}/{picked['segment']}", res["autotuned"] / res[best]))
        log(f"[tune_check]   width {feat}{' bf16' if bf16 else ''}: cut {cut} ({100 * share:.0f} % of the edges in longer rows), "
            f"default {res['default']:.4f} ms, best {best} {res[best]:.4f} ms ({res['default'] / res[best]:.3f}x); autotuned "
            f"{picked['cut']}/{picked['segment']} {picked['tuning']} {res['autotuned']:.4f} ms ({res['autotuned'] / res[best]:.3f}x)")
        del x, out
    return rows


def table(rows):
    cols = ["default", "waves 8", "waves 7", "waves 6", "xcd run 4", "xcd run 16", "xcd run 256", "in flight 2", "in flight 4",
            "cut / 2", "cut x 2", "cut x 4"]
    lines = ["| graph | width | cut (edges in longer rows) | " + " | ".join(cols) + " | best | default / best | autotuned "
             "(cut/segment) | autotuned / best |", "|" + "---|" * (len(cols) + 7)]
    for name, width, res, best, ratio, cut, share, picked, tuned_ratio in rows:
        cells = [f"{res[c]:.4f}" if c in res else "" for c in cols]
        lines.append(f"| {name} | {width} | {cut} ({100 * share:.0f} %) | " + " | ".join(cells) + f" | {best} | {ratio:.3f} | "
                     f"{res['autotuned']:.4f} ({picked}) | {tuned_ratio:.3f} |")
    return "\n".join(lines)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--graphs", default=",".join(GRAPHS))
    ap.add_argument("--out", default="")
    args = ap.parse_args()
    rows = []
    for g in args.graphs.split(","):
        rows += check(g, log=lambda *a: print(*a, file=sys.stderr, flush=True))
    note = ("ms per aggregation layer (sum aggregation, no reuse plan; the variants of a row are timed in turn, 3 rounds "
            "of 8 calls each -- 40 on graphs under 2^19 nodes --, median of the rounds); one setting changed at a time.")
    text = "\n".join(f"* {k}: {GRAPHS[k][0]}" for k in args.graphs.split(",")) + "\n\n" + note + "\n\n" + table(rows) + "\n"
    print(text)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text)


if __name__ == "__main__":
    main()
