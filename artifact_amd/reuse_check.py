"""Where does reuse pay, and does the cost model that decides it choose well?

    python -m artifact_amd.reuse_check [--nodes 1048576] [--feat 64] [--workloads c1,c2,c3,c3:2,c4] [--out table.md]

Upstream always executes the plan it found (reuse_conv_kernel.cu:876-952); this library first prices it: a plan whose
net saving is under a tenth of all row gathers (or under 256 MB) is folded back into the reuse-disabled schedule, and
clusters of destinations that share groups are kept only if they save an eighth of their rows' gathers.  Those gates
were set on the five workload graphs and one planted-reuse graph.  This check sweeps graphs with planted shared
neighbour sets from 80 % down to a few per cent of removable gathers (sets of `set_size` anchors shared by
`members` nodes each, plus `extra` random neighbours per node; also nodes that belong to two or three sets with
different club mates) and times the same plan (upstream search, part size 3)
four ways, in turn: as the library would run it by default, with reuse disabled, with every shared group forced
through LDS clusters, and with every group of two or more consumers forced through workspace rows.  The last column
is the default's time over the best of the four: 1.00 means the gates chose the fastest.  `--workloads` puts the named
workload graphs (at their own widths) through the same comparison.  Needs a GPU.
"""
from __future__ import annotations

import argparse
import sys
import time

import numpy as np

from . import reuse_search_ext as R
from .graphgen import WORKLOADS, csr_from_pairs, make_workload, planted_reuse_csr, rmat_csr
from .layout import Layout, lanes_per_row
from .tune_check import time_round_robin

# (set_size, members per set, extra random neighbours per node[, sets per node: with more than one a node's club mates
# differ from set to set, so its sets cannot all be shared inside one workgroup])
CASES = ((12, 64, 4), (12, 64, 24), (12, 8, 24), (12, 2, 12), (6, 64, 24), (6, 4, 24), (3, 64, 24), (3, 64, 48), (3, 4, 24),
         (3, 2, 24), (12, 8, 12, 2), (6, 16, 12, 2), (3, 16, 24, 2), (3, 64, 24, 3), "mixed")


def mixed_csr(nodes, seed):
    """A heavy-tailed R-MAT graph (average degree 16) whose upper half of the ids also carries planted sets (6 anchors
    x 16 members): rows with hubs and rows with shared neighbour sets in one graph."""
    a_ptr, a_idx = rmat_csr(nodes, 16, seed)
    b_ptr, b_idx = planted_reuse_csr(nodes // 2, 6, 16, 0, seed=seed + 1)
    ua = np.repeat(np.arange(nodes, dtype=np.int64), np.diff(a_ptr))
    ub = np.repeat(np.arange(nodes // 2, dtype=np.int64), np.diff(b_ptr)) + nodes // 2
    return csr_from_pairs(np.concatenate([ua, ub]), np.concatenate([a_idx.astype(np.int64), b_idx.astype(np.int64) + nodes // 2]),
                          nodes, False)


def check(case, nodes, feat, part_size=3, log=print):
    """`case`: (set_size, members, extra) of a planted graph of `nodes` nodes, or the name of a workload."""
    import torch

    t0 = time.time()
    if case == "mixed":
        ip, ix = mixed_csr(nodes, 95)
        label = "R-MAT of degree 16 + planted sets 6 x 16 on half of the nodes"
    elif isinstance(case, str):
        case, _, ps = case.partition(":")              # "c3:2" = workload c3 at part size 2
        part_size = int(ps) if ps else part_size
        ip, ix = make_workload(case)
        feat = WORKLOADS[case]["dims"][-1] if case != "c2" else WORKLOADS[case]["dims"][1]
        label = f"workload {case}, {feat} floats, part size {part_size}"
    else:
        set_size, members, extra = case[:3]
        sets = case[3] if len(case) > 3 else 1
        ip, ix = planted_reuse_csr(nodes, set_size, members, extra, seed=90 + set_size + members + extra, memberships=sets)
        label = f"{set_size} x {members} + {extra}" + (f", {sets} sets per node" if sets > 1 else "")
    n, e = len(ip) - 1, len(ix)
    plan = R.build_plan(ip, ix, part_size)
    v2 = (plan["uniqpart_column_index"], plan["uniqpart_pointers"], plan["part2Node_ptr"], plan["part2Node_col"], n, part_size)
    lpr = lanes_per_row(feat)
    common = dict(lanes_per_row=lpr, row_bytes=feat * 4)
    lays = {
        "default": Layout.from_v2(*v2, **common),
        "reuse disabled": Layout.from_v2(*v2, disable_reuse=True, **common),
        "clusters forced": Layout.from_v2(*v2, local_groups=1, **common),
        "workspace forced": Layout.from_v2(*v2, min_consumers=2, local_groups=-1, **common),
    }
    st = {k: lay.stats() for k, lay in lays.items()}
    # gross share of the graph's row gathers that the plan can remove: every consumer of a picked part but one
    removable = 1.0 - len(plan["uniqpart_column_index"]) / max(1, e)
    x = torch.randn((n, -(-feat // 4) * 4), device="cuda")[:, :feat]
    out = torch.empty((n, feat), device="cuda")
    res = time_round_robin({k: (lay, {}) for k, lay in lays.items()}, x, feat, out, rounds=3, iters=8)
    outs = {}
    for k, lay in lays.items():
        outs[k] = lay.aggregate(x, normalized=False, feat_dim=feat).clone()
    worst = max(float((outs[k] - outs["reuse disabled"]).abs().max()) for k in outs)
    for lay in lays.values():
        lay.close()
    d = st["default"]
    how = ("clusters" if d["cluster_workgroups"] else "") + ("+workspace" if d["materialised_groups"] else "")
    how = how.lstrip("+") or "folded"
    best = min(res, key=res.get)
    log(f"[reuse_check] {label}: {n} nodes, {e} edges, removable "
        f"{100 * removable:.1f} %, default runs {how}: " + ", ".join(f"{k} {v:.4f}" for k, v in res.items())
        + f" ms; best {best}; default / best {res['default'] / res[best]:.3f} ({time.time() - t0:.0f} s)")
    return dict(case=case, label=label, n=n, e=e, removable=removable, how=how, res=res, best=best, ratio=res["default"] / res[best],
                max_diff=worst,
                lds_reads=d["lds_reads"], materialised=d["materialised_groups"])


def table(rows):
    cols = ["default", "reuse disabled", "clusters forced", "workspace forced"]
    lines = ["| anchors per set x members + random neighbours | edges | removable gathers | default runs | "
             + " | ".join(cols) + " | reuse disabled / best | best | default / best |", "|" + "---|" * (len(cols) + 7)]
    for r in rows:
        best = r["res"][r["best"]]
        lines.append(f"| {r['label']} | {r['e'] / 1e6:.1f} M | {100 * r['removable']:.1f} % | {r['how']} | "
                     + " | ".join(f"{r['res'][c]:.4f}" for c in cols)
                     + f" | {r['res']['reuse disabled'] / best:.2f} | {r['best']} | {r['ratio']:.3f} |")
    return "\n".join(lines)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--nodes", type=int, default=1 << 20)
    ap.add_argument("--feat", type=int, default=64)
    ap.add_argument("--workloads", default="", help="named workloads to add, e.g. c1,c2,c3,c3:2,c4 (name:part size)")
    ap.add_argument("--out", default="")
    args = ap.parse_args()
    log = lambda *a: print(*a, file=sys.stderr, flush=True)
    rows = [check(c, args.nodes, args.feat, log=log) for c in CASES]
    rows += [check(w, 0, 0, log=log) for w in args.workloads.split(",") if w]
    text = (f"ms per aggregation layer (sum aggregation; planted graphs: {args.nodes} nodes, {args.feat} floats; upstream search at part size 3; "
            "the four layouts of a row are timed in turn, 3 rounds of 8 calls, median of the rounds; all four give the same sums "
            f"to {max(r['max_diff'] for r in rows):.1e}).\n\n" + table(rows) + "\n")
    print(text)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text)


if __name__ == "__main__":
    main()
