"""Seeded synthetic graphs and features for the aggregation workloads.

The upstream drivers load Planetoid/OGB datasets through a `data_prepare.load_graph`
that is not part of the upstream tree (ROF_evaluation/ROF_main.py:26,40-46) and then
build a CSR with scipy (ROF_main.py:50-64).  These generators produce the same kind of
object -- a symmetric, duplicate-free CSR with sorted int32 columns -- without a network.

Everything here is plain numpy on the host; it is input preparation, not the hot path.
"""
from __future__ import annotations

import numpy as np

__all__ = ["rmat_csr", "sbm_csr", "planted_reuse_csr", "csr_from_pairs", "features", "glorot", "WORKLOADS", "make_workload"]


def csr_from_pairs(u, v, num_nodes, self_loops=False):
    """Symmetrise (A or A^T), drop duplicates, optionally add self loops.

    Returns (indptr int32[N+1], indices int32[E]) with sorted columns per row, the layout
    scipy's coo->csr conversion yields at ROF_main.py:53-60 (values are ignored upstream).
    Self loops drawn by the generator are kept only if `self_loops` is set.
    """
    u = np.asarray(u, dtype=np.int64)
    v = np.asarray(v, dtype=np.int64)
    keep = u != v
    u, v = u[keep], v[keep]
    n = np.int64(num_nodes)
    keys = np.concatenate([u * n + v, v * n + u])
    if self_loops:
        d = np.arange(num_nodes, dtype=np.int64)
        keys = np.concatenate([keys, d * n + d])
    keys = np.unique(keys)
    rows = keys // n
    cols = (keys - rows * n).astype(np.int32)
    counts = np.bincount(rows, minlength=num_nodes)
    indptr = np.zeros(num_nodes + 1, dtype=np.int64)
    np.cumsum(counts, out=indptr[1:])
    assert indptr[-1] < 2**31, "edge count must fit int32 indexing"
    return indptr.astype(np.int32), cols


def _rmat_pairs(rng, scale, m, a, b, c):
    u = np.zeros(m, dtype=np.int64)
    v = np.zeros(m, dtype=np.int64)
    ab = a + b
    abc = a + b + c
    for _ in range(scale):
        r = rng.random(m, dtype=np.float32)
        ubit = r >= ab                      # quadrants c, d -> row bit 1
        vbit = ((r >= a) & (r < ab)) | (r >= abc)   # quadrants b, d -> col bit 1
        u = (u << 1) | ubit
        v = (v << 1) | vbit
    return u, v


def rmat_csr(num_nodes, avg_degree, seed, a=0.57, b=0.19, c=0.19, self_loops=False, distinct_pairs=False):
    """R-MAT(a,b,c,d) graph on `num_nodes` ids inside a 2^ceil(log2 N) id space.

    Draws N*avg_degree/2 undirected pairs; pairs with an endpoint >= N are dropped and
    the draw is topped up until that many in-range pairs exist (matters only when N is
    not a power of two).  With `distinct_pairs` the draw goes on until that many *distinct*
    undirected pairs (no self pairs) remain after de-duplication, so the stored graph has
    exactly N*avg_degree directed edges (the 2.4 M-node workload is specified by its edge
    count after symmetrisation, the power-of-two ones by the number of pairs drawn).
    """
    rng = np.random.Generator(np.random.PCG64(seed))
    scale = int(np.ceil(np.log2(num_nodes)))
    want = int(num_nodes * avg_degree // 2)
    oversample = 1 if (1 << scale) == num_nodes else 1.6
    if distinct_pairs:
        n = np.int64(num_nodes)
        keys = np.empty(0, dtype=np.int64)      # distinct pairs so far, as min*N+max, ascending
        yield_ = 0.7 / oversample               # distinct new pairs per draw, re-estimated after every batch
        while len(keys) < want:
            short = want - len(keys)
            # large batches aim 3 % below the target so that only a small last batch has to be trimmed
            m = max(4096, int((short * 0.97 if short > 100000 else short * 1.5) / yield_))
            u, v = _rmat_pairs(rng, scale, m, a, b, c)
            ok = (u < num_nodes) & (v < num_nodes) & (u != v)
            k = np.minimum(u[ok], v[ok]) * n + np.maximum(u[ok], v[ok])
            del u, v, ok
            fresh = np.setdiff1d(k, keys)       # sorted, distinct
            yield_ = max(len(fresh), 1) / m
            if len(fresh) > short:              # overshoot: keep the pairs that were drawn first
                f2, first = np.unique(k, return_index=True)
                first = first[np.isin(f2, fresh, assume_unique=True)]
                fresh = fresh[np.argsort(first, kind="stable")[:short]]
            keys = np.union1d(keys, fresh)
        return csr_from_pairs(keys // n, keys % n, num_nodes, self_loops)
    us, vs, have = [], [], 0
    while have < want:
        m = max(1024, int((want - have) * 1.05 * oversample))
        u, v = _rmat_pairs(rng, scale, m, a, b, c)
        ok = (u < num_nodes) & (v < num_nodes)
        u, v = u[ok][: want - have], v[ok][: want - have]
        us.append(u)
        vs.append(v)
        have += len(u)
    return csr_from_pairs(np.concatenate(us), np.concatenate(vs), num_nodes, self_loops)


def sbm_csr(num_blocks, block_size, deg_in, deg_out, seed, self_loops=False):
    """Stochastic block model with equal blocks, sampled by edge counts (never O(N^2)).

    Expected intra-block degree `deg_in`, expected inter-block degree `deg_out`.
    """
    rng = np.random.Generator(np.random.PCG64(seed))
    n = num_blocks * block_size
    m_in = rng.binomial(block_size * (block_size - 1) // 2, deg_in / (block_size - 1), size=num_blocks)
    us, vs = [], []
    for blk, m in enumerate(m_in):
        base = blk * block_size
        us.append(base + rng.integers(0, block_size, size=m))
        vs.append(base + rng.integers(0, block_size, size=m))
    m_out = int(rng.binomial(n * (n - block_size) // 2, deg_out / (n - block_size)))
    u = rng.integers(0, n, size=m_out)
    v = rng.integers(0, n - block_size, size=m_out)
    v = v + np.where(v >= (u // block_size) * block_size, block_size, 0)   # skip u's own block
    us.append(u)
    vs.append(v)
    return csr_from_pairs(np.concatenate(us), np.concatenate(vs), n, self_loops)


def planted_reuse_csr(num_nodes, set_size=12, members_per_set=64, extra_degree=4, seed=0, memberships=1):
    """Graph with planted common-neighbour structure: nodes come in clubs of `members_per_set`; every
    member of a club is linked to the same `set_size` anchor nodes (consecutive ids, so the chunks of a
    member's sorted neighbour list coincide with those of its club mates), plus `extra_degree` random
    neighbours.  With `memberships` > 1 every node also joins that many minus one further clubs, drawn by random
    permutations of the members: its club mates then differ from set to set, so no ordering of the nodes brings all
    consumers of every set together.  Symmetric, duplicate-free.  Not one of the upstream-style workloads: it exists
    to show what the reuse plan buys when a graph does contain shared neighbour subsets."""
    rng = np.random.Generator(np.random.PCG64(seed))
    clubs = max(1, num_nodes // (members_per_set + set_size))
    n_anchor = clubs * set_size
    members = np.arange(n_anchor, num_nodes, dtype=np.int64)
    us, vs = [], []
    for k in range(max(1, memberships)):
        order = members - n_anchor if k == 0 else rng.permutation(len(members))
        club = order % clubs
        us.append(np.repeat(members, set_size))
        vs.append(np.repeat(club * set_size, set_size) + np.tile(np.arange(set_size), len(members)))
    ru = rng.integers(n_anchor, num_nodes, size=len(members) * extra_degree // 2)
    rv = rng.integers(n_anchor, num_nodes, size=len(ru))
    return csr_from_pairs(np.concatenate(us + [ru]), np.concatenate(vs + [rv]), num_nodes, False)


def features(num_nodes, dim, seed, kind="normal"):
    rng = np.random.Generator(np.random.PCG64(seed))
    if kind == "normal":
        return rng.standard_normal((num_nodes, dim), dtype=np.float32)
    if kind == "uniform":
        return (rng.random((num_nodes, dim), dtype=np.float32) * 2.0 - 1.0).astype(np.float32)
    raise ValueError(kind)


def glorot(fan_in, fan_out, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    bound = np.sqrt(6.0 / (fan_in + fan_out))
    return ((rng.random((fan_in, fan_out), dtype=np.float32) * 2.0 - 1.0) * bound).astype(np.float32)


# name -> (graph builder kwargs, aggregated width, description); seeds are 1000/2000/3000 + index.
WORKLOADS = {
    "c1": dict(kind="rmat", num_nodes=1 << 14, avg_degree=16, self_loops=True, seed=1001, dims=(32, 32)),
    "c2": dict(kind="rmat", num_nodes=1 << 18, avg_degree=14, self_loops=True, seed=1002, dims=(128, 256, 40)),
    "c3": dict(kind="sbm", num_blocks=256, block_size=4096, deg_in=24, deg_out=2, self_loops=False, seed=1003,
               dims=(64, 64)),
    # specified by its edge count after symmetrisation (~62 M directed): the draw is topped up after de-duplication
    "c4": dict(kind="rmat", num_nodes=2_400_000, avg_degree=26, self_loops=False, seed=1004, dims=(100, 47),
               distinct_pairs=True),
    "c5": dict(kind="rmat", num_nodes=1 << 22, avg_degree=32, self_loops=True, seed=1005, dims=(256, 256)),
    # planted reuse (see planted_reuse_csr): 2^20 nodes, 12 shared anchors + ~4 random neighbours per member
    "hr": dict(kind="planted", num_nodes=1 << 20, set_size=12, members_per_set=64, extra_degree=4, seed=1006,
               dims=(64, 64)),
}


def make_workload(name, scale_down=0):
    """CSR of a named workload; `scale_down` halves the node count that many times
    (same average degree) so the parity tests can run the same shapes at small sizes."""
    w = dict(WORKLOADS[name])
    if w["kind"] == "rmat":
        n = max(64, w["num_nodes"] >> scale_down)
        return rmat_csr(n, w["avg_degree"], w["seed"], self_loops=w["self_loops"],
                        distinct_pairs=w.get("distinct_pairs", False))
    if w["kind"] == "planted":
        n = max(512, w["num_nodes"] >> scale_down)
        return planted_reuse_csr(n, w["set_size"], w["members_per_set"], w["extra_degree"], w["seed"])
    nb = max(2, w["num_blocks"] >> scale_down)
    return sbm_csr(nb, w["block_size"], w["deg_in"], w["deg_out"], w["seed"], self_loops=w["self_loops"])
