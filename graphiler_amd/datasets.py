"""Seeded synthetic workloads (host, numpy).

The reference loads its graphs through DGL / OGB downloads
(python/graphiler/utils/setup.py:22-113) and fills features with ``torch.rand``
(setup.py:85); neither the datasets nor DGL are available offline, so the
benchmark configurations are generated here with fixed seeds.  Everything is a
pure function of its arguments and ``numpy.random.default_rng(seed)``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np


@dataclass
class Workload:
    name: str
    num_nodes: int
    src: np.ndarray                      # int64 (E,), edge-id order
    dst: np.ndarray                      # int64 (E,)
    etype: Optional[np.ndarray] = None   # int64 (E,), non-decreasing
    ntype: Optional[np.ndarray] = None   # int64 (N,), non-decreasing
    num_etypes: int = 0
    num_ntypes: int = 0
    meta: Dict[str, object] = field(default_factory=dict)

    @property
    def num_edges(self) -> int:
        return int(self.src.shape[0])


def glorot(rng, shape, fan_in=None, fan_out=None, dtype=np.float32):
    """Glorot-uniform: U(-a, a), a = sqrt(6 / (fan_in + fan_out))."""
    fan_in = shape[-2] if fan_in is None else fan_in
    fan_out = shape[-1] if fan_out is None else fan_out
    a = np.sqrt(6.0 / (fan_in + fan_out))
    return rng.uniform(-a, a, size=shape).astype(dtype)


def sort_by_dst(src, dst):
    """Reorder an edge list so that edge ids are in-adjacency slot numbers."""
    order = np.argsort(dst, kind="stable")
    return src[order], dst[order]


def rmat_edges(rng, scale: int, n_edges: int, a: float, b: float, c: float,
               num_nodes: int, chunk: int = 1 << 24):
    """R-MAT edge list on 2^scale ids folded modulo ``num_nodes`` (duplicates
    and self loops kept).  Quadrants: a -> (0,0), b -> (0,1), c -> (1,0),
    d = 1-a-b-c -> (1,1) for the (src, dst) bit pair at every level."""
    src = np.empty(n_edges, np.int64)
    dst = np.empty(n_edges, np.int64)
    for lo in range(0, n_edges, chunk):
        hi = min(lo + chunk, n_edges)
        s = np.zeros(hi - lo, np.int64)
        d = np.zeros(hi - lo, np.int64)
        for _ in range(scale):
            r = rng.random(hi - lo, dtype=np.float32)
            sbit = r >= (a + b)
            dbit = ((r >= a) & (r < a + b)) | (r >= a + b + c)
            s = (s << 1) | sbit
            d = (d << 1) | dbit
        src[lo:hi] = s % num_nodes
        dst[lo:hi] = d % num_nodes
    return src, dst


def gcn_uniform(num_nodes=19717, n_edges=88651, seed=0) -> Workload:
    """Config 1: uniform random directed graph plus one self loop per node."""
    rng = np.random.default_rng(seed)
    src = rng.integers(0, num_nodes, n_edges, dtype=np.int64)
    dst = rng.integers(0, num_nodes, n_edges, dtype=np.int64)
    loops = np.arange(num_nodes, dtype=np.int64)
    src, dst = sort_by_dst(np.concatenate([src, loops]),
                           np.concatenate([dst, loops]))
    return Workload("gcn_uniform", num_nodes, src, dst)


def gat_rmat(num_nodes=232965, n_edges=11_600_000, scale=18, seed=1,
             self_loops=False, name="gat_rmat") -> Workload:
    """Configs 2 and 5: power-law R-MAT graph (a=.57, b=.19, c=.19), stored by
    destination so edge ids are in-adjacency slots."""
    rng = np.random.default_rng(seed)
    src, dst = rmat_edges(rng, scale, n_edges, 0.57, 0.19, 0.19, num_nodes)
    if self_loops:
        loops = np.arange(num_nodes, dtype=np.int64)
        src = np.concatenate([src, loops])
        dst = np.concatenate([dst, loops])
    src, dst = sort_by_dst(src, dst)
    return Workload(name, num_nodes, src, dst)


def gat_rmat_large(seed=4) -> Workload:
    """Config 5: 2,449,029 nodes, 61,859,140 R-MAT edges plus self loops."""
    return gat_rmat(2_449_029, 61_859_140, 22, seed, True, "gat_rmat_large")


def rgcn_zipf(num_nodes=100_000, n_edges=1_000_000, n_rel=60, s=1.1,
              seed=2) -> Workload:
    """Config 3: uniform endpoints, relation ~ Zipf(s) truncated to n_rel,
    edges sorted by relation (edge ids of one relation contiguous)."""
    rng = np.random.default_rng(seed)
    src = rng.integers(0, num_nodes, n_edges, dtype=np.int64)
    dst = rng.integers(0, num_nodes, n_edges, dtype=np.int64)
    p = np.arange(1, n_rel + 1, dtype=np.float64) ** (-s)
    p /= p.sum()
    etype = rng.choice(n_rel, size=n_edges, p=p).astype(np.int64)
    order = np.argsort(etype, kind="stable")
    return Workload("rgcn_zipf", num_nodes, src[order], dst[order],
                    etype=etype[order], num_etypes=n_rel)


def hgt_hetero(counts=(40_000, 30_000, 20_000, 10_000), n_etypes=10,
               edges_per_type=200_000, alpha=2.1, seed=3) -> Workload:
    """Config 4: node types contiguous; edge type t joins a fixed
    (source type, destination type) pair; sources follow a power-law
    out-degree (rank popularity r^(-1/(alpha-1)) inside the source type),
    destinations are uniform inside the destination type."""
    rng = np.random.default_rng(seed)
    counts = np.asarray(counts, dtype=np.int64)
    nt = len(counts)
    start = np.concatenate([[0], np.cumsum(counts)])
    num_nodes = int(start[-1])
    ntype = np.repeat(np.arange(nt, dtype=np.int64), counts)
    pairs = [(t % nt, (t * 3 + 1) % nt) for t in range(n_etypes)]
    srcs, dsts = [], []
    for st, dt in pairs:
        n_s = int(counts[st])
        pop = np.arange(1, n_s + 1, dtype=np.float64) ** (-1.0 / (alpha - 1.0))
        pop /= pop.sum()
        ranks = rng.permutation(n_s)
        s = ranks[rng.choice(n_s, size=edges_per_type, p=pop)] + start[st]
        d = rng.integers(0, int(counts[dt]), edges_per_type) + start[dt]
        srcs.append(s.astype(np.int64))
        dsts.append(d.astype(np.int64))
    etype = np.repeat(np.arange(n_etypes, dtype=np.int64), edges_per_type)
    return Workload("hgt_hetero", num_nodes, np.concatenate(srcs),
                    np.concatenate(dsts), etype=etype, ntype=ntype,
                    num_etypes=n_etypes, num_ntypes=nt,
                    meta={"type_pairs": pairs})


def debug_graph() -> Workload:
    """The reference's three-node "debug" graph (setup.py:41-42)."""
    return Workload("debug", 3, np.array([0, 0, 0, 1, 1, 2], np.int64),
                    np.array([0, 1, 2, 1, 2, 2], np.int64))


def debug_hetero_graph() -> Workload:
    """The reference's "debug_hetero" graph (setup.py:73-81) flattened to one
    id space: users 0..2, movies 3..4; relations in the order listed there."""
    rel = [
        ([0, 0, 1], [0, 1, 0], 0, 1),   # user  +1 movie
        ([1, 2, 2], [1, 0, 1], 0, 1),   # user  -1 movie
        ([0], [1], 0, 0),               # user  +1 user
        ([2], [1], 0, 0),               # user  -1 user
        ([0], [1], 1, 1),               # movie +1 movie
        ([1], [0], 1, 1),               # movie -1 movie
    ]
    base = [0, 3]
    src, dst, et = [], [], []
    for t, (s, d, st, dt) in enumerate(rel):
        src += [x + base[st] for x in s]
        dst += [x + base[dt] for x in d]
        et += [t] * len(s)
    return Workload("debug_hetero", 5, np.array(src, np.int64),
                    np.array(dst, np.int64), etype=np.array(et, np.int64),
                    ntype=np.array([0, 0, 0, 1, 1], np.int64), num_etypes=6,
                    num_ntypes=2)
