"""Model-level benchmark driver, the counterpart of the ``profile`` /
``breakdown`` / ``__main__`` blocks of the reference's examples
(examples/GAT/GAT.py:87-187 and the same blocks of GCN.py, RGCN.py, HGT.py):

    python -m graphiler_amd.examples.run MODEL all                 # every dataset -> output/MODEL.pkl
    python -m graphiler_amd.examples.run MODEL breakdown           # levels 0/1/2 -> output/MODEL_breakdown.pkl
    python -m graphiler_amd.examples.run MODEL DATASET [FEAT_DIM]  # one dataset, printed only

MODEL is GCN, GAT, RGCN or HGT; ``REPEAT`` (environment, default 50) is the
number of timed inferences, as in the reference.  The datasets the reference
downloads (python/graphiler/utils/setup.py:16-19,22-72) are not available
offline: each name maps to a seeded synthetic graph with the published node and
edge counts of that dataset (R-MAT for the homogeneous ones; uniform endpoints
with Zipf-distributed relations and contiguous node types for the knowledge
graphs), so the tables have the reference's rows and columns but not its
graphs.  Tags whose library is absent (DGL, PyG) read -1 = "N/A".
"""
from __future__ import annotations

import os
import sys

import numpy as np
import torch

from .. import datasets, prepare_graph
from ..hipgraph import Graphed
from ..mpdfg import GraphData
from ..report import (is_out_of_memory, bench, check_equal, empty_cache, init_log, mark_unavailable,
                      save_logs)
from . import models

DEFAULT_DIM = 64
RGCN_FEAT_DIM = 16          # examples/RGCN/RGCN.py:19

# name -> (feature width (setup.py:16-17), nodes, directed edges, R-MAT scale)
homo_dataset = {
    "cora": (1433, 2_708, 10_556, 12),
    "pubmed": (500, 19_717, 88_651, 15),
    "ppi": (50, 56_944, 818_716, 16),
    "arxiv": (128, 169_343, 1_166_243, 18),
    "reddit": (602, 232_965, 114_615_892, 18),
}
# name -> (nodes, edges, node types, relations) of the RDF / OGB graphs (setup.py:19)
hetero_dataset = {
    "aifb": (7_262, 48_810, 7, 78),
    "mutag": (27_163, 148_100, 5, 46),
    "bgs": (94_806, 672_884, 27, 206),
    "biokg": (93_773, 4_762_678, 5, 51),
    "am": (881_680, 5_668_682, 7, 96),
}


def load_data(name: str, feat_dim: int = DEFAULT_DIM, device="cuda:0", seed: int = 0):
    """Seeded stand-in for setup.py:22-113: returns (GraphData, features)."""
    rng = np.random.default_rng(seed)
    if name in homo_dataset:
        _, n, e, scale = homo_dataset[name]
        src, dst = datasets.rmat_edges(rng, scale, e, 0.57, 0.19, 0.19, n)
        g = prepare_graph(src, dst, n, device=device)
    elif name in hetero_dataset:
        n, e, n_nt, n_rel = hetero_dataset[name]
        wl = datasets.rgcn_zipf(n, e, n_rel, seed=seed)
        ntype = np.sort(rng.integers(0, n_nt, n)).astype(np.int64)
        g = prepare_graph(wl.src, wl.dst, n, device=device, ntype_of=ntype, num_ntypes=n_nt,
                          etype_of=wl.etype, num_etypes=n_rel)
    else:
        raise KeyError("unknown dataset " + name)
    feats = torch.from_numpy(rng.random((g.num_nodes, feat_dim), dtype=np.float32)).to(device)
    return GraphData(g), feats


def _build(model: str, g: GraphData, feat_dim: int, device):
    """Network and the extra call arguments after (g, features)."""
    G = g.graph
    if model == "GCN":
        return models.GCN(feat_dim, DEFAULT_DIM, DEFAULT_DIM, device), ()
    if model == "GAT":
        return models.GAT(feat_dim, DEFAULT_DIM, DEFAULT_DIM, device), ()
    if model == "RGCN":
        norm = torch.rand(G.num_edges, 1, device=device)
        return models.RGCN(feat_dim, DEFAULT_DIM, feat_dim, G.num_etypes, device), (norm,)
    if model == "HGT":
        return models.HGT(feat_dim, DEFAULT_DIM, DEFAULT_DIM, G.num_ntypes, G.num_etypes,
                          device), ()
    raise KeyError("unknown model " + model)


PROFILE_TAGS = {
    "GCN": ["0-DGL-UDF", "1-DGL-primitives", "2-PyG-primitives", "3-Graphiler"],
    "GAT": ["0-DGL-UDF", "1-DGL-primitives", "2-PyG-primitives", "3-Graphiler"],
    "RGCN": ["0-DGL-UDF", "1-DGL-slice", "2-PyG-slice", "3-DGL-bmm", "4-PyG-bmm", "5-Graphiler"],
    "HGT": ["0-DGL-UDF", "1-DGL-slice", "2-PyG-slice", "3-DGL-bmm", "4-PyG-bmm", "5-Graphiler"],
}
EAGER_TAG = "eager-torch"


def _expected(net, params):
    """Expected result for ``check_equal``: the eager network with float64
    per-destination sums (None when it does not fit in memory)."""
    try:
        return net(*params, "eager64")
    except RuntimeError as err:
        if not is_out_of_memory(err):
            raise
        torch.cuda.empty_cache()
        return None


def profile(model: str, dataset: str, feat_dim: int, repeat: int = 1000, device="cuda:0"):
    """The reference's tags, with the compiled network under its "Graphiler"
    tag and the eager baseline under an extra tag; the compiled result is
    checked against the eager network evaluated with float64 sums."""
    tags = PROFILE_TAGS[model]
    log = init_log(tags + [EAGER_TAG], ["time", "mem"])
    for tag in tags[:-1]:
        mark_unavailable(log, tag)
    print("benchmarking on: " + dataset)

    @empty_cache
    def run(log):
        g, feats = load_data(dataset, feat_dim, device)
        net, extra = _build(model, g, feat_dim, device)
        with torch.no_grad():
            compiled = bench(net, (g, feats) + extra + (2,), tag=tags[-1], repeat=repeat,
                             memory=True, log=log)
            bench(net, (g, feats) + extra + ("eager",), tag=EAGER_TAG, repeat=repeat,
                  memory=True, log=log)
            check_equal(compiled, _expected(net, (g, feats) + extra))

    run(log)
    return log


def breakdown(model: str, dataset: str, feat_dim: int, repeat: int = 1000, device="cuda:0"):
    """examples/GAT/GAT.py:140-163: the eager baseline, then the plan at
    optimisation levels 0, 1 and 2 and the level-2 network replayed as a HIP
    graph; every result is checked against the eager network evaluated with
    float64 sums."""
    log = init_log(["0-" + EAGER_TAG, "1+compile", "2+reorder", "3+fusion", "4+hipgraph"],
                   ["time", "mem"])
    print("benchmarking on: " + dataset)
    torch.cuda.empty_cache()
    g, feats = load_data(dataset, feat_dim, device)
    net, extra = _build(model, g, feat_dim, device)
    with torch.no_grad():
        bench(net, (g, feats) + extra + ("eager",), tag="0-" + EAGER_TAG, repeat=repeat,
              memory=True, log=log)
        base = _expected(net, (g, feats) + extra)
        for level, tag in enumerate(["1+compile", "2+reorder", "3+fusion"]):
            res = bench(net, (g, feats) + extra + (level,), tag=tag, repeat=repeat,
                        memory=True, log=log)
            check_equal(res, base)
        # the level-2 network recorded once and replayed as a single HIP graph
        # (memory of a replay is the graph's own pool, held since the recording)
        graphed = Graphed(net, (g, feats) + extra + (2,))
        res = bench(graphed, (), tag="4+hipgraph", repeat=repeat, memory=False, log=log)
        check_equal(res, base)
    return log


def _sets(model: str):
    if model in ("GCN", "GAT"):
        return {d: homo_dataset[d][0] for d in homo_dataset}
    dim = RGCN_FEAT_DIM if model == "RGCN" else DEFAULT_DIM
    return {d: dim for d in hetero_dataset}


def main(argv):
    repeat = int(os.environ.get("REPEAT", 50))
    if len(argv) not in (3, 4) or argv[1] not in PROFILE_TAGS:
        print("usage: python -m graphiler_amd.examples.run GCN|GAT|RGCN|HGT "
              "all|breakdown|DATASET [FEAT_DIM]")
        return 2
    model, what = argv[1], argv[2]
    out_dir = os.environ.get("GRAPHILER_OUTPUT", "output")
    if what == "all":
        logs = {d: profile(model, d, dim, repeat) for d, dim in _sets(model).items()}
        print("wrote", save_logs(logs, model, out_dir))
    elif what == "breakdown":
        logs = {d: breakdown(model, d, dim, repeat) for d, dim in _sets(model).items()}
        print("wrote", save_logs(logs, model + "_breakdown", out_dir))
    else:
        dim = int(argv[3]) if len(argv) == 4 else _sets(model)[what]
        print(profile(model, what, dim, repeat))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
