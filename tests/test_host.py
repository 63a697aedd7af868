"""Host-side logic and C-ABI surface (runs without a GPU)."""
import os
import re

import numpy as np
import pytest

import oracle
from graphiler_amd import capi, datasets
from graphiler_amd.graph import (build_graph_arrays, sort_edges_by_type,
                                 type_pointer)
from helpers import random_graph, skewed_graph

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "graphiler_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ga_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = _declared_symbols()
    assert len(names) >= 12
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
        assert name in capi.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(capi.SIGNATURES) == names
    assert lib.ga_version() >= 100
    assert b"workspace" in lib.ga_error_string(capi.GA_EWORKSPACE)


def test_argument_rejection_without_gpu():
    """Validation happens before any launch, so it is testable on the CPU."""
    lib = capi.load()
    assert lib.ga_spmm_csr(None, None, None, None, None, None, None, 4, 4, 8, 3,
                           0, 0, 0, None, 0, None) == capi.GA_EINVAL   # 8 % 3
    assert lib.ga_spmm_csr(None, None, None, None, None, None, None, 4, 4, 8, 1,
                           7, 0, 0, None, 0, None) == capi.GA_EINVAL   # bad op
    assert lib.ga_spmm_csr(None, None, None, None, None, None, None, 0, 0, 8, 1,
                           0, 0, 0, None, 0, None) == capi.GA_OK       # empty
    assert lib.ga_sddmm_u_add_v(None, None, 16, None, None, None, 4, 1, 0,
                                None) == capi.GA_EINVAL                # idx bits
    assert lib.ga_segment_softmax(None, None, None, None, None, 3, 5, 0,
                                  None, 0, None) == capi.GA_EINVAL     # heads
    assert lib.ga_gather_rows(None, 64, None, None, 0, 16, None) == capi.GA_OK
    assert lib.ga_spmm_workspace_bytes(0, 64) == 0
    assert lib.ga_spmm_workspace_bytes(1000, 64) >= 2 * 64 * 4


@pytest.mark.parametrize("kind", ["uniform", "skewed", "empty"])
def test_build_graph_arrays_matches_oracle_bit_exact(kind):
    rng = np.random.default_rng(3)
    if kind == "uniform":
        n = 500
        s, d = random_graph(rng, n, 4000)
    elif kind == "skewed":
        n = 800
        s, d = skewed_graph(rng, n, 3000, 2500)
    else:
        n, s, d = 9, np.zeros(0, np.int64), np.zeros(0, np.int64)
    arr = build_graph_arrays(s, d, n)
    p, nb, e = oracle.group_edges(n, d, s)
    assert arr.in_pointer.dtype == np.int32 and arr.COO_src.dtype == np.int64
    assert np.array_equal(arr.in_pointer, p)
    assert np.array_equal(arr.in_node_indices, nb)
    assert np.array_equal(arr.in_edge_indices, e)
    p, nb, e = oracle.group_edges(n, s, d)
    assert np.array_equal(arr.out_pointer, p)
    assert np.array_equal(arr.out_node_indices, nb)
    assert np.array_equal(arr.out_edge_indices, e)


def test_build_graph_arrays_rejects_bad_edges():
    with pytest.raises(ValueError):
        build_graph_arrays([0, 5], [1, 1], 3)
    with pytest.raises(ValueError):
        build_graph_arrays([0, 1], [1], 3)


def test_type_sort_and_pointer():
    rng = np.random.default_rng(4)
    s, d = random_graph(rng, 50, 400)
    et = rng.integers(0, 7, 400)
    s2, d2, et2, order = sort_edges_by_type(s, d, et)
    assert np.all(np.diff(et2) >= 0)
    assert np.array_equal(order, np.lexsort((np.arange(400), et)))   # stable
    assert np.array_equal(s2, s[order]) and np.array_equal(d2, d[order])
    ptr = type_pointer(et2, 9)
    assert np.array_equal(ptr, oracle.type_pointer(et2, 9))
    with pytest.raises(ValueError):
        type_pointer(et, 9)


def test_workloads_are_deterministic_and_shaped():
    a = datasets.gcn_uniform()
    b = datasets.gcn_uniform()
    assert a.num_nodes == 19717 and a.num_edges == 88651 + 19717
    assert np.array_equal(a.src, b.src) and np.array_equal(a.dst, b.dst)
    assert np.all(np.diff(a.dst) >= 0)               # stored by destination
    r = datasets.rgcn_zipf(num_nodes=2000, n_edges=30000)
    assert np.all(np.diff(r.etype) >= 0) and r.etype.max() < 60
    cnt = np.bincount(r.etype, minlength=60)
    assert cnt[0] > cnt[10] > cnt[59] >= 0           # Zipf-shaped
    h = datasets.hgt_hetero(counts=(400, 300, 200, 100), edges_per_type=2000)
    assert h.num_nodes == 1000 and h.num_edges == 20000
    start = np.concatenate([[0], np.cumsum([400, 300, 200, 100])])
    for t, (st, dt) in enumerate(h.meta["type_pairs"]):
        sl = slice(t * 2000, (t + 1) * 2000)
        assert np.all((h.src[sl] >= start[st]) & (h.src[sl] < start[st + 1]))
        assert np.all((h.dst[sl] >= start[dt]) & (h.dst[sl] < start[dt + 1]))
    g = datasets.gat_rmat(num_nodes=3000, n_edges=60000, scale=12, seed=1)
    deg = np.bincount(g.dst, minlength=3000)
    assert deg.max() > 20 * deg.mean()               # power-law skew


def test_debug_graphs_match_fixture_file():
    import json
    fx = json.load(open(os.path.join(ROOT, "tests", "golden", "debug_graphs.json")))
    d0, d1 = datasets.debug_graph(), datasets.debug_hetero_graph()
    assert d0.src.tolist() == fx[0]["src"] and d0.dst.tolist() == fx[0]["dst"]
    assert d1.src.tolist() == fx[1]["src"] and d1.dst.tolist() == fx[1]["dst"]
    assert d1.etype.tolist() == fx[1]["etype"]
    arr = build_graph_arrays(d0.src, d0.dst, 3)
    # hand vector from the reference's debug graph
    assert arr.in_pointer.tolist() == [0, 1, 3, 6]
    assert arr.in_node_indices.tolist() == [0, 0, 1, 0, 1, 2]
    assert arr.in_edge_indices.tolist() == [0, 1, 3, 2, 4, 5]
