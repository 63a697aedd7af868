"""Host-side logic and C-ABI surface (runs without a GPU)."""
import ctypes
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


def test_segment_softmax_rejects_partially_overlapping_buffers():
    """y may be x (in place) or disjoint from it; anything in between would make a
    later pass read results as logits.  The check runs before any launch and touches
    no memory, so made-up addresses do for it (the in-place and disjoint calls stop
    later, at the missing workspace)."""
    lib = capi.load()
    edges, heads = 1000, 4
    nbytes = edges * heads * 4
    ptr = row = 0x10000                    # non-null stand-ins, never dereferenced
    x = 0x4000000

    def call(y):
        return lib.ga_segment_softmax(ptr, row, None, x, y, 10, edges, heads, None, 0, None)

    for y in (x + 4, x - 4, x + nbytes - 4, x - nbytes + 4, x + nbytes // 2):
        assert call(y) == capi.GA_EINVAL, hex(y)
    assert lib.ga_softmax_workspace_bytes(edges, heads) > 0
    for y in (x, x + nbytes, x - nbytes):
        assert call(y) == capi.GA_EWORKSPACE, hex(y)

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


# ---- broadcast tables (bcast.cc) ------------------------------------------------

def test_bcast_header_example():
    """The worked example in the reference's bcast.h:24-35: feature shapes (1, 3)
    and (5, 1) give a (5, 3) output and these two offset lists."""
    from graphiler_amd.bcast import calc_bcast_off
    b = calc_bcast_off("add", (7, 1, 3), (7, 5, 1))
    assert b.use_bcast and (b.lhs_len, b.rhs_len, b.out_len, b.reduce_size) == (3, 5, 15, 1)
    assert b.lhs_offset.tolist() == [0, 1, 2] * 5
    assert b.rhs_offset.tolist() == [0, 0, 0, 1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4]


def test_bcast_matches_numpy_broadcasting():
    """Gathering through the tables must reproduce numpy's own broadcasting of
    the per-row feature blocks (any mistake in stride or dimension order fails)."""
    from graphiler_amd.bcast import calc_bcast_off
    rng = np.random.default_rng(5)
    cases = [((4, 3), (4, 1)), ((4, 1), (4, 6)), ((4, 2, 1, 5), (4, 1, 3, 5)),
             ((4, 3, 5), (4, 5)), ((4, 5), (4, 2, 1)), ((4, 8, 16), (4, 8, 1)),
             ((4, 2, 3, 4), (4, 3, 1))]
    for ls, rs in cases:
        lhs, rhs = rng.standard_normal(ls), rng.standard_normal(rs)
        b = calc_bcast_off("mul", ls, rs)
        assert b.use_bcast
        for row in range(ls[0]):
            want = (lhs[row] * rhs[row]).reshape(-1)
            got = lhs[row].reshape(-1)[b.lhs_offset] * rhs[row].reshape(-1)[b.rhs_offset]
            assert b.out_len == want.size
            np.testing.assert_array_equal(got, want)


def test_bcast_dot_and_plain_shapes():
    from graphiler_amd.bcast import calc_bcast_off, use_bcast
    # same shapes: no table, lengths only
    b = calc_bcast_off("add", (9, 8, 16), (9, 8, 16))
    assert not b.use_bcast and b.out_len == 128 and b.reduce_size == 1
    assert b.lhs_offset.tolist() == [0] and b.rhs_offset.tolist() == [0]
    # dot over the last dimension, heads kept (HGT's u_dot_v: (E, 8, 16) -> (E, 8))
    b = calc_bcast_off("dot", (9, 8, 16), (9, 8, 16))
    assert not b.use_bcast and b.out_len == 8 and b.reduce_size == 16
    # copies never broadcast and take the length of the copied side
    assert not use_bcast("copy_lhs", (3, 4), (3, 7, 2))
    assert calc_bcast_off("copy_rhs", (3, 4), (3, 7, 2)).out_len == 14
    # broadcast dot: (E, 1, 16) . (E, 8, 16) -> 8 outputs of 16-vectors; offsets
    # count vectors, not elements
    b = calc_bcast_off("dot", (9, 1, 16), (9, 8, 16))
    assert b.use_bcast and b.reduce_size == 16 and b.out_len == 8
    assert b.lhs_offset.tolist() == [0] * 8 and b.rhs_offset.tolist() == list(range(8))
    rng = np.random.default_rng(6)
    u, v = rng.standard_normal((1, 16)), rng.standard_normal((8, 16))
    got = [(u.reshape(-1, 16)[b.lhs_offset[k]] * v.reshape(-1, 16)[b.rhs_offset[k]]).sum()
           for k in range(b.out_len)]
    np.testing.assert_allclose(got, (u * v).sum(-1))


def test_static_scratch_sizing_query_without_gpu():
    """ga_gat_static_scratch_needed is host arithmetic: the sizes quoted beside the entry
    point's declaration, the three state layouts (x 1.5 fp32 lanes of four, x 1.25 bf16
    lanes of eight, x 3 one feature per lane), never above the workspace bound of
    ga_gat_aggregate, and the refusal of what the 32 MiB buffer cannot hold."""
    lib = capi.load()
    cap = 32 << 20
    need = lib.ga_gat_static_scratch_needed
    assert need(0, 1, 64, capi.GA_F32, 1) == 0
    assert need(-1, 1, 64, capi.GA_F32, 1) == capi.GA_EINVAL
    assert need(10, 0, 64, capi.GA_F32, 1) == capi.GA_EINVAL
    assert need(10, 1, 64, 99, 1) == capi.GA_EINVAL
    c5 = need(64_308_169, 4, 64, capi.GA_BF16, 1)
    c2 = need(11_600_000, 1, 64, capi.GA_F32, 1)
    assert 15e6 < c5 <= cap and 3e6 < c2 <= cap
    e = 4_000_000
    a4 = need(e, 4, 16, capi.GA_F32, 1)           # lanes of four fp32 features
    a8 = need(e, 4, 16, capi.GA_BF16, 1)          # lanes of eight bf16 features
    s1 = need(e, 4, 16, capi.GA_F32, 0)           # unaligned rows, several heads: scalar lanes
    assert 0 < a8 < a4 < s1            # 6 floats per 4 features, 10 per 8, 3 per feature
    for heads, dim, dt, al in ((4, 16, capi.GA_F32, 1), (4, 16, capi.GA_BF16, 1), (4, 16, capi.GA_F32, 0),
                               (1, 17, capi.GA_F32, 1), (3, 5, capi.GA_BF16, 0), (1, 200, capi.GA_BF16, 1)):
        assert 0 < need(e, heads, dim, dt, al) <= lib.ga_gat_workspace_bytes(e, heads * dim, heads)
    assert need(2_000_000_000, 1, 4096, capi.GA_F32, 1) > cap


def test_new_entry_points_reject_bad_arguments_without_gpu():
    """ga_segment_mm_gated and ga_transpose_scale_blocks_as validate before any launch."""
    lib = capi.load()
    one = ctypes.c_void_p(256)          # an aligned, never dereferenced address
    # empty problems are fine whatever the pointers
    assert lib.ga_segment_mm_gated(None, 4, None, None, None, None, 1, 0, 128, 128, capi.GA_BF16, None) == capi.GA_OK
    assert lib.ga_segment_mm_gated(None, 0, None, None, None, None, 1, 10, 128, 128, capi.GA_BF16, None) == capi.GA_OK
    # a missing gate, a bad dtype, a bad shape
    assert lib.ga_segment_mm_gated(one, 4, one, one, one, None, 1, 10, 128, 128, capi.GA_BF16, None) == capi.GA_EINVAL
    assert lib.ga_segment_mm_gated(one, 4, one, one, one, one, 1, 10, 128, 128, 7, None) == capi.GA_EINVAL
    assert lib.ga_segment_mm_gated(one, 4, one, one, one, one, 1, 10, 0, 128, capi.GA_BF16, None) == capi.GA_EINVAL
    # fp32, or a width the wide kernel does not take: the caller forms the per-row factor
    assert lib.ga_segment_mm_gated(one, 4, one, one, one, one, 1, 10, 128, 128, capi.GA_F32, None) == capi.GA_EUNSUPPORTED
    assert lib.ga_segment_mm_gated(one, 4, one, one, one, one, 1, 10, 128, 64, capi.GA_BF16, None) == capi.GA_EUNSUPPORTED
    odd = ctypes.c_void_p(258)
    assert lib.ga_segment_mm_gated(one, 4, one, one, one, odd, 1, 10, 128, 128, capi.GA_BF16, None) == capi.GA_EALIGN
    tsb = lib.ga_transpose_scale_blocks_as
    assert tsb(None, None, capi.GA_F32, 1.0, None, 0, 16, capi.GA_BF16, None) == capi.GA_OK
    assert tsb(one, None, 9, 1.0, ctypes.c_void_p(512), 4, 16, capi.GA_BF16, None) == capi.GA_EINVAL
    assert tsb(one, None, capi.GA_F32, 1.0, one, 4, 16, capi.GA_BF16, None) == capi.GA_EINVAL      # in place
    assert tsb(one, ctypes.c_void_p(257), capi.GA_BF16, 1.0, ctypes.c_void_p(512), 4, 16, capi.GA_BF16, None) == capi.GA_EALIGN


def test_scaled_sum_and_projection_reject_bad_arguments_without_gpu():
    """ga_spmm_csr_scaled and ga_linear_rows_scaled validate before any launch."""
    lib = capi.load()
    one, odd = ctypes.c_void_p(256), ctypes.c_void_p(258)
    sp = lib.ga_spmm_csr_scaled
    # (pointer, row_of_slot, nbr, eid, u, out, row_scale, activation, n_rows, n_edges, feat, op,
    #  dtype, workspace, workspace_bytes, stream)
    assert sp(None, None, None, None, None, None, None, 0, 0, 0, 8, capi.GA_COPY_U, capi.GA_F32, None, 0, None) == capi.GA_OK
    assert sp(one, one, one, None, one, one, None, 3, 4, 4, 8, capi.GA_COPY_U, capi.GA_F32, one, 1 << 20, None) == capi.GA_EINVAL   # activation
    assert sp(one, one, one, None, one, one, None, 0, 4, 4, 8, capi.GA_U_MUL_E, capi.GA_F32, one, 1 << 20, None) == capi.GA_EINVAL  # copies only
    assert sp(one, one, one, None, one, one, None, 0, 4, 4, 0, capi.GA_COPY_U, capi.GA_F32, one, 1 << 20, None) == capi.GA_EINVAL   # feat
    assert sp(one, one, one, None, one, one, None, 0, 4, 4, 8, capi.GA_COPY_U, 5, one, 1 << 20, None) == capi.GA_EINVAL             # dtype
    assert sp(one, one, None, None, one, one, None, 0, 4, 4, 8, capi.GA_COPY_U, capi.GA_F32, one, 1 << 20, None) == capi.GA_EINVAL  # no neighbours
    assert sp(one, one, one, None, one, one, None, 0, 4, 4, 8, capi.GA_COPY_U, capi.GA_F32, one, 16, None) == capi.GA_EWORKSPACE
    assert sp(one, one, one, None, one, one, odd, 0, 4, 4, 8, capi.GA_COPY_U, capi.GA_F32, one, 1 << 20, None) == capi.GA_EALIGN
    lin = lib.ga_linear_rows_scaled
    # (X, W, row_scale, Z, rows, K, M, stream)
    assert lin(None, None, None, None, 0, 8, 8, None) == capi.GA_OK
    assert lin(one, one, one, one, 4, 0, 8, None) == capi.GA_EINVAL
    assert lin(one, one, one, None, 4, 8, 8, None) == capi.GA_EINVAL
    assert lin(one, one, odd, one, 4, 8, 8, None) == capi.GA_EALIGN
    assert lin(one, one, one, one, 4, 1 << 23, 8, None) == capi.GA_EUNSUPPORTED
