"""Pins the CPU oracle (runs without a GPU).

The reference has no golden vectors for its operators, so every oracle function
is checked against something that does not share its code: hand-evaluated
fixtures on the reference's two debug graphs (tests/golden), library routines
(scipy.sparse products, numpy fancy indexing / einsum, scipy.special.softmax,
numpy matmul), brute-force Python loops and invariants of the mathematics.
Each check is chosen so that a plausible slip (wrong index column, transposed
operand, dropped term, wrong reducer start) fails it.
"""
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp
from scipy.special import softmax as scipy_softmax

import oracle
from helpers import random_graph, skewed_graph

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "debug_graphs.json")


def _fixtures():
    with open(GOLDEN) as f:
        return json.load(f)


def _arr(fx, key, dtype):
    return np.asarray(fx[key], dtype=dtype)


def _graph(rng, kind="uniform"):
    if kind == "uniform":
        n = 200
        s, d = random_graph(rng, n, 1500)
    else:
        n = 400
        s, d = skewed_graph(rng, n, 1500, 700)
    ptr, nbr, eid = oracle.group_edges(n, d, s)
    return n, s, d, ptr, nbr, eid


# ------------------------------------------------------------- fixtures ----
@pytest.mark.parametrize("fx", _fixtures(), ids=lambda f: f["name"])
def test_golden_debug_graphs(fx):
    n = fx["num_nodes"]
    src, dst = _arr(fx, "src", np.int64), _arr(fx, "dst", np.int64)
    ptr, nbr, eid = oracle.group_edges(n, dst, src)
    assert ptr.tolist() == fx["in_pointer"]
    assert nbr.tolist() == fx["in_node_indices"]
    assert eid.tolist() == fx["in_edge_indices"]
    optr, onbr, oeid = oracle.group_edges(n, src, dst)
    assert optr.tolist() == fx["out_pointer"]
    assert onbr.tolist() == fx["out_node_indices"]
    assert oeid.tolist() == fx["out_edge_indices"]
    x, m = _arr(fx, "x", np.float32), _arr(fx, "m", np.float32)
    w = _arr(fx, "w", np.float32)
    # integer-valued inputs: every expected value is exact
    assert oracle.spmm(ptr, nbr, eid, x, op="copy_u").tolist() == fx["copy_u_sum"]
    assert oracle.spmm(ptr, nbr, eid, m, op="copy_e").tolist() == fx["copy_e_sum"]
    assert oracle.spmm(ptr, nbr, eid, x, w, op="u_mul_e").tolist() == fx["u_mul_e_sum"]
    assert oracle.spmm(optr, onbr, oeid, x, w, op="u_mul_e").tolist() == fx["dst_mul_e_sum"]
    assert oracle.spmm_sum_f32(ptr, nbr, eid, x, w, op="u_mul_e").tolist() == fx["u_mul_e_sum"]
    mx = oracle.spmm(ptr, nbr, eid, x, op="copy_u", reduce="max")
    want = np.array([[-np.inf if v is None else v for v in row]
                     for row in fx["copy_u_max"]], np.float32)
    assert np.array_equal(mx, want)
    ul, vr = _arr(fx, "ul", np.float32), _arr(fx, "vr", np.float32)
    assert oracle.sddmm_u_add_v(src, dst, ul[:, None], vr[:, None])[:, 0].tolist() == fx["u_add_v"]
    assert oracle.sddmm_u_dot_v(src, dst, x, x)[:, 0].tolist() == fx["u_dot_v"]
    sm = oracle.segment_softmax(ptr, eid, w)
    np.testing.assert_allclose(sm, np.asarray(fx["edge_softmax_w"]), rtol=1e-6)
    assert oracle.gather_rows(src, x).tolist() == fx["gather_src"]
    assert oracle.gather_rows(dst, x).tolist() == fx["gather_dst"]
    if "etype" in fx:
        et = _arr(fx, "etype", np.int64)
        tp = oracle.type_pointer(et, len(fx["W"]))
        assert tp.tolist() == fx["etype_pointer"]
        y = oracle.segment_mm(tp, m, _arr(fx, "W", np.float32))
        assert y.tolist() == fx["segment_mm_edge"]


# ------------------------------------------------------- graph grouping ----
@pytest.mark.parametrize("kind", ["uniform", "skewed"])
def test_group_edges_invariants(kind):
    rng = np.random.default_rng(1)
    n, s, d, ptr, nbr, eid = _graph(rng, kind)
    e = s.shape[0]
    assert ptr[0] == 0 and ptr[-1] == e and np.all(np.diff(ptr) >= 0)
    assert np.array_equal(np.sort(eid), np.arange(e))          # a permutation
    assert np.array_equal(nbr, s[eid])                         # other endpoint
    rows = np.repeat(np.arange(n), np.diff(ptr))
    assert np.array_equal(d[eid], rows)                        # grouped by key
    assert np.array_equal(np.diff(ptr), np.bincount(d, minlength=n))
    # within one group the edge ids ascend == lexicographic (key, edge id) sort
    assert np.array_equal(eid, np.lexsort((np.arange(e), d)))


def test_group_edges_rejects_out_of_range():
    with pytest.raises(ValueError):
        oracle.group_edges(3, np.array([0, 3]), np.array([0, 1]))


def test_type_pointer():
    t = np.array([0, 0, 2, 2, 2, 5], np.int64)
    assert oracle.type_pointer(t, 7).tolist() == [0, 2, 2, 5, 5, 5, 6, 6]
    with pytest.raises(ValueError):
        oracle.type_pointer(np.array([1, 0]), 2)               # not sorted


# ------------------------------------------------------------------ SpMM ----
@pytest.mark.parametrize("kind", ["uniform", "skewed"])
def test_spmm_sum_matches_scipy(kind):
    rng = np.random.default_rng(2)
    n, s, d, ptr, nbr, eid = _graph(rng, kind)
    e = s.shape[0]
    x = rng.standard_normal((n, 9))
    w = rng.standard_normal(e)
    m = rng.standard_normal((e, 5))
    a_ones = sp.csr_matrix((np.ones(e), (d, s)), shape=(n, n))   # duplicates add
    a_w = sp.csr_matrix((w.astype(np.float32).astype(np.float64), (d, s)), shape=(n, n))
    x32 = x.astype(np.float32)
    np.testing.assert_allclose(oracle.spmm(ptr, nbr, eid, x32, op="copy_u"),
                               a_ones @ x32.astype(np.float64), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(
        oracle.spmm(ptr, nbr, eid, x32, w.astype(np.float32), op="u_mul_e"),
        a_w @ x32.astype(np.float64), rtol=1e-6, atol=1e-6)
    # copy_e: incidence matrix (node x edge) times the edge rows
    inc = sp.csr_matrix((np.ones(e), (d, np.arange(e))), shape=(n, e))
    m32 = m.astype(np.float32)
    np.testing.assert_allclose(oracle.spmm(ptr, nbr, eid, m32, op="copy_e"),
                               inc @ m32.astype(np.float64), rtol=1e-6, atol=1e-6)
    # sequential-fp32 variant stays within the fp32 parity tolerance
    f32 = oracle.spmm_sum_f32(ptr, nbr, eid, x32, w.astype(np.float32), op="u_mul_e")
    ref = oracle.spmm(ptr, nbr, eid, x32, w.astype(np.float32), op="u_mul_e")
    assert np.abs(f32 - ref).max() <= 1e-5 * np.abs(ref).max()


def test_spmm_multi_head_matches_einsum_scatter():
    rng = np.random.default_rng(3)
    n, s, d, ptr, nbr, eid = _graph(rng)
    e, H, D = s.shape[0], 4, 6
    x = rng.standard_normal((n, H, D)).astype(np.float32)
    w = rng.standard_normal((e, H)).astype(np.float32)
    msg = x[s].astype(np.float64) * w[:, :, None]
    want = np.zeros((n, H, D))
    np.add.at(want, d, msg)
    got = oracle.spmm(ptr, nbr, eid, x.reshape(n, H * D), w, op="u_mul_e", heads=H)
    np.testing.assert_allclose(got, want.reshape(n, H * D), rtol=1e-6, atol=1e-6)


def test_spmm_invariants():
    rng = np.random.default_rng(4)
    n, s, d, ptr, nbr, eid = _graph(rng, "skewed")
    e = s.shape[0]
    x = rng.standard_normal((n, 8)).astype(np.float32)
    y = rng.standard_normal((n, 8)).astype(np.float32)
    w = rng.standard_normal((e, 1)).astype(np.float32)
    f = lambda a: oracle.spmm(ptr, nbr, eid, a, w, op="u_mul_e").astype(np.float64)
    # linear in the node features
    np.testing.assert_allclose(f(x) + 2 * f(y), f((x + 2 * y).astype(np.float32)),
                               rtol=1e-4, atol=1e-4)
    # column sums equal the sum of all messages
    np.testing.assert_allclose(f(x).sum(0), (x[s].astype(np.float64) * w).sum(0),
                               rtol=1e-6, atol=1e-4)
    # rows without in-edges are exactly zero
    assert not f(x)[np.diff(ptr) == 0].any()
    # relabelling the edge ids (with their data) changes nothing
    perm = rng.permutation(e)
    ptr2, nbr2, eid2 = oracle.group_edges(n, d[perm], s[perm])
    got2 = oracle.spmm(ptr2, nbr2, eid2, x, w[perm], op="u_mul_e")
    np.testing.assert_allclose(got2, f(x), rtol=1e-6, atol=1e-6)


def test_spmm_max_min_against_reduceat_and_ties():
    rng = np.random.default_rng(5)
    n, s, d, ptr, nbr, eid = _graph(rng, "skewed")
    x = rng.integers(-3, 4, (n, 5)).astype(np.float32)      # many ties
    msgs = x[nbr]
    nonempty = np.diff(ptr) > 0
    starts = ptr[:-1][nonempty]
    for red, ufunc, fill in (("max", np.maximum, -np.inf), ("min", np.minimum, np.inf)):
        got, arg_u, arg_e = oracle.spmm(ptr, nbr, eid, x, op="copy_u", reduce=red,
                                        want_arg=True)
        want = np.full((n, 5), fill, np.float32)
        want[nonempty] = ufunc.reduceat(msgs, starts, axis=0)
        assert np.array_equal(got, want)
        # arg outputs: FIRST extremum in group order (strict comparison)
        for v in np.flatnonzero(nonempty)[:50]:
            seg = slice(ptr[v], ptr[v + 1])
            for f in range(5):
                col = msgs[seg, f]
                first = int(np.argmax(col)) if red == "max" else int(np.argmin(col))
                assert arg_u[v, f] == nbr[seg][first]
                assert arg_e[v, f] == eid[seg][first]
        assert not arg_u[~nonempty].any() and not arg_e[~nonempty].any()


# ----------------------------------------------------------------- SDDMM ----
def test_spmm_add_sub_div_against_scatter_and_reduceat():
    """The other binary operators of the generic kernel (functor.cuh:19-72):
    sum against np.add.at on explicitly formed messages (operand order and the
    per-head broadcast of w matter for sub / div), max against reduceat."""
    rng = np.random.default_rng(15)
    n, s, d, ptr, nbr, eid = _graph(rng, "skewed")
    e, H, D = s.shape[0], 2, 3
    x = rng.standard_normal((n, H, D)).astype(np.float32)
    w = (rng.uniform(0.5, 2.0, (e, H)) * rng.choice([-1, 1], (e, H))).astype(np.float32)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)[:, :, None]
    forms = {"u_add_e": x64[s] + w64, "u_sub_e": x64[s] - w64, "u_div_e": x64[s] / w64}
    nonempty = np.diff(ptr) > 0
    for op, msg in forms.items():
        want = np.zeros((n, H, D))
        np.add.at(want, d, msg)
        got = oracle.spmm(ptr, nbr, eid, x.reshape(n, H * D), w, op=op, heads=H)
        np.testing.assert_allclose(got, want.reshape(n, H * D), rtol=1e-5, atol=1e-5, err_msg=op)
        grouped = msg.reshape(e, H * D)[eid]                 # messages in group order
        wmax = np.full((n, H * D), -np.inf)
        wmax[nonempty] = np.maximum.reduceat(grouped, ptr[:-1][nonempty], axis=0)
        gmax = oracle.spmm(ptr, nbr, eid, x.reshape(n, H * D), w, op=op, reduce="max", heads=H)
        np.testing.assert_allclose(gmax, wmax.astype(np.float32), rtol=1e-6, err_msg=op)
    # u_sub_e is not e_sub_u, u_div_e is not e_div_u
    a = oracle.spmm(ptr, nbr, eid, x.reshape(n, H * D), w, op="u_sub_e", heads=H)
    b = oracle.spmm(ptr, nbr, eid, x.reshape(n, H * D), w, op="u_add_e", heads=H)
    deg_w = np.zeros((n, H))
    np.add.at(deg_w, d, w.astype(np.float64))
    np.testing.assert_allclose((b - a).reshape(n, H, D), 2 * deg_w[:, :, None] * np.ones(D),
                               rtol=1e-4, atol=1e-4)


def test_sddmm_against_numpy_indexing():
    rng = np.random.default_rng(6)
    n, s, d, *_ = _graph(rng)
    u = rng.standard_normal((n, 3)).astype(np.float32)
    v = rng.standard_normal((n, 3)).astype(np.float32)
    assert np.array_equal(oracle.sddmm_u_add_v(s, d, u, v), u[s] + v[d])
    # a swapped (src, dst) pair must not pass
    assert not np.array_equal(oracle.sddmm_u_add_v(s, d, u, v), u[d] + v[s])
    # the other functors: numpy's own fp32 arithmetic on the indexed rows, bit for bit
    v_nz = np.where(np.abs(v) < 0.1, 1.0, v).astype(np.float32)
    for op, fn in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply),
                   ("div", np.divide)):
        assert np.array_equal(oracle.sddmm_u_op_v(op, s, d, u, v_nz), fn(u[s], v_nz[d])), op
    assert not np.array_equal(oracle.sddmm_u_op_v("sub", s, d, u, v_nz), v_nz[d] - u[s])
    a = rng.standard_normal((n, 4, 7)).astype(np.float32)
    b = rng.standard_normal((n, 4, 7)).astype(np.float32)
    want = np.einsum("ehk,ehk->eh", a[s].astype(np.float64), b[d].astype(np.float64))
    np.testing.assert_allclose(oracle.sddmm_u_dot_v(s, d, a, b), want, rtol=1e-6, atol=1e-6)


# --------------------------------------------------------------- softmax ----
@pytest.mark.parametrize("heads", [1, 3])
def test_segment_softmax_against_scipy(heads):
    rng = np.random.default_rng(7)
    n, s, d, ptr, nbr, eid = _graph(rng, "skewed")
    e = s.shape[0]
    x = (rng.standard_normal((e, heads)) * 5).astype(np.float32)
    got = oracle.segment_softmax(ptr, eid, x)
    for v in range(n):
        ids = eid[ptr[v]:ptr[v + 1]]
        if len(ids):
            np.testing.assert_allclose(got[ids], scipy_softmax(x[ids].astype(np.float64), axis=0),
                                       rtol=2e-6, atol=1e-12)


def test_segment_softmax_invariants_and_reference_floor():
    rng = np.random.default_rng(8)
    n, s, d, ptr, nbr, eid = _graph(rng)
    e = s.shape[0]
    x = rng.standard_normal(e).astype(np.float32)
    y = oracle.segment_softmax(ptr, eid, x)
    sums = np.zeros(n)
    np.add.at(sums, d, y)
    deg = np.diff(ptr)
    np.testing.assert_allclose(sums[deg > 0], 1.0, rtol=1e-6)
    # shift invariance, equal logits -> 1/deg, single-edge segment -> 1
    np.testing.assert_allclose(oracle.segment_softmax(ptr, eid, x + 3.0), y, rtol=1e-5)
    flat = oracle.segment_softmax(ptr, eid, np.full(e, 0.7, np.float32))
    np.testing.assert_allclose(flat, 1.0 / deg[d], rtol=1e-6)
    assert np.all(y[np.isin(d, np.flatnonzero(deg == 1))] == 1.0)
    # the reference's running maximum starts at 0 (segment_softmax_kernel.cu:9):
    # same numbers inside the parity tolerance while logits are in a sane range,
    # NaN once every logit of a segment is far below zero
    yq = oracle.segment_softmax(ptr, eid, x - 20.0, zero_floor=True)
    assert np.abs(yq - y).max() <= 1e-5 * y.max()
    deep = oracle.segment_softmax(ptr, eid, x - 200.0, zero_floor=True)
    assert np.isnan(deep).any()
    assert np.isfinite(oracle.segment_softmax(ptr, eid, x - 200.0)).all()


# ------------------------------------------------------------ segment_mm ----
@pytest.mark.parametrize("heads", [1, 2])
def test_segment_mm_against_numpy(heads):
    rng = np.random.default_rng(9)
    counts = [5, 0, 17, 1, 0, 40]                  # empty segments included
    tp = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows, K, M = int(tp[-1]), 6, 4
    X = rng.standard_normal((rows, heads, K)).astype(np.float32)
    W = rng.standard_normal((len(counts), heads, K, M)).astype(np.float32)
    want = np.concatenate([
        np.einsum("rhk,hkm->rhm", X[tp[t]:tp[t + 1]].astype(np.float64), W[t].astype(np.float64))
        for t in range(len(counts))])
    got = oracle.segment_mm(tp, X.reshape(rows, heads * K), W, heads=heads)
    np.testing.assert_allclose(got, want.reshape(rows, heads * M), rtol=1e-6, atol=1e-6)
    # W is (K, M), not (M, K): a transposed operand gives a different answer
    if heads == 1:
        wrong = np.concatenate([X[tp[t]:tp[t + 1], 0, :4] @ W[t, 0, :4, :].T
                                for t in range(len(counts))])
        assert not np.allclose(got, wrong)
    f32 = oracle.segment_mm(tp, X.reshape(rows, heads * K), W, heads=heads, f32_accumulate=True)
    assert np.abs(f32 - got).max() <= 1e-5 * np.abs(got).max()


# ---------------------------------------------------------------- gather ----
def test_gather_rows():
    rng = np.random.default_rng(10)
    x = rng.integers(-1000, 1000, (50, 3, 2)).astype(np.int64)
    idx = rng.integers(0, 50, 300)
    assert np.array_equal(oracle.gather_rows(idx, x), x[idx])
    with pytest.raises(ValueError):
        oracle.gather_rows(np.array([50]), x)


# ------------------------------------------------------------- GAT chain ----
def test_gat_aggregate_is_masked_dense_attention():
    """On a simple graph (no parallel edges) the chain equals textbook
    softmax(scores + mask) @ Z with scores[v, u] = leaky_relu(el[u] + er[v])."""
    rng = np.random.default_rng(12)
    n, H, D = 40, 2, 5
    adj = rng.random((n, n)) < 0.15
    adj[7, :] = False                                # a node without in-edges
    d, s = np.nonzero(adj)                           # adj[v, u]: edge u -> v
    ptr, nbr, eid = oracle.group_edges(n, d, s)
    el = rng.standard_normal((n, H)).astype(np.float32)
    er = rng.standard_normal((n, H)).astype(np.float32)
    z = rng.standard_normal((n, H, D)).astype(np.float32)
    got = oracle.gat_aggregate(ptr, nbr, el, er, z.reshape(n, H * D), heads=H, slope=0.2)
    want = np.zeros((n, H, D))
    for h in range(H):
        sc = (el[None, :, h] + er[:, None, h]).astype(np.float64)
        sc = np.where(sc >= 0, sc, 0.2 * sc)
        sc = np.where(adj, sc, -np.inf)
        with np.errstate(invalid="ignore"):
            att = scipy_softmax(sc, axis=1)
        att = np.nan_to_num(att)
        want[:, h] = att @ z[:, h].astype(np.float64)
    np.testing.assert_allclose(got, want.reshape(n, H * D), rtol=1e-5, atol=1e-6)


def test_gat_aggregate_equals_operator_chain():
    rng = np.random.default_rng(13)
    n, s, d, ptr, nbr, eid = _graph(rng, "skewed")    # parallel edges, shuffled ids
    H, D = 2, 4
    el = rng.standard_normal((n, H)).astype(np.float32)
    er = rng.standard_normal((n, H)).astype(np.float32)
    z = rng.standard_normal((n, H * D)).astype(np.float32)
    logits = oracle.sddmm_u_add_v(s, d, el, er)
    logits = np.where(logits >= 0, logits, np.float32(0.2) * logits).astype(np.float32)
    att = oracle.segment_softmax(ptr, eid, logits)
    want = oracle.spmm(ptr, nbr, eid, z, att, op="u_mul_e", heads=H)
    got = oracle.gat_aggregate(ptr, nbr, el, er, z, heads=H, slope=0.2)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
