"""Randomised shapes, fixed seeds.  Every test draws a random graph, dtype (fp32 or
bf16), head count and widths from its seed -- including shapes the kernels refuse,
where the wrappers must fall back or say GA_EUNSUPPORTED -- and checks one family of
operators against numpy float64 or the oracle:

  typed products      plain, through the COO column, per-row factor, dot epilogue
  softmax sums        softmax-weighted sum of per-edge rows, both fused GAT passes
  projection          dense projection with its attention terms
  row reductions      every SpMM operator x reducer, both adjacencies
  edge operators      SDDMM add / sub / mul / div (bit-exact) and dot, multi-head
                      softmax, row gather, device-side graph preparation (bit-exact)

fp32 results are held to 1e-5, bf16 results to 2e-2 (helpers.TOL_*), relative to the
magnitude of the expected output.
"""
import numpy as np
import pytest
import torch

import oracle
from graphiler_amd import capi, ops, prepare_graph
from graphiler_amd.graph import build_graph_arrays
from helpers import TOL_BF16, TOL_F32, assert_close, to_bf16_f32

pytestmark = pytest.mark.gpu

TYPED_SEEDS = range(1, 97)
CORE_SEEDS = range(1, 65)


class Case:
    """A random graph with its device form, and the draw it came from."""

    def __init__(self, device, seed, typed):
        self.dev = device
        self.rng = rng = np.random.default_rng(seed)
        self.bf16 = bool(rng.integers(0, 2))
        self.tol = TOL_BF16 if self.bf16 else TOL_F32
        if typed:      # a few relations, one of them possibly large; destinations bunched
            self.n = n = int(rng.integers(1, 400))
            self.n_rel = int(rng.integers(1, 7))
            counts = rng.integers(0, 300, self.n_rel)
            counts[rng.integers(0, self.n_rel)] += int(rng.integers(0, 3000))
            self.etype = np.repeat(np.arange(self.n_rel), counts).astype(np.int64)
            self.e = e = self.etype.shape[0]
            self.src = rng.integers(0, n, e, dtype=np.int64)
            self.dst = rng.integers(0, max(1, n // int(rng.integers(1, 4))), e, dtype=np.int64)
            self.g = prepare_graph(self.src, self.dst, n, device=device, etype_of=self.etype,
                                   num_etypes=self.n_rel)
        else:          # uniform, Zipf-skewed or pre-sorted destinations; 0 to 20,000 edges
            self.n = n = int(rng.integers(1, 600))
            self.e = e = int(rng.choice([0, 1, 5, 60, 700, 5000, 20000]))
            self.src = rng.integers(0, n, e, dtype=np.int64)
            kind = rng.integers(0, 3)
            if kind == 0:
                self.dst = rng.integers(0, n, e, dtype=np.int64)
            elif kind == 1:
                self.dst = (rng.zipf(1.6, e) % n).astype(np.int64)
            else:
                self.dst = np.sort(rng.integers(0, max(1, n // 3), e, dtype=np.int64))
            self.g = prepare_graph(self.src, self.dst, n, device=device)
        self.arr = build_graph_arrays(self.src, self.dst, self.n)
        self.in_adj = (self.arr.in_pointer, self.arr.in_node_indices, self.arr.in_edge_indices)

    def normal(self, *shape, scale=1.0):
        """N(0, scale) values, rounded to bf16 when the case is a bf16 one."""
        a = (self.rng.standard_normal(shape) * scale).astype(np.float32)
        return to_bf16_f32(a) if self.bf16 else a

    def dev_of(self, a, storage=False):
        """Device tensor; ``storage``: in the case's dtype (bf16 cases store bf16)."""
        t = torch.from_numpy(np.ascontiguousarray(a)).to(self.dev)
        return t.bfloat16() if (storage and self.bf16) else t


def _host(t, shape=None):
    a = t.float().cpu().numpy()
    return a if shape is None else a.reshape(shape)


# ---------------------------------------------------------------- typed products ----
@pytest.mark.parametrize("seed", TYPED_SEEDS)
def test_typed_products(device, seed):
    c = Case(device, seed, typed=True)
    rng, e, n = c.rng, c.e, c.n
    heads = int(rng.choice([1, 1, 2, 3, 4, 5, 8]))
    K = int(rng.choice([4, 8, 12, 16, 20, 32, 40, 64, 100, 128]))
    M = int(rng.choice([8, 16, 24, 32, 48, 64, 128]))
    if c.bf16 and rng.integers(0, 2):
        K = max(8, K // 8 * 8)
    if heads * K > 256 or heads * M > 256:
        heads = 1
    X, Q = c.normal(n, heads * K), c.normal(n, heads * M)
    W = c.normal(c.n_rel, heads, K, M, scale=1 / np.sqrt(K))
    dX, dQ, dW = c.dev_of(X, True), c.dev_of(Q, True), c.dev_of(W, True)
    what = f"seed {seed} bf16={c.bf16} H={heads} K={K} M={M}"

    # through the COO column: rows, per-row factor
    which = int(rng.integers(0, 2))
    col, other = (c.src, c.dst) if which == 0 else (c.dst, c.src)
    y64 = np.einsum("ehk,ehkm->ehm", X[col].reshape(e, heads, K).astype(np.float64),
                    W[c.etype].astype(np.float64)) if e else np.zeros((0, heads, M))
    norm = rng.uniform(0.3, 2, (e, 1)).astype(np.float32)
    scaled = bool(rng.integers(0, 2))
    got = ops.SegmentMMEdgeGather(dX, dW, which, c.g, row_scale=c.dev_of(norm) if scaled else None)
    assert_close(_host(got), y64.reshape(e, heads * M) * (norm if scaled else 1.0), c.tol,
                 f"gathered product, {what}")
    # dot epilogue with a per-type factor
    scale = rng.uniform(0.5, 2, (c.n_rel, heads)).astype(np.float32)
    want = np.einsum("ehm,ehm->eh", y64, Q[other].reshape(e, heads, M).astype(np.float64)) * scale[c.etype]
    got = ops.SegmentMMEdgeDot(dX, dW, which, dQ, 1 - which, c.g, scale=c.dev_of(scale))
    assert_close(_host(got), want, c.tol, f"dot epilogue, {what}")
    # plain typed product on per-edge rows
    Xe = c.normal(e, heads * K)
    want = np.einsum("ehk,ehkm->ehm", Xe.reshape(e, heads, K).astype(np.float64),
                     W[c.etype].astype(np.float64)).reshape(e, heads * M) if e else np.zeros((0, heads * M))
    assert_close(_host(ops.SegmentMMEdge(c.dev_of(Xe, True), dW, c.g)), want, c.tol,
                 f"typed product, {what}")


# ------------------------------------------------ softmax-weighted sums, fused GAT ----
@pytest.mark.parametrize("seed", TYPED_SEEDS)
def test_softmax_weighted_sums(device, seed):
    c = Case(device, seed, typed=True)
    rng, e, n = c.rng, c.e, c.n
    dim = int(rng.choice([1, 4, 8, 16, 24, 32, 64]))
    heads = int(rng.choice([1, 2, 3, 4, 8]))
    what = f"seed {seed} bf16={c.bf16} {heads}x{dim}"
    logit = (rng.standard_normal((e, heads)) * 3).astype(np.float32)
    m = c.normal(e, heads * dim)
    att = oracle.segment_softmax(c.arr.in_pointer, c.arr.in_edge_indices, logit)
    prod = (m.reshape(e, heads, dim).astype(np.float64) * att[:, :, None]).reshape(e, heads * dim)
    want = oracle.spmm(*c.in_adj, prod.astype(np.float32), op="copy_e")
    got = ops.edge_softmax_sum(c.dev_of(logit), c.dev_of(m, True), c.g)
    assert_close(_host(got), want, c.tol, f"edge_softmax_sum, {what}")

    z = c.normal(n, heads * dim)
    a_l = (rng.standard_normal((heads, dim)) / np.sqrt(dim)).astype(np.float32)
    er = rng.standard_normal((n, heads), dtype=np.float32)
    el = np.einsum("nhd,hd->nh", z.reshape(n, heads, dim).astype(np.float64), a_l).astype(np.float32)
    want = oracle.gat_aggregate(c.arr.in_pointer, c.arr.in_node_indices, el, er, z, heads=heads, slope=0.2)
    got = ops.gat_aggregate(c.dev_of(el), c.dev_of(er), c.dev_of(z, True), c.g, 0.2)
    assert_close(_host(got, want.shape), want, c.tol, f"gat_aggregate, {what}")
    try:       # the source term recomputed from the rows: head widths it takes only
        got = ops.gat_aggregate_from_z(c.dev_of(a_l), c.dev_of(er), c.dev_of(z, True), c.g, 0.2)
    except capi.GraphilerError as err:
        assert err.code == capi.GA_EUNSUPPORTED
    else:
        # the logits differ from the oracle's by the rounding of el (one fp32 dot product)
        assert_close(_host(got, want.shape), want, c.tol, f"gat_aggregate_from_z, {what}")


# ------------------------------------------------------------------- projection ----
@pytest.mark.parametrize("seed", TYPED_SEEDS)
def test_projection_with_attention_terms(device, seed):
    rng = np.random.default_rng(seed + 1000)
    bf16 = bool(rng.integers(0, 2))
    rows = int(rng.integers(1, 700))
    K = int(rng.choice([8, 16, 40, 100, 128, 200, 256]))
    dph = int(rng.choice([16, 32, 64, 128]))
    heads = int(rng.choice([1, 2, 4]))
    M = dph * heads
    x = rng.standard_normal((rows, K), dtype=np.float32)
    w = (rng.standard_normal((K, M)) / np.sqrt(K)).astype(np.float32)
    a = rng.standard_normal((2, heads, dph), dtype=np.float32)
    if bf16:
        x, w = to_bf16_f32(x), to_bf16_f32(w)

    def dev_of(t, storage=False):
        t = torch.from_numpy(np.ascontiguousarray(t)).to(device)
        return t.bfloat16() if (storage and bf16) else t

    try:
        z, el, er = ops.linear_attn(dev_of(x, True), dev_of(w, True), dev_of(a[0]), dev_of(a[1]))
    except capi.GraphilerError as err:
        assert err.code == capi.GA_EUNSUPPORTED
        return
    what = f"seed {seed} bf16={bf16} {rows}x{K}->{heads}x{dph}"
    z64 = x.astype(np.float64) @ w.astype(np.float64)
    assert_close(_host(z), z64, TOL_BF16 if bf16 else TOL_F32, f"projection, {what}")
    # el / er come from the fp32 accumulators (before z is rounded), so fp32 accuracy
    # also for bf16 storage
    zh = z64.reshape(rows, heads, dph)
    assert_close(_host(el), (zh * a[0]).sum(-1), TOL_F32, f"el, {what}")
    assert_close(_host(er), (zh * a[1]).sum(-1), TOL_F32, f"er, {what}")


# --------------------------------------------------------------- row reductions ----
@pytest.mark.parametrize("seed", CORE_SEEDS)
def test_row_reductions(device, seed):
    c = Case(device, seed, typed=False)
    rng, e, n = c.rng, c.e, c.n
    heads = int(rng.choice([1, 1, 2, 4, 8]))
    dim = int(rng.choice([1, 2, 3, 4, 8, 16, 17, 32, 64, 128]))
    feat = heads * dim
    x, m = c.normal(n, feat), c.normal(e, feat)
    w = rng.uniform(0.2, 2.0, (e, heads)).astype(np.float32)
    op = str(rng.choice(["copy_u", "copy_e", "u_mul_e", "u_add_e", "u_sub_e", "u_div_e"]))
    red = str(rng.choice(["sum", "max", "min"]))
    u = m if op == "copy_e" else x
    ww = None if op in ("copy_u", "copy_e") else w
    what = f"seed {seed} bf16={c.bf16} n={n} e={e} {heads}x{dim}"
    want = oracle.spmm(*c.in_adj, u, ww, op=op, reduce=red, heads=heads)
    got = ops.spmm(c.g, op, red, c.dev_of(u, True), None if ww is None else c.dev_of(ww))
    assert_close(_host(got, want.shape), want, c.tol, f"{op} {red}, {what}")
    want = oracle.spmm(c.arr.out_pointer, c.arr.out_node_indices, c.arr.out_edge_indices, x, w,
                       op="u_mul_e", heads=heads)
    got = ops.gspmm_dst_mul_e_sum(c.dev_of(x, True), c.dev_of(w), [1], False, None, c.g)
    assert_close(_host(got, want.shape), want, c.tol, f"u_mul_e over the out-adjacency, {what}")


# --------------------------------------------------------------- edge operators ----
@pytest.mark.parametrize("seed", CORE_SEEDS)
def test_edge_operators_and_graph_preparation(device, seed):
    c = Case(device, seed, typed=False)
    rng, e, n = c.rng, c.e, c.n
    heads = int(rng.choice([1, 1, 2, 4, 8]))
    dim = int(rng.choice([1, 2, 3, 4, 8, 16, 17, 32, 64, 128]))
    what = f"seed {seed} bf16={c.bf16} n={n} e={e} {heads}x{dim}"
    uu = rng.standard_normal((n, heads), dtype=np.float32)
    vv = rng.standard_normal((n, heads), dtype=np.float32)
    got = ops.gsddmm_u_add_v_mul_alpha(c.dev_of(uu), c.dev_of(vv), 1, c.g)
    assert np.array_equal(_host(got), oracle.sddmm_u_add_v(c.src, c.dst, uu, vv)), f"u_add_v, {what}"
    sop = str(rng.choice(["sub", "mul", "div"]))
    got = ops.gsddmm_u_op_v(sop, c.dev_of(uu), c.dev_of(vv + 3), c.g)
    assert np.array_equal(_host(got), oracle.sddmm_u_op_v(sop, c.src, c.dst, uu, vv + 3)), f"u_{sop}_v, {what}"
    k3 = c.normal(n, heads, dim)
    got = ops.gsddmm_u_dot_v(c.dev_of(k3, True), c.dev_of(k3, True), c.g)
    assert_close(_host(got), oracle.sddmm_u_dot_v(c.src, c.dst, k3, k3), TOL_F32, f"u_dot_v, {what}")
    lg = (rng.standard_normal((e, heads)) * 4).astype(np.float32)
    want = oracle.segment_softmax(c.arr.in_pointer, c.arr.in_edge_indices, lg)
    assert_close(_host(ops.SegmentSoftmax(c.dev_of(lg), 1, None, c.g)), want, TOL_F32,
                 f"softmax, {what}", mag=want)
    x = c.normal(n, heads * dim)
    assert np.array_equal(_host(ops.BroadcastSrcNode(c.dev_of(x, True), c.g)), x[c.src]), f"gather, {what}"
    for name in ("in_pointer", "in_node_indices", "in_edge_indices", "out_pointer",
                 "out_node_indices", "out_edge_indices"):
        assert np.array_equal(getattr(c.g, name).cpu().numpy(), getattr(c.arr, name)), \
            f"graph preparation: {name}, {what}"
