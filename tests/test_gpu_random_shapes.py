"""Randomised shapes: typed products (plain, through the COO column, with the
dot epilogue, per-type and per-row factors), the softmax-weighted sum of per-edge
rows, both fused GAT passes and the projection with attention terms, each on a
random typed graph with random head counts and widths (including shapes the
kernels refuse, where the wrappers must fall back or say GA_EUNSUPPORTED),
against numpy float64 and the oracle.  Seeds are fixed; a sweep of 2,300 further
seeds of the same generator passed when this file was written.  A second test
does the same for the reference's own operators on random graphs."""
import numpy as np
import pytest
import torch
import oracle
from graphiler_amd import capi, ops, prepare_graph
from graphiler_amd.graph import build_graph_arrays
from helpers import rel_err, to_bf16_f32
pytestmark = pytest.mark.gpu

def rel(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    if ref.size == 0:
        return 0.0
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))

@pytest.mark.parametrize('seed', range(1, 97))
def test_random_shapes(device, seed):
    dev = device

    def D(a, bf16=False):
        t = torch.from_numpy(np.ascontiguousarray(a)).to(dev)
        return t.bfloat16() if bf16 else t
    rng = np.random.default_rng(seed)
    bf16 = bool(rng.integers(0, 2))
    tol = 0.02 if bf16 else 3e-05
    n = int(rng.integers(1, 400))
    n_rel = int(rng.integers(1, 7))
    counts = rng.integers(0, 300, n_rel)
    counts[rng.integers(0, n_rel)] += int(rng.integers(0, 3000))
    etype = np.repeat(np.arange(n_rel), counts).astype(np.int64)
    e = etype.shape[0]
    src = rng.integers(0, n, e, dtype=np.int64)
    dst = rng.integers(0, max(1, n // int(rng.integers(1, 4))), e, dtype=np.int64)
    g = prepare_graph(src, dst, n, device=dev, etype_of=etype, num_etypes=n_rel)
    arr = build_graph_arrays(src, dst, n)
    heads = int(rng.choice([1, 1, 2, 3, 4, 5, 8]))
    K = int(rng.choice([4, 8, 12, 16, 20, 32, 40, 64, 100, 128]))
    M = int(rng.choice([8, 16, 24, 32, 48, 64, 128]))
    if bf16:
        K = max(8, K // 8 * 8) if rng.integers(0, 2) else K
    if heads * K > 256 or heads * M > 256:
        heads = 1
    X = rng.standard_normal((n, heads * K), dtype=np.float32)
    Q = rng.standard_normal((n, heads * M), dtype=np.float32)
    W = (rng.standard_normal((n_rel, heads, K, M)) / np.sqrt(K)).astype(np.float32)
    if bf16:
        (X, Q, W) = (to_bf16_f32(X), to_bf16_f32(Q), to_bf16_f32(W))
    (dX, dQ, dW) = (D(X, bf16), D(Q, bf16), D(W, bf16))
    # typed product through the COO column: rows, per-row factor, dot epilogue with per-type factor
    which = int(rng.integers(0, 2))
    col = src if which == 0 else dst
    oth = dst if which == 0 else src
    y64 = np.einsum('ehk,ehkm->ehm', X[col].reshape(e, heads, K).astype(np.float64), W[etype].astype(np.float64)) if e else np.zeros((0, heads, M))
    norm = rng.uniform(0.3, 2, (e, 1)).astype(np.float32)
    scaled = bool(rng.integers(0, 2))
    got = ops.SegmentMMEdgeGather(dX, dW, which, g, row_scale=D(norm) if scaled else None)
    ref = y64.reshape(e, heads * M) * (norm if scaled else 1.0)
    r1 = rel(got.float().cpu().numpy(), ref)
    assert r1 <= tol, ('gather', r1)
    scale = rng.uniform(0.5, 2, (n_rel, heads)).astype(np.float32)
    want = np.einsum('ehm,ehm->eh', y64, Q[oth].reshape(e, heads, M).astype(np.float64)) * scale[etype]
    got = ops.SegmentMMEdgeDot(dX, dW, which, dQ, 1 - which, g, scale=D(scale))
    r2 = rel(got.cpu().numpy(), want)
    assert r2 <= tol, ('dot', r2)
    # plain typed product on per-edge rows
    Xe = rng.standard_normal((e, heads * K), dtype=np.float32)
    if bf16:
        Xe = to_bf16_f32(Xe)
    got = ops.SegmentMMEdge(D(Xe, bf16), dW, g)
    ref = np.einsum('ehk,ehkm->ehm', Xe.reshape(e, heads, K).astype(np.float64), W[etype].astype(np.float64)).reshape(e, heads * M) if e else np.zeros((0, heads * M))
    r3 = rel(got.float().cpu().numpy(), ref)
    assert r3 <= tol, ('segmm', r3)
    # softmax-weighted sum of per-edge rows and the two fused GAT passes
    dim = int(rng.choice([1, 4, 8, 16, 24, 32, 64]))
    H2 = int(rng.choice([1, 2, 3, 4, 8]))
    logit = (rng.standard_normal((e, H2)) * 3).astype(np.float32)
    m = rng.standard_normal((e, H2 * dim), dtype=np.float32)
    if bf16:
        m = to_bf16_f32(m)
    att = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, logit)
    prod = (m.reshape(e, H2, dim).astype(np.float64) * att[:, :, None]).reshape(e, H2 * dim)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices, prod.astype(np.float32), op='copy_e')
    got = ops.edge_softmax_sum(D(logit), D(m, bf16), g)
    r4 = rel(got.float().cpu().numpy(), ref)
    assert r4 <= tol, ('ess', r4)
    z = rng.standard_normal((n, H2 * dim), dtype=np.float32)
    if bf16:
        z = to_bf16_f32(z)
    a_l = (rng.standard_normal((H2, dim)) / np.sqrt(dim)).astype(np.float32)
    er = rng.standard_normal((n, H2), dtype=np.float32)
    el = np.einsum('nhd,hd->nh', z.reshape(n, H2, dim).astype(np.float64), a_l).astype(np.float32)
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, z, heads=H2, slope=0.2)
    got = ops.gat_aggregate(D(el), D(er), D(z, bf16), g, 0.2)
    r5 = rel(got.float().cpu().numpy().reshape(ref.shape), ref)
    assert r5 <= tol, ('gat', r5)
    try:
        got = ops.gat_aggregate_from_z(D(a_l), D(er), D(z, bf16), g, 0.2)
        r6 = rel(got.float().cpu().numpy().reshape(ref.shape), ref)
        assert r6 <= max(tol, 0.0001), ('gatz', r6)
    except capi.GraphilerError as err:
        assert err.code == capi.GA_EUNSUPPORTED
    # projection with attention terms
    rows = int(rng.integers(1, 700))
    Kp = int(rng.choice([8, 16, 40, 100, 128, 200, 256]))
    dph = int(rng.choice([16, 32, 64, 128]))
    Hp = int(rng.choice([1, 2, 4]))
    Mp = dph * Hp
    if Mp <= 512:
        x = rng.standard_normal((rows, Kp), dtype=np.float32)
        w = (rng.standard_normal((Kp, Mp)) / np.sqrt(Kp)).astype(np.float32)
        a = rng.standard_normal((2, Hp, dph), dtype=np.float32)
        if bf16:
            (x, w) = (to_bf16_f32(x), to_bf16_f32(w))
        try:
            (zz, l, r) = ops.linear_attn(D(x, bf16), D(w, bf16), D(a[0]), D(a[1]))
            zr = x.astype(np.float64) @ w.astype(np.float64)
            r7 = rel(zz.float().cpu().numpy(), zr)
            assert r7 <= tol, ('proj z', r7)
            r8 = rel(l.cpu().numpy(), (zr.reshape(rows, Hp, dph) * a[0]).sum(-1))
            assert r8 <= 0.0001, ('proj el', r8)
            r9 = rel(r.cpu().numpy(), (zr.reshape(rows, Hp, dph) * a[1]).sum(-1))
            assert r9 <= 0.0001, ('proj er', r9)
        except capi.GraphilerError as err:
            assert err.code == capi.GA_EUNSUPPORTED

@pytest.mark.parametrize('seed', range(1, 65))
def test_random_graphs_core_operators(device, seed):
    """The reference's operators on random graphs (uniform, Zipf-skewed or
    pre-sorted destinations; 0 to 20,000 edges), random head counts and widths,
    fp32 or bf16: every SpMM operator x reducer, the out-adjacency form, SDDMM
    add / sub / mul / div (bit-exact) and dot, multi-head softmax, the gather and
    the device-side graph preparation (bit-exact)."""
    dev = device

    def D(a, bf16=False):
        t = torch.from_numpy(np.ascontiguousarray(a)).to(dev)
        return t.bfloat16() if bf16 else t
    rng = np.random.default_rng(seed)
    bf16 = bool(rng.integers(0, 2))
    tol = 0.02 if bf16 else 2e-05
    n = int(rng.integers(1, 600))
    e = int(rng.choice([0, 1, 5, 60, 700, 5000, 20000]))
    src = rng.integers(0, n, e, dtype=np.int64)
    kind = rng.integers(0, 3)
    if kind == 0:
        dst = rng.integers(0, n, e, dtype=np.int64)
    elif kind == 1:
        dst = (rng.zipf(1.6, e) % n).astype(np.int64)
    else:
        dst = np.sort(rng.integers(0, max(1, n // 3), e, dtype=np.int64))
    g = prepare_graph(src, dst, n, device=dev)
    arr = build_graph_arrays(src, dst, n)
    heads = int(rng.choice([1, 1, 2, 4, 8]))
    dim = int(rng.choice([1, 2, 3, 4, 8, 16, 17, 32, 64, 128]))
    feat = heads * dim
    x = rng.standard_normal((n, feat), dtype=np.float32)
    m = rng.standard_normal((e, feat), dtype=np.float32)
    w = rng.uniform(0.2, 2.0, (e, heads)).astype(np.float32)
    if bf16:
        (x, m) = (to_bf16_f32(x), to_bf16_f32(m))
    op = str(rng.choice(['copy_u', 'copy_e', 'u_mul_e', 'u_add_e', 'u_sub_e', 'u_div_e']))
    red = str(rng.choice(['sum', 'max', 'min']))
    u = m if op == 'copy_e' else x
    ww = None if op in ('copy_u', 'copy_e') else w
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices, u, ww, op=op, reduce=red, heads=heads)
    got = ops.spmm(g, op, red, D(u, bf16), None if ww is None else D(ww))
    r = rel_err(got.float().cpu().numpy().reshape(ref.shape), ref)
    assert r <= tol, (op, red, r)
    ref = oracle.spmm(arr.out_pointer, arr.out_node_indices, arr.out_edge_indices, x, w, op='u_mul_e', heads=heads)
    got = ops.gspmm_dst_mul_e_sum(D(x, bf16), D(w), [1], False, None, g)
    r = rel_err(got.float().cpu().numpy().reshape(ref.shape), ref)
    assert r <= tol, ('dst_mul_e', r)
    uu = rng.standard_normal((n, heads), dtype=np.float32)
    vv = rng.standard_normal((n, heads), dtype=np.float32)
    got = ops.gsddmm_u_add_v_mul_alpha(D(uu), D(vv), 1, g)
    assert np.array_equal(got.cpu().numpy(), oracle.sddmm_u_add_v(src, dst, uu, vv)), 'u_add_v'
    sop = str(rng.choice(['sub', 'mul', 'div']))
    got = ops.gsddmm_u_op_v(sop, D(uu), D(vv + 3), g)
    assert np.array_equal(got.cpu().numpy(), oracle.sddmm_u_op_v(sop, src, dst, uu, vv + 3)), 'u_op_v'
    k3 = x.reshape(n, heads, dim)
    got = ops.gsddmm_u_dot_v(D(k3, bf16), D(k3, bf16), g)
    r = rel_err(got.cpu().numpy(), oracle.sddmm_u_dot_v(src, dst, k3, k3))
    assert r <= 2e-05, ('dot', r)
    lg = (rng.standard_normal((e, heads)) * 4).astype(np.float32)
    got = ops.SegmentSoftmax(D(lg), 1, None, g)
    r = rel_err(got.cpu().numpy(), oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, lg))
    assert r <= 2e-05, ('softmax', r)
    got = ops.BroadcastSrcNode(D(x, bf16), g)
    assert np.array_equal(got.float().cpu().numpy(), x[src]), 'gather'
    for (a, b) in ((g.in_pointer, arr.in_pointer), (g.in_node_indices, arr.in_node_indices), (g.in_edge_indices, arr.in_edge_indices), (g.out_pointer, arr.out_pointer), (g.out_node_indices, arr.out_node_indices), (g.out_edge_indices, arr.out_edge_indices)):
        assert np.array_equal(a.cpu().numpy(), b), 'prep'
