"""Parity at the benchmark configurations' full sizes.

Configs 2-4 are small enough for the C oracle to evaluate completely; config 5
(64 M edges x 256 features) is checked on every row of a seeded sample (the
oracle runs on the sub-adjacency of the sampled destinations, including the
highest-degree row) and through size-independent properties: the column sums
of an SpMM equal the sums of its messages, and every softmax segment sums to 1.
"""
import numpy as np
import pytest
import torch

import oracle
from graphiler_amd import datasets, layers, ops, prepare_graph
from helpers import TOL_BF16, TOL_F32, assert_close, to_bf16_f32

pytestmark = pytest.mark.gpu


def _t(a, device, bf16=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(device)
    return t.to(torch.bfloat16) if bf16 else t


def _host(g):
    return (g.in_pointer.cpu().numpy(), g.in_node_indices.cpu().numpy(),
            g.in_edge_indices.cpu().numpy())


def test_config2_gat_full(device):
    wl = datasets.gat_rmat()                     # N=232,965  E=11.6 M
    n, e = wl.num_nodes, wl.num_edges
    g = prepare_graph(wl.src, wl.dst, n, device=device)
    ptr, nbr, eid = _host(g)
    assert g.in_eid_is_identity and np.array_equal(eid, np.arange(e, dtype=np.int32))
    # the grouping done on the GPU against the oracle's, both directions, bit-exact
    for want, got in zip(oracle.group_edges(n, wl.dst, wl.src), (ptr, nbr, eid)):
        assert np.array_equal(want, got)
    for want, got in zip(oracle.group_edges(n, wl.src, wl.dst),
                         (g.out_pointer, g.out_node_indices, g.out_edge_indices)):
        assert np.array_equal(want, got.cpu().numpy())
    rng = np.random.default_rng(1)
    z = rng.standard_normal((n, 64), dtype=np.float32)
    el = rng.standard_normal((n, 1), dtype=np.float32)
    er = rng.standard_normal((n, 1), dtype=np.float32)
    dz, dl, dr = _t(z, device), _t(el, device), _t(er, device)
    ref = oracle.gat_aggregate(ptr, nbr, el, er, z, heads=1, slope=0.2)
    assert_close(ops.gat_aggregate(dl, dr, dz, g, 0.2).cpu().numpy(), ref, TOL_F32,
                 "config 2 fused GAT")
    logits = ops.gsddmm_u_add_v_mul_alpha(dl, dr, 1, g)
    assert np.array_equal(logits.cpu().numpy(),
                          oracle.sddmm_u_add_v(wl.src, wl.dst, el, er))
    att = ops.SegmentSoftmax(torch.nn.functional.leaky_relu(logits, 0.2), 1, None, g)
    out = ops.gspmm_src_mul_e_sum(dz, att, [1], False, None, g)
    assert_close(out.cpu().numpy(), ref, TOL_F32, "config 2 four-operator plan")
    # max over in-edges, bit-exact (values are copies)
    got = ops.spmm(g, "copy_u", "max", dz).cpu().numpy()
    assert np.array_equal(got, oracle.spmm(ptr, nbr, eid, z, op="copy_u", reduce="max"))


@pytest.mark.parametrize("bf16", [False, True])
def test_config3_rgcn_full(device, bf16):
    wl = datasets.rgcn_zipf()                    # N=100k  E=1M  R=60
    n = wl.num_nodes
    g = prepare_graph(wl.src, wl.dst, n, device=device, etype_of=wl.etype,
                      num_etypes=60)
    ptr, nbr, eid = _host(g)
    rng = np.random.default_rng(2)
    x = rng.standard_normal((n, 16), dtype=np.float32)
    w1 = datasets.glorot(rng, (60, 16, 64))
    if bf16:
        x, w1 = to_bf16_f32(x), to_bf16_f32(w1)
    deg = np.maximum(np.bincount(wl.dst, minlength=n), 1)
    norm = (1.0 / deg[wl.dst]).astype(np.float32)[:, None]
    got = layers.rgcn_layer(g, _t(x, device, bf16), _t(w1, device, bf16), _t(norm, device))
    etp = oracle.type_pointer(wl.etype, 60)
    msg = oracle.segment_mm(etp, oracle.gather_rows(wl.src, x), w1) * norm
    ref = oracle.spmm(ptr, nbr, eid, msg.astype(np.float32), op="copy_e")
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 "config 3 RGCN layer 1 (16 -> 64)")
    # second layer (64 -> 8) on the device's own first-layer output after relu, so that
    # the check is of this layer alone
    w2 = datasets.glorot(rng, (60, 64, 8))
    if bf16:
        w2 = to_bf16_f32(w2)
    h1 = torch.relu(got)
    got2 = layers.rgcn_layer(g, h1, _t(w2, device, bf16), _t(norm, device))
    h1_h = h1.float().cpu().numpy()
    msg = oracle.segment_mm(etp, oracle.gather_rows(wl.src, h1_h), w2) * norm
    ref2 = oracle.spmm(ptr, nbr, eid, msg.astype(np.float32), op="copy_e")
    assert_close(got2.float().cpu().numpy(), ref2, TOL_BF16 if bf16 else TOL_F32,
                 "config 3 RGCN layer 2 (64 -> 8)")


def test_config4_hgt_operators_full(device):
    wl = datasets.hgt_hetero()                   # N=100k  E=2M  8 heads x 16
    n, e, heads, d = wl.num_nodes, wl.num_edges, 8, 16
    g = prepare_graph(wl.src, wl.dst, n, device=device, ntype_of=wl.ntype,
                      num_ntypes=4, etype_of=wl.etype, num_etypes=10)
    ptr, nbr, eid = _host(g)
    rng = np.random.default_rng(3)
    h = to_bf16_f32(rng.standard_normal((n, 128), dtype=np.float32))
    wq = to_bf16_f32(datasets.glorot(rng, (4, 128, 128)))
    q = ops.SegmentMMNode(_t(h, device, True), _t(wq, device, True), g)
    q_ref = oracle.segment_mm(oracle.type_pointer(wl.ntype, 4), h, wq)
    assert_close(q.float().cpu().numpy(), q_ref, TOL_BF16, "config 4 Q projection")
    ke = to_bf16_f32(rng.standard_normal((e, 128), dtype=np.float32))
    ratt = to_bf16_f32(datasets.glorot(rng, (10, heads, d, d)))
    got = ops.SegmentMMEdge(_t(ke, device, True), _t(ratt, device, True), g)
    ref = oracle.segment_mm(oracle.type_pointer(wl.etype, 10), ke, ratt, heads=heads)
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16, "config 4 relation transform")
    k3 = h.reshape(n, heads, d)
    dot = ops.gsddmm_u_dot_v(_t(k3, device, True), _t(k3, device, True), g)
    assert_close(dot.cpu().numpy(), oracle.sddmm_u_dot_v(wl.src, wl.dst, k3, k3),
                 TOL_F32, "config 4 u_dot_v")
    logits = (rng.standard_normal((e, heads)) * 3).astype(np.float32)
    att = ops.SegmentSoftmax(_t(logits, device), 1, None, g)
    att_ref = oracle.segment_softmax(ptr, eid, logits)
    assert_close(att.cpu().numpy(), att_ref, TOL_F32, "config 4 softmax")
    out = ops.gspmm_src_mul_e_sum(_t(h, device, True), att, [1], False, None, g)
    ref = oracle.spmm(ptr, nbr, eid, h, att_ref, op="u_mul_e", heads=heads)
    assert_close(out.float().cpu().numpy(), ref, TOL_BF16, "config 4 u_mul_e")


def test_config4_hgt_fused_operators_full(device):
    """The fused forms at config 4's size (2 M edges, 8 heads x 16, bf16): typed
    product through the COO column, its dot epilogue with the relation prior,
    and the softmax-weighted sum of per-edge rows; expected values from the
    oracle's segment_mm / softmax / copy_e sum on numpy-gathered rows."""
    wl = datasets.hgt_hetero()
    n, e, heads, d = wl.num_nodes, wl.num_edges, 8, 16
    g = prepare_graph(wl.src, wl.dst, n, device=device, ntype_of=wl.ntype,
                      num_ntypes=4, etype_of=wl.etype, num_etypes=10)
    ptr, nbr, eid = _host(g)
    rng = np.random.default_rng(33)
    k = to_bf16_f32(rng.standard_normal((n, 128), dtype=np.float32))
    q = to_bf16_f32(rng.standard_normal((n, 128), dtype=np.float32))
    ratt = to_bf16_f32(datasets.glorot(rng, (10, heads, d, d)))
    pri = rng.uniform(0.5, 1.5, (10, heads)).astype(np.float32)
    etp = oracle.type_pointer(wl.etype, 10)
    ke = oracle.segment_mm(etp, oracle.gather_rows(wl.src, k), ratt, heads=heads)   # fp32, unrounded
    got = ops.SegmentMMEdgeGather(_t(k, device, True), _t(ratt, device, True), 0, g)
    assert_close(got.float().cpu().numpy(), ke, TOL_BF16, "config 4 gathered relation transform")
    want = (ke.reshape(e, heads, d).astype(np.float64) *
            oracle.gather_rows(wl.dst, q).reshape(e, heads, d)).sum(-1) * pri[wl.etype]
    score = ops.SegmentMMEdgeDot(_t(k, device, True), _t(ratt, device, True), 0,
                                 _t(q, device, True), 1, g, scale=_t(pri, device))
    assert_close(score.cpu().numpy(), want, TOL_F32, "config 4 attention scores")
    # reduce tail on the device's own scores (scaled down to softmax range)
    logits = (want / 8).astype(np.float32)
    ve = to_bf16_f32(rng.standard_normal((e, 128), dtype=np.float32))
    att = oracle.segment_softmax(ptr, eid, logits)
    msg = (ve.reshape(e, heads, d).astype(np.float64) * att[:, :, None]).reshape(e, 128)
    ref = oracle.spmm(ptr, nbr, eid, msg.astype(np.float32), op="copy_e")
    out = ops.edge_softmax_sum(_t(logits, device), _t(ve, device, True), g)
    assert_close(out.float().cpu().numpy(), ref, TOL_BF16, "config 4 softmax-weighted sum")


@pytest.mark.timeout(400)
def test_config5_large_gat_sampled_and_properties(device):
    wl = datasets.gat_rmat_large()               # N=2,449,029  E=64,308,169
    n, e, heads, d = wl.num_nodes, wl.num_edges, 4, 64
    assert e == 61_859_140 + n
    deg = np.bincount(wl.dst, minlength=n)
    assert deg.max() > 10_000, "config 5 must exercise long segments"
    g = prepare_graph(wl.src, wl.dst, n, device=device)
    ptr = g.in_pointer.cpu().numpy()
    # index work is bit-exact: pointer = running sum of in-degrees, rows sorted
    assert np.array_equal(np.diff(ptr), deg)
    assert np.array_equal(g.in_node_indices.cpu().numpy(), wl.src.astype(np.int32))
    rows_dev = g.in_row_of_slot
    assert torch.equal(rows_dev.long(), _t(wl.dst, device))
    rng = np.random.default_rng(4)
    z = to_bf16_f32(rng.standard_normal((n, heads * d), dtype=np.float32))
    el = rng.standard_normal((n, heads), dtype=np.float32)
    er = rng.standard_normal((n, heads), dtype=np.float32)
    dz, dl, dr = _t(z, device, True), _t(el, device), _t(er, device)
    out = ops.gat_aggregate(dl, dr, dz, g, 0.2).float().cpu().numpy()
    # oracle on the sub-adjacency of sampled destinations (+ the heaviest rows)
    sample = np.unique(np.concatenate([rng.integers(0, n, 3000),
                                       np.argsort(deg)[-3:], [0, n - 1]]))
    sub_ptr = np.concatenate([[0], np.cumsum(deg[sample])]).astype(np.int32)
    sub_nbr = np.concatenate([wl.src[ptr[v]:ptr[v + 1]] for v in sample]).astype(np.int32)
    ref = oracle.gat_aggregate(sub_ptr, sub_nbr, el, er[sample], z, heads=heads, slope=0.2)
    assert_close(out[sample], ref, TOL_BF16, "config 5 fused GAT (sampled rows)")
    assert not out[deg == 0].any()
    # the variant that recomputes the source term from the gathered rows
    a_l = (rng.standard_normal((heads, d)) / 8).astype(np.float32)
    el2 = np.einsum("nhd,hd->nh", z.reshape(n, heads, d).astype(np.float64), a_l).astype(np.float32)
    out2 = ops.gat_aggregate_from_z(_t(a_l, device), dr, dz, g, 0.2).float().cpu().numpy()
    ref2 = oracle.gat_aggregate(sub_ptr, sub_nbr, el2, er[sample], z, heads=heads, slope=0.2)
    assert_close(out2[sample], ref2, TOL_BF16, "config 5 fused GAT, source term from z")
    assert not out2[deg == 0].any()
    # properties over ALL rows: softmax segments sum to one; SpMM column sums
    logits = ops.gsddmm_u_add_v_mul_alpha(dl, dr, 1, g)
    att = ops.SegmentSoftmax(logits, 1, None, g)
    sums = ops.SpMMEdge(att, [1], False, None, g).cpu().numpy()
    assert np.abs(sums[deg > 0] - 1.0).max() < 1e-4
    assert not sums[deg == 0].any()
    x32 = torch.randn(n, 16, device=device)
    col = ops.SpMMSrc(x32, [1], False, None, g).double().sum(0).cpu().numpy()
    want = (x32.double() * _t(np.bincount(wl.src, minlength=n).astype(np.float64),
                              device)[:, None]).sum(0).cpu().numpy()
    np.testing.assert_allclose(col, want, rtol=1e-6, atol=1e-3 * np.abs(want).max())


@pytest.mark.timeout(600)
def test_config5_three_layer_network_layer_by_layer(device):
    """The 3-layer network of configuration 5 (100 -> 256 -> 256 -> 256, 4 heads x 64,
    bf16 storage, elu between layers) at full size.  Each layer is checked on its own:
    the oracle gets the device's input to that layer and is evaluated on sampled
    destination rows plus the three heaviest ones (their in-edges reach most of the
    graph's nodes, so the projection is computed for every node, in fp32 on the host)."""
    wl = datasets.gat_rmat_large()
    n, heads, d = wl.num_nodes, 4, 64
    deg = np.bincount(wl.dst, minlength=n)
    g = prepare_graph(wl.src, wl.dst, n, device=device)
    ptr = g.in_pointer.cpu().numpy()
    rng = np.random.default_rng(45)
    sample = np.unique(np.concatenate([rng.integers(0, n, 2000), np.argsort(deg)[-3:], [0, n - 1]]))
    sub_ptr = np.concatenate([[0], np.cumsum(deg[sample])]).astype(np.int32)
    sub_nbr = np.concatenate([wl.src[ptr[v]:ptr[v + 1]] for v in sample]).astype(np.int32)
    x = _t(to_bf16_f32(rng.standard_normal((n, 100), dtype=np.float32)), device, True)
    for layer, k in enumerate((100, 256, 256)):
        w = to_bf16_f32(datasets.glorot(rng, (k, heads * d)))
        a = datasets.glorot(rng, (2, heads, d), fan_in=2 * d, fan_out=1)
        out = layers.gat_layer(g, x, _t(w, device, True), _t(a, device), heads, 0.2, fused=True)
        x_h = x.float().cpu().numpy()
        z32 = x_h @ w                                        # fp32 accumulate, like the device
        zh = z32.reshape(n, heads, d)
        el = (zh * a[0]).sum(-1).astype(np.float32)
        er = (zh * a[1]).sum(-1).astype(np.float32)
        z = to_bf16_f32(z32)                                 # the rows the aggregation reads are stored bf16
        ref = oracle.gat_aggregate(sub_ptr, sub_nbr, el, er[sample], z, heads=heads, slope=0.2)
        assert_close(out.float().cpu().numpy()[sample], ref, TOL_BF16,
                     f"config 5 network, layer {layer + 1} ({k} -> 256), sampled rows")
        x = torch.nn.functional.elu(out)


def _hgt_reference(wl, ptr, nbr, eid, h, wk, wq, wv, wa, ratt, rmsg, rpri, skip, heads, d, cast):
    """The unfused HGT plan (examples/HGT/HGT.py:28-60, one (D x D) block per head) on
    the oracle; ``cast`` rounds where the device stores tensors of the feature dtype.
    Returns (K, Q, V, t, out): node projections, the aggregate, the layer output."""
    n, e, hid = wl.num_nodes, wl.num_edges, heads * d
    ntp, etp = oracle.type_pointer(wl.ntype, 4), oracle.type_pointer(wl.etype, 10)
    K = cast(oracle.segment_mm(ntp, h, wk))
    V = cast(oracle.segment_mm(ntp, h, wv))
    Q = cast(oracle.segment_mm(ntp, h, wq))
    k_e = oracle.segment_mm(etp, oracle.gather_rows(wl.src, K), ratt, heads=heads)
    q_e = oracle.gather_rows(wl.dst, Q)
    attn = np.einsum("ehd,ehd->eh", k_e.reshape(e, heads, d).astype(np.float64),
                     q_e.reshape(e, heads, d))
    del k_e, q_e
    attn = (attn * rpri[wl.etype] / np.sqrt(d)).astype(np.float32)
    a = oracle.segment_softmax(ptr, eid, attn)
    v_e = oracle.segment_mm(etp, oracle.gather_rows(wl.src, V), rmsg, heads=heads)
    m = (v_e.reshape(e, heads, d) * a[:, :, None]).reshape(e, hid).astype(np.float32)
    del v_e
    t = oracle.spmm(ptr, nbr, eid, m, op="copy_e")
    gate = (1.0 / (1.0 + np.exp(-skip[wl.ntype])))[:, None]
    return K, Q, V, t, oracle.segment_mm(ntp, cast(t), wa) * gate


@pytest.mark.timeout(600)
@pytest.mark.parametrize("bf16", [True, False])
def test_config4_hgt_layer_pair_form_full(device, bf16, monkeypatch):
    """The path the benchmark times at config 4: ``hgt_layer(fused=True)``, which on this
    graph (2 M edges, 269,078 (destination, relation) pairs) applies the relation
    matrices per pair, and ``relation_pair_attention`` on its own, both against the
    unfused plan evaluated by the oracle on all 2 M edges."""
    wl = datasets.hgt_hetero()
    n, heads, d = wl.num_nodes, 8, 16
    hid = heads * d
    g = prepare_graph(wl.src, wl.dst, n, device=device, ntype_of=wl.ntype,
                      num_ntypes=4, etype_of=wl.etype, num_etypes=10)
    ptr, nbr, eid = _host(g)
    pairs = g.relation_pairs()
    key = wl.dst.astype(np.int64) * 10 + wl.etype
    assert pairs is not None and pairs.num_pairs == len(np.unique(key))
    assert wl.num_edges >= layers.PAIRS_MIN_EDGES_PER_PAIR * pairs.num_pairs
    cast = to_bf16_f32 if bf16 else (lambda a: np.asarray(a, dtype=np.float32))
    tol = TOL_BF16 if bf16 else TOL_F32
    rng = np.random.default_rng(34)
    h = cast(rng.standard_normal((n, hid), dtype=np.float32))
    wk, wq, wv, wa = (cast(datasets.glorot(rng, (4, hid, hid))) for _ in range(4))
    ratt, rmsg = (cast(datasets.glorot(rng, (10, heads, d, d))) for _ in range(2))
    rpri = cast(rng.uniform(0.5, 1.5, (10, heads)).astype(np.float32))
    skip = rng.standard_normal(4).astype(np.float32)
    K, Q, V, t_ref, out_ref = _hgt_reference(wl, ptr, nbr, eid, h, wk, wq, wv, wa, ratt, rmsg,
                                             rpri, skip, heads, d, cast)
    calls = []
    real = ops.relation_pair_attention

    def counted(*a, **kw):
        calls.append(1)
        return real(*a, **kw)

    monkeypatch.setattr(ops, "relation_pair_attention", counted)
    got = layers.hgt_layer(g, _t(h, device, bf16), _t(wk, device, bf16), _t(wq, device, bf16),
                           _t(wv, device, bf16), _t(wa, device, bf16), _t(ratt, device, bf16),
                           _t(rmsg, device, bf16), _t(rpri, device, bf16), _t(skip, device),
                           heads, fused=True)
    assert calls == [1], "the layer must take the per-pair form on this graph"
    assert_close(got.float().cpu().numpy(), out_ref, tol, f"config 4 HGT layer, pairs, bf16={bf16}")
    # the attention stage alone, on the oracle's own (rounded) K, Q, V
    t = real(_t(K, device, bf16), _t(Q, device, bf16), _t(V, device, bf16), _t(ratt, device, bf16),
             _t(rmsg, device, bf16), _t(rpri, device), g, factor=1.0 / np.sqrt(d))
    assert_close(t.float().cpu().numpy(), t_ref, tol,
                 f"config 4 relation_pair_attention, bf16={bf16}")
    # and the per-edge form of the same layer
    per_edge = layers.hgt_layer(g, _t(h, device, bf16), _t(wk, device, bf16), _t(wq, device, bf16),
                                _t(wv, device, bf16), _t(wa, device, bf16), _t(ratt, device, bf16),
                                _t(rmsg, device, bf16), _t(rpri, device, bf16), _t(skip, device),
                                heads, fused="edges")
    assert calls == [1]
    assert_close(per_edge.float().cpu().numpy(), out_ref, tol,
                 f"config 4 HGT layer, per edge, bf16={bf16}")


@pytest.mark.parametrize("bf16", [False, True])
def test_config3_rgcn_network_with_fused_relu_full(device, bf16):
    """The calls the benchmark times at config 3: layer 1 with the relu applied by the
    one-pass kernel to the sums it stores, layer 2 plain on that output."""
    wl = datasets.rgcn_zipf()
    n = wl.num_nodes
    g = prepare_graph(wl.src, wl.dst, n, device=device, etype_of=wl.etype, num_etypes=60)
    ptr, nbr, eid = _host(g)
    rng = np.random.default_rng(22)
    x = rng.standard_normal((n, 16), dtype=np.float32)
    w1, w2 = datasets.glorot(rng, (60, 16, 64)), datasets.glorot(rng, (60, 64, 8))
    if bf16:
        x, w1, w2 = to_bf16_f32(x), to_bf16_f32(w1), to_bf16_f32(w2)
    deg = np.maximum(np.bincount(wl.dst, minlength=n), 1)
    norm = (1.0 / deg[wl.dst]).astype(np.float32)[:, None]
    etp = oracle.type_pointer(wl.etype, 60)
    tol = TOL_BF16 if bf16 else TOL_F32

    def ref_layer(hh, w):
        msg = oracle.segment_mm(etp, oracle.gather_rows(wl.src, hh), w) * norm
        return oracle.spmm(ptr, nbr, eid, msg.astype(np.float32), op="copy_e")

    assert ops.typed_spmm_preferred(_t(x, device, bf16), _t(w1, device, bf16))
    h1 = layers.rgcn_layer(g, _t(x, device, bf16), _t(w1, device, bf16), _t(norm, device),
                           fused=True, activation="relu")
    r1 = np.maximum(ref_layer(x, w1), 0)
    assert_close(h1.float().cpu().numpy(), r1, tol, "config 3 layer 1 with relu in the kernel")
    assert bool((h1 == 0).any()) and not bool((h1 < 0).any())
    h2 = layers.rgcn_layer(g, h1, _t(w2, device, bf16), _t(norm, device), fused=True)
    assert_close(h2.float().cpu().numpy(), ref_layer(h1.float().cpu().numpy(), w2), tol,
                 "config 3 layer 2 on the device's layer 1")
    # elu through the same epilogue
    e1 = layers.rgcn_layer(g, _t(x, device, bf16), _t(w1, device, bf16), _t(norm, device),
                           fused=True, activation="elu")
    pre = ref_layer(x, w1).astype(np.float64)
    assert_close(e1.float().cpu().numpy(), np.where(pre > 0, pre, np.expm1(pre)), tol,
                 "config 3 layer 1 with elu in the kernel")


@pytest.mark.timeout(600)
def test_config5_network_as_benchmarked(device):
    """The three calls of the benchmarked network, ``gat_layer(..., fused=True,
    activation="elu")`` for the hidden layers and no activation on the last one, each on
    the device's own previous output; sampled destination rows and the heaviest ones."""
    wl = datasets.gat_rmat_large()
    n, heads, d = wl.num_nodes, 4, 64
    deg = np.bincount(wl.dst, minlength=n)
    g = prepare_graph(wl.src, wl.dst, n, device=device)
    ptr = g.in_pointer.cpu().numpy()
    rng = np.random.default_rng(46)
    sample = np.unique(np.concatenate([rng.integers(0, n, 2000), np.argsort(deg)[-3:], [0, n - 1]]))
    sub_ptr = np.concatenate([[0], np.cumsum(deg[sample])]).astype(np.int32)
    sub_nbr = np.concatenate([wl.src[ptr[v]:ptr[v + 1]] for v in sample]).astype(np.int32)
    x = _t(to_bf16_f32(rng.standard_normal((n, 100), dtype=np.float32)), device, True)
    for layer, k in enumerate((100, 256, 256)):
        act = "elu" if layer < 2 else None
        w = to_bf16_f32(datasets.glorot(rng, (k, heads * d)))
        a = datasets.glorot(rng, (2, heads, d), fan_in=2 * d, fan_out=1)
        out = layers.gat_layer(g, x, _t(w, device, True), _t(a, device), heads, 0.2, fused=True,
                               activation=act)
        z32 = x.float().cpu().numpy() @ w
        zh = z32.reshape(n, heads, d)
        z = to_bf16_f32(z32)
        # the source term as the pass forms it: from the stored (rounded) rows
        el = (z.reshape(n, heads, d) * a[0]).sum(-1).astype(np.float32)
        er = (zh * a[1]).sum(-1).astype(np.float32)
        ref = oracle.gat_aggregate(sub_ptr, sub_nbr, el, er[sample], z, heads=heads,
                                   slope=0.2).astype(np.float64)
        if act:
            ref = np.where(ref > 0, ref, np.expm1(ref))
        assert_close(out.float().cpu().numpy()[sample], ref, TOL_BF16,
                     f"config 5 network as benchmarked, layer {layer + 1} ({k} -> 256, {act})")
        x = out


@pytest.mark.timeout(600)
def test_tensors_beyond_two_to_the_31_elements(device):
    """Per-edge tensors of config 5's graph with 40 features: 2.57 G elements, 10.3 GB --
    every offset past 2^31 elements / 2^32 bytes.  References are torch's own indexing
    and float64 scatter-adds on the GPU (independent kernels)."""
    wl = datasets.gat_rmat_large()
    n, e, feat = wl.num_nodes, wl.num_edges, 40
    assert e * feat > 2 ** 31
    g = prepare_graph(wl.src, wl.dst, n, device=device)
    src, dst = _t(wl.src, device), _t(wl.dst, device)
    gen = torch.Generator(device=device).manual_seed(3)
    x = torch.randn(n, feat, device=device, generator=gen)
    y = torch.randn(n, feat, device=device, generator=gen)

    def summed(rows):           # float64 scatter-add by destination
        return torch.zeros(n, feat, device=device, dtype=torch.float64).index_add_(0, dst, rows.double())

    assert torch.equal(ops.BroadcastSrcNode(x, g), x[src])
    assert torch.equal(ops.BroadcastDstNode(x, g), x[dst])
    m = ops.gsddmm_u_add_v_mul_alpha(x, y, 1, g)                    # (E, 40): the per-edge tensor below
    want = x[src]
    want += y[dst]
    assert m.shape == (e, feat) and torch.equal(m, want)
    want = x[src]
    want *= m
    assert torch.equal(ops.gsddmm(g, "mul", x, m, "u", "e"), want)
    del want
    got = ops.SpMMEdge(m, [1], False, None, g)
    ref, mag = summed(m), summed(m.abs())
    assert float(((got - ref).abs() / mag.clamp_min(1e-30)).max()) <= TOL_F32, "SpMMEdge"
    assert torch.equal(ops.spmm_scaled(m, g, activation="relu", edge_rows=True), torch.relu(got))
    del got, ref, mag
    w = torch.rand(e, 1, device=device, generator=gen)
    got = ops.gspmm_src_mul_e_sum(x, w, [1], False, None, g)
    xw = x[src] * w
    assert float(((got - summed(xw)).abs() / summed(xw.abs()).clamp_min(1e-30)).max()) <= TOL_F32, "u_mul_e"
    del xw, got
    sm = ops.SegmentSoftmax(m, 1, None, g)                          # 40 heads: the 64-lane-head layout
    deg = torch.bincount(dst, minlength=n)
    sums = summed(sm)[deg > 0]
    assert float((sums - 1).abs().max()) <= 2e-5
    ptr = g.in_pointer.long()
    for v in (0, 1, int(deg.argmax()), n - 1, n // 2, 12345, 2_000_000):
        a, b = int(ptr[v]), int(ptr[v + 1])
        if b > a:
            assert torch.allclose(sm[a:b], torch.softmax(m[a:b].double(), 0).float(), rtol=2e-5, atol=1e-9)
    del sm, sums
    logit = torch.randn(e, 8, device=device, generator=gen)         # 8 heads x 5
    got = ops.edge_softmax_sum(logit, m, g)
    att = ops.SegmentSoftmax(logit, 1, None, g)
    ref = summed((m.view(e, 8, 5) * att.unsqueeze(-1)).view(e, feat))
    assert float((got - ref).abs().max()) <= TOL_F32 * float(ref.abs().max()), "edge_softmax_sum"
    del got, ref, att, logit, m
    torch.cuda.empty_cache()
    # typed products: (E, 32) @ (T, 32, 40) -> (E, 40)
    from graphiler_amd.graph import sort_edges_by_type
    n_types = 4
    et = np.sort(np.random.default_rng(5).integers(0, n_types, e))
    s2, d2, et2, _ = sort_edges_by_type(wl.src, wl.dst, et)
    gt = prepare_graph(s2, d2, n, device=device, etype_of=et2, num_etypes=n_types)
    xe = torch.randn(e, 32, device=device, generator=gen)
    xn = torch.randn(n, 32, device=device, generator=gen)
    wt = torch.randn(n_types, 32, feat, device=device, generator=gen) / 6
    per_edge, gathered = ops.SegmentMMEdge(xe, wt, gt), ops.SegmentMMEdgeGather(xn, wt, 0, gt)
    tp, s2d = gt.etype_pointer.cpu().numpy(), _t(s2, device)
    for t in range(n_types):
        a, b = int(tp[t]), int(tp[t + 1])
        for got, rows in ((per_edge, xe[a:b]), (gathered, xn[s2d[a:b]])):
            ref = torch.mm(rows.double(), wt[t].double())
            assert float((got[a:b] - ref).abs().max()) <= TOL_F32 * float(ref.abs().max()), f"typed product {t}"
