"""End-to-end layer forwards (the reference's optimised plans) against the
oracle composed per the same plan, on reduced copies of the five workloads."""
import numpy as np
import pytest
import torch

import oracle
from graphiler_amd import capi, datasets, layers, prepare_graph
from graphiler_amd.graph import build_graph_arrays, sort_edges_by_type
from helpers import TOL_BF16, TOL_F32, assert_close, to_bf16_f32

pytestmark = pytest.mark.gpu


def _t(a, device, bf16=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(device)
    return t.to(torch.bfloat16) if bf16 else t


def test_gcn_two_layers(device):
    """Config 1: symmetric-normalised 2-layer GCN, 500 -> 16 -> 3."""
    wl = datasets.gcn_uniform()
    n = wl.num_nodes
    g = prepare_graph(wl.src, wl.dst, n, device=device)
    arr = build_graph_arrays(wl.src, wl.dst, n)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((n, 500), dtype=np.float32)
    w1, w2 = datasets.glorot(rng, (500, 16)), datasets.glorot(rng, (16, 3))
    deg = np.bincount(wl.dst, minlength=n).astype(np.float32)
    norm = (deg ** -0.5)[:, None].astype(np.float32)
    dn = _t(norm, device)
    h1 = layers.gcn_layer(g, _t(x, device), _t(w1, device), dn, dn, relu=True)
    h2 = layers.gcn_layer(g, h1, _t(w2, device), dn, dn, relu=False)

    def ref_layer(h, w, relu):
        m = ((h.astype(np.float64) @ w.astype(np.float64)) * norm).astype(np.float32)
        out = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices, m) * norm
        return np.maximum(out, 0) if relu else out

    r1 = ref_layer(x, w1, True)
    assert_close(h1.cpu().numpy(), r1, TOL_F32, "GCN layer 1")
    assert_close(h2.cpu().numpy(), ref_layer(r1.astype(np.float32), w2, False),
                 TOL_F32, "GCN layer 2")


@pytest.mark.parametrize("heads", [1, 4])
def test_gat_layer_switches_to_source_term_from_rows(device, heads, monkeypatch):
    """gat_layer takes the variant that recomputes the source term once the
    (N, heads) table passes a size limit; both routes give the layer's result."""
    wl = datasets.gat_rmat(num_nodes=3000, n_edges=60_000, scale=12, seed=3)
    n = wl.num_nodes
    g = prepare_graph(wl.src, wl.dst, n, device=device)
    rng = np.random.default_rng(3)
    h = torch.from_numpy(rng.standard_normal((n, 40), dtype=np.float32)).to(device)
    w = torch.from_numpy(datasets.glorot(rng, (40, heads * 32))).to(device)
    a = torch.from_numpy(rng.standard_normal((2, heads, 32), dtype=np.float32) / 6).to(device)
    base = layers.gat_layer(g, h, w, a, heads, 0.2)
    calls = []
    real = layers.ops.gat_aggregate_from_z
    monkeypatch.setattr(layers.ops, "gat_aggregate_from_z",
                        lambda *args: calls.append(1) or real(*args))
    monkeypatch.setattr(layers, "SOURCE_TERM_TABLE_LIMIT", 0)
    alt = layers.gat_layer(g, h, w, a, heads, 0.2)
    assert calls, "the size limit did not select the variant"
    assert_close(alt.cpu().numpy(), base.cpu().numpy(), TOL_F32, "gat_layer, both routes")


@pytest.mark.parametrize("heads,bf16", [(1, False), (4, False), (4, True)])
def test_gat_layer(device, heads, bf16):
    wl = datasets.gat_rmat(num_nodes=20_000, n_edges=600_000, scale=15, seed=1,
                           self_loops=True)
    n = wl.num_nodes
    g = prepare_graph(wl.src, wl.dst, n, device=device)
    arr = build_graph_arrays(wl.src, wl.dst, n)
    rng = np.random.default_rng(1)
    d = 64
    z = rng.standard_normal((n, heads * d), dtype=np.float32)
    el = rng.standard_normal((n, heads), dtype=np.float32)
    er = rng.standard_normal((n, heads), dtype=np.float32)
    if bf16:
        z = to_bf16_f32(z)
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, z,
                               heads=heads, slope=0.2)
    tol = TOL_BF16 if bf16 else TOL_F32
    dz, dl, dr = _t(z, device, bf16), _t(el, device), _t(er, device)
    fused = layers.ops.gat_aggregate(dl, dr, dz, g, 0.2)
    assert_close(fused.float().cpu().numpy(), ref, tol, "fused GAT")
    plan = layers.gat_aggregate_plan(g, dz, dl, dr, 0.2)
    assert_close(plan.float().cpu().numpy(), ref, tol, "GAT plan")


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("bf16", [False, True])
def test_rgcn_two_layers(device, bf16, fused):
    wl = datasets.rgcn_zipf(num_nodes=10_000, n_edges=100_000)
    n = wl.num_nodes
    g = prepare_graph(wl.src, wl.dst, n, device=device, etype_of=wl.etype,
                      num_etypes=60)
    arr = build_graph_arrays(wl.src, wl.dst, n)
    rng = np.random.default_rng(2)
    x = rng.standard_normal((n, 16), dtype=np.float32)
    w1, w2 = datasets.glorot(rng, (60, 16, 64)), datasets.glorot(rng, (60, 64, 8))
    if bf16:
        x, w1, w2 = to_bf16_f32(x), to_bf16_f32(w1), to_bf16_f32(w2)
    deg = np.maximum(np.bincount(wl.dst, minlength=n), 1)
    norm = (1.0 / deg[wl.dst]).astype(np.float32)[:, None]
    etp = oracle.type_pointer(wl.etype, 60)

    def ref_layer(h, w):
        msg = oracle.segment_mm(etp, oracle.gather_rows(wl.src, h), w) * norm
        return oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                           msg.astype(np.float32), op="copy_e")

    dn = _t(norm, device)
    h1 = torch.relu(layers.rgcn_layer(g, _t(x, device, bf16), _t(w1, device, bf16), dn,
                                      fused=fused))
    h2 = layers.rgcn_layer(g, h1, _t(w2, device, bf16), dn, fused=fused)
    r1 = np.maximum(ref_layer(x, w1), 0).astype(np.float32)
    tol = TOL_BF16 if bf16 else TOL_F32
    assert_close(h1.float().cpu().numpy(), r1, tol, "RGCN layer 1")
    assert_close(h2.float().cpu().numpy(), ref_layer(r1, w2), 2 * tol, "RGCN layer 2")


@pytest.mark.parametrize("fused", [True, "pairs", "edges", False])
@pytest.mark.parametrize("bf16", [False, True])
def test_hgt_layer(device, bf16, fused):
    wl = datasets.hgt_hetero(counts=(800, 600, 400, 200), edges_per_type=4000)
    n, e = wl.num_nodes, wl.num_edges
    heads, d = 8, 16
    hid = heads * d
    g = prepare_graph(wl.src, wl.dst, n, device=device, ntype_of=wl.ntype,
                      num_ntypes=4, etype_of=wl.etype, num_etypes=10)
    arr = build_graph_arrays(wl.src, wl.dst, n)
    rng = np.random.default_rng(3)
    cast = to_bf16_f32 if bf16 else (lambda a: a)
    h = cast(rng.standard_normal((n, hid), dtype=np.float32))
    wk, wq, wv, wa = (cast(datasets.glorot(rng, (4, hid, hid))) for _ in range(4))
    ratt, rmsg = (cast(datasets.glorot(rng, (10, heads, d, d))) for _ in range(2))
    rpri = cast(datasets.glorot(rng, (10, heads)))
    skip = np.ones(4, np.float32)
    got = layers.hgt_layer(g, _t(h, device, bf16), _t(wk, device, bf16),
                           _t(wq, device, bf16), _t(wv, device, bf16),
                           _t(wa, device, bf16), _t(ratt, device, bf16),
                           _t(rmsg, device, bf16), _t(rpri, device, bf16),
                           _t(skip, device), heads, fused=fused)
    # the same plan on the oracle (fp64 accumulation; bf16 rounding applied where
    # the device stores bf16 tensors)
    ntp, etp = oracle.type_pointer(wl.ntype, 4), oracle.type_pointer(wl.etype, 10)
    K = cast(oracle.segment_mm(ntp, h, wk))
    V = cast(oracle.segment_mm(ntp, h, wv))
    Q = cast(oracle.segment_mm(ntp, h, wq))
    k_e = cast(oracle.segment_mm(etp, oracle.gather_rows(wl.src, K), ratt, heads=heads))
    v_e = cast(oracle.segment_mm(etp, oracle.gather_rows(wl.src, V), rmsg, heads=heads))
    q_e = oracle.gather_rows(wl.dst, Q)
    attn = (k_e.reshape(e, heads, d) * q_e.reshape(e, heads, d)).sum(-1)
    attn = (attn * rpri[wl.etype] / np.sqrt(d)).astype(np.float32)
    a = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, attn)
    m = cast((v_e.reshape(e, heads, d) * a[:, :, None]).reshape(e, hid).astype(np.float32))
    t = cast(oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices, m,
                         op="copy_e"))
    out = oracle.segment_mm(ntp, t, wa) * (1.0 / (1.0 + np.exp(-skip[wl.ntype])))[:, None]
    assert_close(got.float().cpu().numpy(), out, TOL_BF16 if bf16 else TOL_F32,
                 f"HGT layer bf16={bf16}")


@pytest.mark.parametrize("heads,d", [(8, 16), (2, 32), (1, 16), (4, 8), (8, 12), (2, 24)])
def test_hgt_pair_form_equals_edge_form(device, heads, d):
    """The relation matrices applied per (destination, relation) pair against per edge:
    few edges per pair, destinations without in-edges, a relation without edges, a
    destination with a large share of the edges; fp32, so the two forms differ by
    rounding order only.  Head widths the typed product does not take fall back."""
    rng = np.random.default_rng(heads * 100 + d)
    n, e, tn, te = 900, 7000, 3, 6
    hid = heads * d
    src = rng.integers(0, n, e)
    dst = rng.integers(0, n // 2, e)                 # upper half: no in-edges
    dst[: e // 4] = 7                                 # one destination with a quarter of the edges
    et = rng.choice([0, 1, 2, 4, 5], size=e)          # relation 3 has no edges
    src, dst, et, _ = sort_edges_by_type(src, dst, et)
    nt = np.sort(rng.integers(0, tn, n))
    g = prepare_graph(src, dst, n, device=device, ntype_of=nt, num_ntypes=tn, etype_of=et,
                      num_etypes=te)
    pairs = g.relation_pairs()
    key = np.unique(dst.astype(np.int64) * te + et)
    assert pairs is not None and pairs.num_pairs == len(key)
    assert np.array_equal(pairs.pair_dst.cpu().numpy(), key // te)
    counts = np.diff(pairs.pair_pointer.cpu().numpy())
    assert counts.sum() == e and counts.min() >= 1
    h = _t(rng.standard_normal((n, hid), dtype=np.float32), device)
    wk, wq, wv, wa = (_t(datasets.glorot(rng, (tn, hid, hid)), device) for _ in range(4))
    ratt, rmsg = (_t(datasets.glorot(rng, (te, heads, d, d)), device) for _ in range(2))
    rpri = _t(rng.uniform(0.5, 1.5, (te, heads)).astype(np.float32), device)
    skip = _t(rng.standard_normal(tn).astype(np.float32), device)
    args = (g, h, wk, wq, wv, wa, ratt, rmsg, rpri, skip, heads)
    want = layers.hgt_layer(*args, fused=False)
    got = layers.hgt_layer(*args, fused="pairs")
    assert_close(got.cpu().numpy(), want.cpu().numpy(), 2 * TOL_F32, f"HGT pairs {heads}x{d}")
    auto = layers.hgt_layer(*args, fused=True)
    assert_close(auto.cpu().numpy(), want.cpu().numpy(), 2 * TOL_F32, f"HGT auto {heads}x{d}")


def test_type_dependent_layouts_follow_the_edge_type_pointer(device):
    """Replacing a graph's edge type pointer drops the layouts prepared from the old one
    (the (destination, relation) pairs and the typed tiles)."""
    from graphiler_amd import ops
    rng = np.random.default_rng(3)
    n, e = 300, 4000
    src, dst = rng.integers(0, n, e), rng.integers(0, 60, e)
    et = np.sort(rng.integers(0, 4, e))
    g = prepare_graph(src, dst, n, device=device, etype_of=et, num_etypes=4)
    before = g.relation_pairs().num_pairs
    tiles_before = ops._typed_tiles(g)
    assert before == len(np.unique(dst * 4 + et))
    one_type = torch.tensor([0, e], dtype=torch.int32, device=device)
    g.SetEtypePointer(one_type)
    assert g.num_etypes == 1 and g.relation_pairs().num_pairs == len(np.unique(dst))
    assert ops._typed_tiles(g) is not tiles_before
    x = _t(rng.standard_normal((n, 16), dtype=np.float32), device)
    w = _t(rng.standard_normal((1, 16, 8), dtype=np.float32), device)
    got = ops.TypedSpMMEdge(x, w, g)
    want = ops.SpMMEdge(ops.SegmentMMEdgeGather(x, w, 0, g), [1], False, None, g)
    assert_close(got.cpu().numpy(), want.cpu().numpy(), 2 * TOL_F32, "typed sum after a new type pointer")
