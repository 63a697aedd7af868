"""torch.ops.my_ops.* / torch.classes.my_classes.DGLGraph on the GPU: the same
checks a user of the reference's library would run, against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from graphiler_amd import datasets, prepare_graph, torch_boundary
from graphiler_amd.graph import build_graph_arrays
from helpers import TOL_F32, assert_close, skewed_graph

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def setup(device):
    torch_boundary.load()
    rng = np.random.default_rng(21)
    src, dst = skewed_graph(rng, 700, 5000, 3000)
    n = 700
    g = prepare_graph(src, dst, n, device=device)
    return torch_boundary.script_graph(g), build_graph_arrays(src, dst, n), rng


def _t(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def test_every_reference_operator(setup, device):
    sg, arr, rng = setup
    n, e = arr.num_nodes, arr.COO_src.shape[0]
    x = rng.standard_normal((n, 32), dtype=np.float32)
    m = rng.standard_normal((e, 32), dtype=np.float32)
    w = rng.standard_normal((e, 1), dtype=np.float32)
    ops = torch.ops.my_ops
    P, NB, EI = arr.in_pointer, arr.in_node_indices, arr.in_edge_indices
    assert_close(ops.SpMMSrc(_t(x, device), [1], False, None, sg).cpu().numpy(),
                 oracle.spmm(P, NB, EI, x, op="copy_u"), TOL_F32, "SpMMSrc")
    assert_close(ops.SpMMEdge(_t(m, device), [1], False, None, sg).cpu().numpy(),
                 oracle.spmm(P, NB, EI, m, op="copy_e"), TOL_F32, "SpMMEdge")
    assert_close(ops.gspmm_src_mul_e_sum(_t(x, device), _t(w, device), [1], False, None, sg).cpu().numpy(),
                 oracle.spmm(P, NB, EI, x, w, op="u_mul_e"), TOL_F32, "src_mul_e")
    assert_close(ops.gspmm_dst_mul_e_sum(_t(x, device), _t(w, device), [1], False, None, sg).cpu().numpy(),
                 oracle.spmm(arr.out_pointer, arr.out_node_indices, arr.out_edge_indices,
                             x, w, op="u_mul_e"), TOL_F32, "dst_mul_e")
    u, v = x[:, :1].copy(), x[:, 1:2].copy()
    got = ops.gsddmm_u_add_v_mul_alpha(_t(u, device), _t(v, device), 1, sg)
    assert np.array_equal(got.cpu().numpy(), oracle.sddmm_u_add_v(arr.COO_src, arr.COO_dst, u, v))
    got = ops.SegmentSoftmax(_t(w, device), 1, None, sg)
    assert_close(got.cpu().numpy(), oracle.segment_softmax(P, EI, w), TOL_F32, "softmax")
    assert np.array_equal(ops.BroadcastSrcNode(_t(x, device), sg).cpu().numpy(), x[arr.COO_src])
    assert np.array_equal(ops.BroadcastDstNode(_t(x, device), sg).cpu().numpy(), x[arr.COO_dst])
    assert ops.get_feat_dim(_t(x, device)) == 32
    # additions of this build
    got = ops.gspmm(_t(x, device), None, "copy_u", "max", sg).cpu().numpy()
    assert np.array_equal(got, oracle.spmm(P, NB, EI, x, op="copy_u", reduce="max"))
    got = ops.gsddmm_u_dot_v(_t(x, device), _t(x, device), sg).cpu().numpy()
    assert_close(got, oracle.sddmm_u_dot_v(arr.COO_src, arr.COO_dst, x, x), TOL_F32, "u_dot_v")


def test_scripted_gat_plan_runs_unchanged(setup, device):
    """A TorchScript graph of my_ops nodes (what mpdfg_builder emits for
    examples/GAT/GAT.py at opt level 2) executes on the HIP kernels."""
    sg, arr, rng = setup

    @torch.jit.script
    def gat_plan(g: torch.classes.my_classes.DGLGraph, z: torch.Tensor,
                 el: torch.Tensor, er: torch.Tensor):
        e = torch.ops.my_ops.gsddmm_u_add_v_mul_alpha(el, er, 1, g)
        e = torch.nn.functional.leaky_relu(e, 0.2)
        a = torch.ops.my_ops.SegmentSoftmax(e, 1, None, g)
        return torch.ops.my_ops.gspmm_src_mul_e_sum(z, a, [1], False, None, g)

    n = arr.num_nodes
    z = rng.standard_normal((n, 64), dtype=np.float32)
    el = rng.standard_normal((n, 1), dtype=np.float32)
    er = rng.standard_normal((n, 1), dtype=np.float32)
    got = gat_plan(sg, _t(z, device), _t(el, device), _t(er, device)).cpu().numpy()
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, z, heads=1, slope=0.2)
    assert_close(got, ref, TOL_F32, "scripted GAT plan")
    fused = torch.ops.my_ops.gat_aggregate(_t(el, device), _t(er, device), _t(z, device), 0.2, sg)
    assert_close(fused.cpu().numpy(), ref, TOL_F32, "fused GAT op")


def test_linear_attn_op(setup, device):
    """The projection kernel through the TorchScript boundary: z = x @ w in fp32
    (fp64 numpy product as the reference) and both attention terms."""
    sg, arr, rng = setup
    n = arr.num_nodes
    x = rng.standard_normal((n, 50), dtype=np.float32)
    w = rng.standard_normal((50, 64), dtype=np.float32) / 7
    al = rng.standard_normal((2, 32), dtype=np.float32)
    ar = rng.standard_normal((2, 32), dtype=np.float32)
    z, el, er = torch.ops.my_ops.linear_attn(_t(x, device), _t(w, device), _t(al, device),
                                             _t(ar, device))
    zr = x.astype(np.float64) @ w.astype(np.float64)
    assert_close(z.cpu().numpy(), zr, TOL_F32, "linear_attn z")
    assert_close(el.cpu().numpy(), np.einsum("nhd,hd->nh", zr.reshape(n, 2, 32), al), TOL_F32, "el")
    assert_close(er.cpu().numpy(), np.einsum("nhd,hd->nh", zr.reshape(n, 2, 32), ar), TOL_F32, "er")


def test_gat_aggregate_al_small_and_large_tables(setup, device):
    """gat_aggregate_al = gat_aggregate for a small table of source terms; with
    1.1 M nodes x 4 heads (17.6 MB) it takes the pass that recomputes the term from
    the gathered rows, and must still equal gat_aggregate fed with el = z . a_l."""
    sg, arr, rng = setup
    heads, d = 4, 16
    for n_nodes, n_edges, graph in ((arr.num_nodes, None, sg), (1_100_000, 3_000_000, None)):
        if graph is None:
            src = rng.integers(0, n_nodes, n_edges, dtype=np.int64)
            dst = rng.integers(0, n_nodes // 2, n_edges, dtype=np.int64)     # upper half: no in-edges
            graph = torch_boundary.script_graph(prepare_graph(src, dst, n_nodes, device=device))
        z = torch.randn(n_nodes, heads, d, device=device)
        a_l = torch.randn(1, heads, d, device=device) / 4
        er = torch.randn(n_nodes, heads, 1, device=device)
        el = (z * a_l).sum(2, keepdim=True)
        want = torch.ops.my_ops.gat_aggregate(el, er, z, 0.2, graph)
        got = torch.ops.my_ops.gat_aggregate_al(a_l, el, er, z, 0.2, graph)
        assert got.shape == want.shape == (n_nodes, heads, d)
        err = float((got - want).abs().max() / want.abs().max())
        assert err <= TOL_F32, f"gat_aggregate_al differs by {err:.2e} at {n_nodes} nodes"


def test_gat_aggregate_takes_bf16_attention_terms(setup, device):
    """A bf16 plan whose projection was not rewritten hands el / er over in bf16: the
    operator takes them (read as fp32) and gives what it gives for the same values in
    fp32."""
    sg, arr, rng = setup
    heads, d = 2, 32
    z = torch.randn(arr.num_nodes, heads, d, device=device).bfloat16()
    el = torch.randn(arr.num_nodes, heads, 1, device=device).bfloat16()
    er = torch.randn(arr.num_nodes, heads, 1, device=device).bfloat16()
    got = torch.ops.my_ops.gat_aggregate(el, er, z, 0.2, sg)
    want = torch.ops.my_ops.gat_aggregate(el.float(), er.float(), z, 0.2, sg)
    assert got.dtype == torch.bfloat16 and torch.equal(got.view(torch.int16), want.view(torch.int16))
    with pytest.raises(RuntimeError):
        torch.ops.my_ops.gat_aggregate(el.int(), er, z, 0.2, sg)


@pytest.mark.parametrize("bf16", [False, True])
def test_relation_pair_attention_op(device, bf16):
    """my_ops::relation_pair_attention = edge_softmax_sum(SegmentMMEdgeDot(...) / c,
    SegmentMMEdgeGather(...)): on a graph with many edges per (destination, relation)
    pair it takes the per-pair form, on one with a pair per edge the per-edge operators;
    (T, H, D, D) and (T, D, D) relation matrices."""
    torch_boundary.load()
    from graphiler_amd import ops as pyops
    from graphiler_amd.graph import sort_edges_by_type
    ops = torch.ops.my_ops
    rng = np.random.default_rng(77)
    dt = torch.bfloat16 if bf16 else torch.float32
    tol = 2e-2 if bf16 else 2 * TOL_F32
    for n, e, te, dst_range in ((600, 9000, 3, 150), (3000, 2500, 5, 3000)):
        src = rng.integers(0, n, e)
        dst = rng.integers(0, dst_range, e)
        et = rng.integers(0, te, e)
        src, dst, et, _ = sort_edges_by_type(src, dst, et)
        g = prepare_graph(src, dst, n, device=device, etype_of=et, num_etypes=te)
        pairs = len(np.unique(dst.astype(np.int64) * te + et))
        assert (e >= 2 * pairs) == (dst_range == 150)
        sg = torch_boundary.script_graph(g)
        for heads, d in ((4, 16), (1, 32)):
            hid = heads * d
            k, q, v = (torch.randn(n, hid, device=device).to(dt) for _ in range(3))
            shape = (te, heads, d, d) if heads > 1 else (te, d, d)
            att, msg = ((torch.randn(*shape, device=device) / d ** 0.5).to(dt) for _ in range(2))
            pri = (torch.rand(te, heads, device=device) + 0.5).to(dt)
            for scale, divisor in ((pri, 4.0), (None, 1.0)):
                got = ops.relation_pair_attention(k, q, v, att, msg, scale, divisor, sg)
                score = ops.SegmentMMEdgeDot(k, att, 0, q, 1, scale, sg) / divisor
                want = ops.edge_softmax_sum(score, ops.SegmentMMEdgeGather(v, msg, 0, None, sg), sg)
                assert got.shape == want.shape and got.dtype == want.dtype
                assert_close(got.float().cpu().numpy(), want.float().cpu().numpy(), tol,
                             f"relation_pair_attention {heads}x{d} e={e} scale={scale is not None}")
                if scale is None and divisor == 1.0:
                    k3 = k.view(n, heads, d)
                    att_only = ops.dot_attention_sum(k3, q.view(n, heads, d), v.view(n, heads, d), sg)
                    same_op = pyops.dot_attention_sum(k3, q.view(n, heads, d), v.view(n, heads, d), g)
                    assert att_only.shape == (n, heads, d) and torch.equal(
                        att_only.view(torch.int16 if bf16 else torch.int32),
                        same_op.view(torch.int16 if bf16 else torch.int32))
                if scale is None and heads > 1 and e >= 2 * pairs:
                    # the per-pair form was taken: the bits of the Python composition of the
                    # same entry points, not those of the per-edge operators
                    same = pyops.relation_pair_attention(k, q, v, att, msg, None, g)
                    assert torch.equal(got.view(torch.int16 if bf16 else torch.int32),
                                       same.view(torch.int16 if bf16 else torch.int32))
                    assert not torch.equal(got, want)


def test_general_broadcast_forms_through_torchscript(device):
    """my_ops::gspmm_bcast / my_ops::gsddmm build the offset tables of bcast.cc:19-71 in
    C++ and run the kernels the Python wrappers run (those are checked against numpy
    broadcasting in test_gpu_bcast.py): same shapes out, same bits."""
    from graphiler_amd import ops as pyops
    torch_boundary.load()
    rng = np.random.default_rng(33)
    n = 300
    src, dst = skewed_graph(rng, n, 1200, 2500)
    g = prepare_graph(src, dst, n, device=device)
    sg = torch_boundary.script_graph(g)
    e = src.shape[0]
    for u_feat, e_feat in (((4, 1), (1, 8)), ((3,), (1,)), ((2, 3), (3,)), ((5,), (5,)),
                           ((1, 6), (4, 1)), ((2, 1, 3), (4, 1))):
        u = _t(rng.standard_normal((n,) + u_feat).astype(np.float32), device)
        w = _t(rng.uniform(0.5, 2.0, (e,) + e_feat).astype(np.float32), device)
        for op in ("add", "sub", "mul", "div"):
            for reduce, reverse in (("sum", False), ("max", False), ("min", True)):
                got = torch.ops.my_ops.gspmm_bcast(u, w, op, reduce, reverse, sg)
                want = pyops.gspmm(g, op, reduce, u, w, reverse=reverse)
                assert got.shape == want.shape and torch.equal(got, want), (op, reduce, u_feat)
        assert torch.equal(torch.ops.my_ops.gspmm_bcast(u, None, "copy_lhs", "sum", False, sg),
                           pyops.gspmm(g, "copy_lhs", "sum", u, None))
        assert torch.equal(torch.ops.my_ops.gspmm_bcast(None, w, "copy_rhs", "max", False, sg),
                           pyops.gspmm(g, "copy_rhs", "max", None, w))
    rows = {"u": n, "e": e, "v": n}
    for lt, rt in (("u", "v"), ("u", "e"), ("e", "v"), ("v", "u"), ("e", "e")):
        for l_feat, r_feat in (((4,), (4,)), ((3, 1), (1, 5)), ((2, 3), (3,)), ((1,), (6,))):
            lhs = _t(rng.standard_normal((rows[lt],) + l_feat).astype(np.float32), device)
            rhs = _t(rng.uniform(0.5, 2.0, (rows[rt],) + r_feat).astype(np.float32), device)
            for op in ("add", "sub", "mul", "div", "copy_lhs", "copy_rhs"):
                got = torch.ops.my_ops.gsddmm(lhs, rhs, op, lt, rt, sg)
                want = pyops.gsddmm(g, op, lhs, rhs, lt, rt)
                assert got.shape == want.shape and torch.equal(got, want), (op, lt, rt, l_feat)
        for l_feat, r_feat in (((4, 8), (4, 8)), ((4, 8), (1, 8)), ((16,), (16,)), ((2, 1, 5), (3, 5))):
            lhs = _t(rng.standard_normal((rows[lt],) + l_feat).astype(np.float32), device)
            rhs = _t(rng.standard_normal((rows[rt],) + r_feat).astype(np.float32), device)
            got = torch.ops.my_ops.gsddmm(lhs, rhs, "dot", lt, rt, sg)
            want = pyops.gsddmm(g, "dot", lhs, rhs, lt, rt)
            assert got.shape == want.shape and torch.equal(got, want), ("dot", lt, rt, l_feat)
    x = torch.zeros(n, 3, device=device)
    with pytest.raises(RuntimeError, match="number of rows"):
        torch.ops.my_ops.gsddmm(x, x, "add", "e", "v", sg)
    with pytest.raises(RuntimeError, match="do not broadcast"):
        torch.ops.my_ops.gsddmm(x, torch.zeros(n, 4, device=device), "add", "u", "v", sg)
    with pytest.raises(RuntimeError, match="Unsupported SpMM binary operator"):
        torch.ops.my_ops.gspmm_bcast(x, x, "dot", "sum", False, sg)


def test_error_convention(setup, device):
    sg, arr, rng = setup
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        torch.ops.my_ops.SpMMSrc(torch.ones(arr.num_nodes, 4), [1], False, None, sg)
    xt = torch.ones(4, arr.num_nodes, device=device).t()
    with pytest.raises(RuntimeError, match="must be contiguous"):
        torch.ops.my_ops.SpMMSrc(xt, [1], False, None, sg)
    with pytest.raises(RuntimeError, match="node-type"):
        torch.ops.my_ops.BroadcastNodeType(torch.ones(2, 2, device=device), sg)


def test_typed_sum_and_stacked_products_through_torchscript(device):
    """my_ops::TypedSpMMEdge (= SpMMEdge(SegmentMMEdgeGather(x, w, 0, s))) and
    my_ops::SegmentMMNodeStacked (= one SegmentMMNode per weight) against the python
    operators, at a shape that takes the one-pass kernels and at ones that do not."""
    from graphiler_amd import ops as pyops
    from graphiler_amd.graph import sort_edges_by_type
    torch_boundary.load()
    rng = np.random.default_rng(33)
    n, e, r, tn = 600, 7000, 5, 3
    src, dst = rng.integers(0, n, e), rng.integers(0, n, e)
    et = rng.integers(0, r, e)
    src, dst, et, _ = sort_edges_by_type(src, dst, et)
    nt = np.sort(rng.integers(0, tn, n))
    g = prepare_graph(src, dst, n, device=device, ntype_of=nt, num_ntypes=tn, etype_of=et,
                      num_etypes=r)
    sg = torch_boundary.script_graph(g)
    ops = torch.ops.my_ops
    norm = _t(rng.uniform(0.1, 1.0, (e, 1)).astype(np.float32), device)
    for k, m in ((16, 64), (32, 64), (64, 8), (64, 64), (16, 24)):      # one pass, one pass, one pass, pair, pair
        x = _t(rng.standard_normal((n, k), dtype=np.float32), device)
        w = _t((rng.standard_normal((r, k, m)) / np.sqrt(k)).astype(np.float32), device)
        want = pyops.SpMMEdge(pyops.SegmentMMEdgeGather(x, w, 0, g, row_scale=norm), [1], False, None, g)
        got = ops.TypedSpMMEdge(x, w, norm, sg)
        assert_close(got.cpu().numpy(), want.cpu().numpy(), 2 * TOL_F32, f"TypedSpMMEdge {k}->{m}")
        got = ops.TypedSpMMEdge(x, w, None, sg)
        want = pyops.SpMMEdge(pyops.SegmentMMEdgeGather(x, w, 0, g), [1], False, None, g)
        assert_close(got.cpu().numpy(), want.cpu().numpy(), 2 * TOL_F32, f"TypedSpMMEdge {k}->{m} plain")
    h = _t(rng.standard_normal((n, 128), dtype=np.float32), device).bfloat16()
    ws = [_t(datasets.glorot(rng, (tn, 128, 128)), device).bfloat16() for _ in range(3)]
    outs = ops.SegmentMMNodeStacked(h, ws, sg)
    assert len(outs) == 3
    for w, y in zip(ws, outs):
        assert torch.equal(y.view(torch.int16), ops.SegmentMMNode(h, w, sg).view(torch.int16))
    # the product with a per-node factor: in the kernel when the factor is (N, 1) and does
    # not promote the result, as two steps otherwise -- the same values either way
    for w, dt in ((ws[0], torch.bfloat16), (ws[0].float(), torch.float32)):
        hh = h.to(dt)
        plain = ops.SegmentMMNode(hh, w, sg)
        for fac in (torch.rand(n, 1, device=device).to(dt), torch.rand(n, 1, device=device),
                    torch.rand(n, device=device).to(dt)[:, None].expand(n, 128)):
            got = ops.SegmentMMNodeScaled(hh, w, fac, sg)
            want = plain * fac
            assert got.dtype == want.dtype and got.shape == want.shape
            assert_close(got.float().cpu().numpy(), want.float().cpu().numpy(),
                         2e-2 if dt == torch.bfloat16 else 2 * TOL_F32, f"SegmentMMNodeScaled {dt}")
    # ... and with a gate per node type (HGT's sigmoid(skip)): in the kernel for the wide
    # bf16 shape, through the per-row factor otherwise -- the ctypes wrapper does the same
    for w, dt in ((ws[0], torch.bfloat16), (ws[0].float(), torch.float32)):
        hh = h.to(dt)
        gate = torch.randn(tn, device=device).to(dt)       # a gate of the model's dtype
        for sig in (True, False):
            got = ops.SegmentMMNodeGated(hh, w, gate, sig, sg)
            fac = (torch.sigmoid(gate.float()) if sig else gate.float())[g.ntype_COO][:, None]
            want = ops.SegmentMMNode(hh, w, sg).float() * fac
            assert got.dtype == dt and got.shape == want.shape
            assert_close(got.float().cpu().numpy(), want.cpu().numpy(),
                         2e-2 if dt == torch.bfloat16 else 2 * TOL_F32, f"SegmentMMNodeGated {dt} {sig}")
            mirror = pyops.SegmentMMNodeGated(hh, w, gate.float(), g, sigmoid=sig)
            assert torch.equal(got.view(torch.int16 if dt == torch.bfloat16 else torch.int32),
                               mirror.view(torch.int16 if dt == torch.bfloat16 else torch.int32))
    # a factor that promotes the product keeps the meaning of `product * factor`: fp32 out
    wide = ops.SegmentMMNodeGated(h, ws[0], torch.randn(tn, device=device), True, sg)
    assert wide.dtype == torch.float32
    e_all = g.num_edges
    for m_cols in (64, 256):        # a width the gathered product's kernel takes, and one it does not
        w_e = _t(datasets.glorot(rng, (r, 128, m_cols)), device).bfloat16()
        plain = ops.SegmentMMEdgeGather(h, w_e, 0, None, sg)
        s32 = torch.rand(e_all, 1, device=device) + 0.5
        same = ops.SegmentMMEdgeGather(h, w_e, 0, s32.bfloat16(), sg)
        promoted = ops.SegmentMMEdgeGather(h, w_e, 0, s32, sg)
        assert plain.dtype == same.dtype == torch.bfloat16 and promoted.dtype == torch.float32
        assert_close(promoted.cpu().numpy(), (plain.float() * s32).cpu().numpy(), 2 * TOL_F32,
                     f"gathered product times an fp32 factor, {m_cols} columns")
        assert_close(same.float().cpu().numpy(), (plain.float() * s32.bfloat16().float()).cpu().numpy(), 2e-2,
                     f"gathered product times a bf16 factor, {m_cols} columns")
        flat = ops.SegmentMMEdgeGather(h, w_e, 0, s32.bfloat16().reshape(-1), sg)     # (E,): per row too
        assert torch.equal(flat.view(torch.int16), same.view(torch.int16))
    mixed = [ws[0], ws[1][:, :, :64].contiguous()]          # different shapes: one product each
    outs = ops.SegmentMMNodeStacked(h, mixed, sg)
    assert outs[1].shape == (n, 64)
    assert torch.equal(outs[1].view(torch.int16), ops.SegmentMMNode(h, mixed[1], sg).view(torch.int16))


def test_sum_with_row_wise_tail(setup, device):
    """my_ops::SpMMScaled = act(SpMMSrc | SpMMEdge (x) * s): in the sum's store for an
    fp32 (N, 1) factor on fp32 features, by torch's own multiplication (broadcasting and
    promotion included) for any other factor -- the same values and dtype as the three
    separate operators either way."""
    sg, arr, rng = setup
    ops = torch.ops.my_ops
    n, e = arr.num_nodes, arr.COO_src.shape[0]
    for edge_rows, rows in ((False, n), (True, e)):
        plain_op = ops.SpMMEdge if edge_rows else ops.SpMMSrc
        for dt in (torch.float32, torch.bfloat16):
            x = _t(rng.standard_normal((rows, 24), dtype=np.float32) + np.float32(0.2), device).to(dt)
            plain = plain_op(x, [1], False, None, sg)
            factors = (None, torch.rand(n, 1, device=device) - 0.4,                   # per row
                       (torch.rand(n, 1, device=device) - 0.4).to(dt),
                       torch.rand(24, device=device), torch.rand(n, 24, device=device).double())
            for fac in factors:
                for act, fn in ((0, lambda t: t), (1, torch.relu), (2, torch.nn.functional.elu)):
                    got = ops.SpMMScaled(x, fac, act, edge_rows, sg)
                    want = fn(plain if fac is None else plain * fac)
                    assert got.dtype == want.dtype and got.shape == want.shape, (dt, fac, act)
                    tol = 2e-2 if want.dtype == torch.bfloat16 else 2 * TOL_F32
                    assert_close(got.double().cpu().numpy(), want.double().cpu().numpy(), tol,
                                 f"SpMMScaled {dt} act {act} edge_rows {edge_rows}")
            # three-dimensional features: a factor per row is (N, 1, 1)
            x3 = x.view(rows, 4, 6)
            fac3 = torch.rand(n, 1, 1, device=device)
            got = ops.SpMMScaled(x3, fac3, 1, edge_rows, sg)
            want = torch.relu(plain_op(x3, [1], False, None, sg) * fac3)
            assert got.shape == (n, 4, 6) and got.dtype == want.dtype
            assert_close(got.float().cpu().numpy(), want.float().cpu().numpy(), 2 * TOL_F32, "3-d features")
    with pytest.raises(RuntimeError, match="activation"):
        ops.SpMMScaled(x, None, 3, True, sg)
    with pytest.raises(RuntimeError, match="rows"):
        ops.SpMMScaled(x, None, 0, False, sg)
