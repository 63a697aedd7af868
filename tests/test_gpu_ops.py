"""Parity of the HIP operators (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from graphiler_amd import capi, datasets, ops, prepare_graph
from graphiler_amd.graph import build_graph_arrays
from helpers import (TOL_BF16, TOL_F32, assert_close, random_graph,
                     skewed_graph, to_bf16_f32)

pytestmark = pytest.mark.gpu


def _graphs():
    rng = np.random.default_rng(11)
    dbg = datasets.debug_graph()
    out = {"debug": (dbg.src, dbg.dst, 3)}
    s, d = random_graph(rng, 300, 2000)
    out["uniform"] = (s, d, 300)
    s, d = skewed_graph(rng, 1000, 6000, 9000)
    out["skewed"] = (s, d, 1000)
    wl = datasets.gat_rmat(num_nodes=5000, n_edges=150_000, scale=13, seed=5)
    out["rmat_by_dst"] = (wl.src, wl.dst, wl.num_nodes)
    out["no_edges"] = (np.zeros(0, np.int64), np.zeros(0, np.int64), 17)
    out["one_row"] = (rng.integers(0, 5, 4000, dtype=np.int64),
                      np.zeros(4000, np.int64), 5)
    return out


GRAPHS = _graphs()


@pytest.fixture(scope="module", params=list(GRAPHS))
def graph(request, device):
    src, dst, n = GRAPHS[request.param]
    g = prepare_graph(src, dst, n, device=device)
    return request.param, g, build_graph_arrays(src, dst, n)


def _dev(a, device, bf16=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(device)
    return t.to(torch.bfloat16) if bf16 else t


def test_row_ids_bit_exact(graph):
    name, g, arr = graph
    want = np.repeat(np.arange(arr.num_nodes, dtype=np.int32),
                     np.diff(arr.in_pointer))
    assert np.array_equal(g.in_row_of_slot.cpu().numpy(), want)
    want = np.repeat(np.arange(arr.num_nodes, dtype=np.int32),
                     np.diff(arr.out_pointer))
    assert np.array_equal(g.out_row_of_slot.cpu().numpy(), want)


def test_graph_prep_on_device_bit_exact(graph):
    """prepare_graph groups the edge list on the GPU; every column must equal the
    oracle's stable grouping and the host construction, bit for bit."""
    name, g, arr = graph
    for side, key, other in (("in", arr.COO_dst, arr.COO_src), ("out", arr.COO_src, arr.COO_dst)):
        ptr, nbr, eid = oracle.group_edges(arr.num_nodes, key, other)
        assert np.array_equal(getattr(g, side + "_pointer").cpu().numpy(), ptr), f"{name} {side} pointer"
        assert np.array_equal(getattr(g, side + "_node_indices").cpu().numpy(), nbr), f"{name} {side} nbr"
        assert np.array_equal(getattr(g, side + "_edge_indices").cpu().numpy(), eid), f"{name} {side} eid"
        assert np.array_equal(ptr, getattr(arr, side + "_pointer"))
        assert np.array_equal(eid, getattr(arr, side + "_edge_indices"))
    assert g.in_pointer.dtype == torch.int32 and g.COO_src.dtype == torch.int64


def test_graph_prep_rejects_bad_endpoints_and_sorts_types(device):
    from graphiler_amd.graph import group_on_device
    src = np.array([0, 1, 2, 7], np.int64)
    dst = np.array([1, 2, 0, 1], np.int64)
    with pytest.raises(ValueError, match="outside"):
        prepare_graph(src, dst, 3, device)
    with pytest.raises(ValueError, match="outside"):
        prepare_graph(dst, np.array([0, -1, 2, 1], np.int64), 3, device)
    # grouping by type: pointer = running count, order = stable permutation
    rng = np.random.default_rng(9)
    et = rng.integers(0, 7, 5000).astype(np.int64)
    ptr, _, order, status = group_on_device(torch.from_numpy(et).to(device), None, 9)
    assert int(status.item()) == 0
    assert np.array_equal(order.cpu().numpy(), np.argsort(et, kind="stable").astype(np.int32))
    assert np.array_equal(ptr.cpu().numpy(), oracle.type_pointer(np.sort(et), 9))
    with pytest.raises(ValueError, match="sorted by type"):
        prepare_graph(np.array([0, 1], np.int64), np.array([1, 0], np.int64), 2, device,
                      etype_of=np.array([1, 0]), num_etypes=2)
    g = prepare_graph(np.array([0, 1], np.int64), np.array([1, 0], np.int64), 2, device,
                      etype_of=np.array([0, 1]), num_etypes=3)
    assert g.etype_pointer.cpu().tolist() == [0, 1, 2, 2]


@pytest.mark.parametrize("feat", [1, 3, 16, 64, 100, 256, 602])
@pytest.mark.parametrize("op", ["copy_u", "copy_e"])
def test_spmm_copy_sum_f32(graph, device, feat, op):
    name, g, arr = graph
    rng = np.random.default_rng(feat)
    rows = arr.num_nodes if op == "copy_u" else arr.COO_src.shape[0]
    x = rng.standard_normal((rows, feat), dtype=np.float32)
    fn = ops.SpMMSrc if op == "copy_u" else ops.SpMMEdge
    got = fn(_dev(x, device), [1], False, None, g).cpu().numpy()
    adj = (arr.in_pointer, arr.in_node_indices, arr.in_edge_indices)
    ref = oracle.spmm(*adj, x, op=op)
    assert_close(got, ref, TOL_F32, f"{op} sum {name} F={feat}",
                 mag=oracle.spmm(*adj, np.abs(x), op=op))
    # rows without in-edges are exactly zero
    empty = np.diff(arr.in_pointer) == 0
    assert not got[empty].any()


@pytest.mark.parametrize("feat", [1, 3, 16, 40, 64, 602])
@pytest.mark.parametrize("op", ["copy_u", "copy_e"])
@pytest.mark.parametrize("bf16", [False, True])
def test_spmm_scaled_is_the_separate_operators(graph, device, feat, op, bf16):
    """Sum, row factor and activation in the store of the sum: against the oracle's sum
    scaled and activated in float64, and bit for bit against SpMMSrc / SpMMEdge followed
    by the multiplication and the activation in fp32 (one rounding at the end)."""
    name, g, arr = graph
    rng = np.random.default_rng(feat * 3 + bf16)
    n = arr.num_nodes
    rows = n if op == "copy_u" else arr.COO_src.shape[0]
    # a mean away from 0: the 4000-edge row's sum must not cancel to nothing
    x = rng.standard_normal((rows, feat), dtype=np.float32) + np.float32(0.3)
    if bf16:
        x = to_bf16_f32(x)
    scale = rng.uniform(-1.5, 1.5, (n, 1)).astype(np.float32)
    xd, sd = _dev(x, device, bf16), _dev(scale, device)
    adj = (arr.in_pointer, arr.in_node_indices, arr.in_edge_indices)
    ref = oracle.spmm(*adj, x, op=op).astype(np.float64)
    mag = oracle.spmm(*adj, np.abs(x), op=op)
    plain = (ops.SpMMSrc if op == "copy_u" else ops.SpMMEdge)(xd, [1], False, None, g)
    for act in (None, "relu", "elu"):
        for sc in (None, sd, sd.view(-1)):
            got = ops.spmm_scaled(xd, g, row_scale=sc, activation=act, edge_rows=op == "copy_e")
            assert got.dtype == xd.dtype and got.shape == (n, feat)
            want = ref if sc is None else ref * scale
            if act == "relu":
                want = np.maximum(want, 0)
            elif act == "elu":
                want = np.where(want > 0, want, np.expm1(np.minimum(want, 0)))
            assert_close(got.float().cpu().numpy(), want, TOL_BF16 if bf16 else TOL_F32,
                         f"spmm_scaled {op} {name} F={feat} act={act} scale={sc is not None}",
                         mag=mag * (1 if sc is None else np.abs(scale)))
            # the device's elu is a polynomial near 0, not torch's expm1; a bf16 sum that
            # is scaled is rounded once here and twice by the separate operators
            if act != "elu" and not (bf16 and sc is not None):
                sep = plain if sc is None else plain * sd
                sep = torch.relu(sep) if act == "relu" else sep
                assert torch.equal(got, sep), f"{op} {name} F={feat} act={act}"
    # no factor, no activation: the plain operator
    assert torch.equal(ops.spmm_scaled(xd, g, edge_rows=op == "copy_e"),
                       (ops.SpMMSrc if op == "copy_u" else ops.SpMMEdge)(xd, [1], False, None, g))


@pytest.mark.parametrize("feat", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("bf16", [False, True])
def test_narrow_sums_with_a_row_across_many_workgroups(device, feat, bf16):
    """Rows of at most eight features take the lanes-per-slot kernel; a destination
    with 380,000 in-edges spans hundreds of its workgroups (the cooperative fold of the
    second kernel), next to short rows, rows without edges and a shuffled edge order."""
    rng = np.random.default_rng(40 + feat)
    n, e = 3000, 400_000
    src = rng.integers(0, n, e)
    dst = rng.integers(0, n // 2, e)                 # the upper half has no in-edges
    dst[rng.permutation(e)[:380_000]] = 17
    g = prepare_graph(src, dst, n, device=device)
    arr = build_graph_arrays(src, dst, n)
    assert not g.in_eid_is_identity
    x = rng.standard_normal((n, feat), dtype=np.float32) + np.float32(0.25)
    m = rng.standard_normal((e, feat), dtype=np.float32) + np.float32(0.25)
    w = rng.uniform(0.5, 1.5, (e, 1)).astype(np.float32)
    if bf16:
        x, m = to_bf16_f32(x), to_bf16_f32(m)
    xd, md, wd = _dev(x, device, bf16), _dev(m, device, bf16), _dev(w, device)
    adj = (arr.in_pointer, arr.in_node_indices, arr.in_edge_indices)
    tol = TOL_BF16 if bf16 else TOL_F32
    cases = (("copy_u", lambda: ops.SpMMSrc(xd, [1], False, None, g), (x, None)),
             ("copy_e", lambda: ops.SpMMEdge(md, [1], False, None, g), (m, None)),
             ("u_mul_e", lambda: ops.gspmm_src_mul_e_sum(xd, wd, [1], False, None, g), (x, w)),
             ("u_div_e", lambda: ops.spmm(g, "u_div_e", "sum", xd, wd), (x, w)))
    for op, fn, (u, ww) in cases:
        got = fn()
        assert got.dtype == xd.dtype and got.shape == (n, feat)
        ref = oracle.spmm(*adj, u, ww, op=op)
        mag = oracle.spmm(*adj, np.abs(u), ww, op=op)
        assert_close(got.float().cpu().numpy(), ref, tol, f"{op} F={feat} bf16={bf16}", mag=mag)
        assert not got[n // 2:].any()               # rows without in-edges
        assert torch.equal(got, fn())               # the same bits every time
    got = ops.spmm_scaled(xd, g, row_scale=_dev(np.full((n, 1), 0.5, np.float32), device), activation="relu")
    want = np.maximum(oracle.spmm(*adj, x, op="copy_u") * 0.5, 0)
    assert_close(got.float().cpu().numpy(), want, tol, f"scaled F={feat} bf16={bf16}",
                 mag=oracle.spmm(*adj, np.abs(x), op="copy_u") * 0.5)


def test_spmm_scaled_non_finite_factor_and_arguments(device):
    """A row without edges is 0 * factor: an infinite factor (degree 0 to the power -1/2)
    shows as NaN there, as it does after the separate multiplication."""
    src, dst = np.array([0, 1, 1], np.int64), np.array([1, 0, 0], np.int64)
    g = prepare_graph(src, dst, 3, device=device)
    x = torch.ones(3, 4, device=device)
    scale = torch.tensor([2.0, float("inf"), float("inf")], device=device)
    got = ops.spmm_scaled(x, g, row_scale=scale, activation="relu").cpu().numpy()
    assert np.array_equal(got[0], np.full(4, 4.0, np.float32))
    assert np.isposinf(got[1]).all() and np.isnan(got[2]).all()
    with pytest.raises(RuntimeError, match="row_scale"):
        ops.spmm_scaled(x, g, row_scale=scale[:2])
    with pytest.raises(RuntimeError, match="row_scale"):
        ops.spmm_scaled(x, g, row_scale=scale.double())
    with pytest.raises(RuntimeError, match="activation"):
        ops.spmm_scaled(x, g, activation="tanh")
    with pytest.raises(RuntimeError, match="rows"):
        ops.spmm_scaled(x[:2], g)


@pytest.mark.parametrize("feat,heads", [(1, 1), (5, 1), (64, 1), (64, 4),
                                        (128, 8), (256, 4), (12, 3)])
@pytest.mark.parametrize("reverse", [False, True])
def test_spmm_u_mul_e_sum_f32(graph, device, feat, heads, reverse):
    name, g, arr = graph
    rng = np.random.default_rng(feat * 7 + heads)
    e = arr.COO_src.shape[0]
    x = rng.standard_normal((arr.num_nodes, feat), dtype=np.float32)
    w = rng.standard_normal((e, heads), dtype=np.float32)
    fn = ops.gspmm_dst_mul_e_sum if reverse else ops.gspmm_src_mul_e_sum
    got = fn(_dev(x, device), _dev(w, device), [1], False, None, g).cpu().numpy()
    adj = (arr.out_pointer, arr.out_node_indices, arr.out_edge_indices) if reverse else \
        (arr.in_pointer, arr.in_node_indices, arr.in_edge_indices)
    ref = oracle.spmm(*adj, x, w, op="u_mul_e", heads=heads)
    assert_close(got, ref, TOL_F32, f"u_mul_e {name} F={feat} H={heads}",
                 mag=oracle.spmm(*adj, np.abs(x), np.abs(w), op="u_mul_e", heads=heads))


@pytest.mark.parametrize("op", ["u_add_e", "u_sub_e", "u_div_e"])
@pytest.mark.parametrize("reduce", ["sum", "max", "min"])
@pytest.mark.parametrize("feat,heads,bf16", [(64, 4, False), (6, 2, False), (64, 1, True)])
def test_spmm_add_sub_div(graph, device, op, reduce, feat, heads, bf16):
    name, g, arr = graph
    rng = np.random.default_rng(feat + 3 * heads)
    e = arr.COO_src.shape[0]
    x = rng.standard_normal((arr.num_nodes, feat), dtype=np.float32)
    w = (rng.uniform(0.5, 2.0, (e, heads)) * rng.choice([-1, 1], (e, heads))).astype(np.float32)
    if bf16:
        x = to_bf16_f32(x)
    got = ops.spmm(g, op, reduce, _dev(x, device, bf16), _dev(w, device)).float().cpu().numpy()
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices, x, w,
                      op=op, reduce=reduce, heads=heads)
    finite = np.isfinite(ref)
    assert np.array_equal(np.isfinite(got), finite), f"{name}: empty rows differ"
    assert_close(np.where(finite, got, 0), np.where(finite, ref, 0),
                 TOL_BF16 if bf16 else TOL_F32, f"{op} {reduce} {name}")


def test_spmm_u_mul_e_shaped_operands(graph, device):
    """(N, H, D) features with (E, H, 1) weights: the per-head broadcast of the
    reference's shape tables, served by the row-reduction kernel; any other broadcast
    takes the general kernel (bcast.cc:19-71 tables consumed on the device)."""
    name, g, arr = graph
    rng = np.random.default_rng(11)
    e = arr.COO_src.shape[0]
    x = rng.standard_normal((arr.num_nodes, 4, 8), dtype=np.float32)
    w = rng.standard_normal((e, 4, 1), dtype=np.float32)
    got = ops.gspmm_src_mul_e_sum(_dev(x, device), _dev(w, device), [1], False, None, g)
    assert tuple(got.shape) == (arr.num_nodes, 4, 8)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      x.reshape(arr.num_nodes, 32), w.reshape(e, 4), op="u_mul_e", heads=4)
    assert_close(got.cpu().numpy().reshape(arr.num_nodes, 32), ref, TOL_F32, f"shaped {name}")
    per_feat = rng.standard_normal((e, 1, 8), dtype=np.float32)      # per feature, not per head
    got = ops.gspmm_src_mul_e_sum(_dev(x, device), _dev(per_feat, device), [1], False, None, g)
    want = np.zeros((arr.num_nodes, 4, 8))
    np.add.at(want, arr.COO_dst, x[arr.COO_src].astype(np.float64) * per_feat)
    assert_close(got.cpu().numpy(), want, TOL_F32, f"shaped, per-feature weights {name}")


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("op,feat,heads", [("copy_u", 64, 1), ("copy_u", 7, 1),
                                           ("copy_e", 32, 1),
                                           ("u_mul_e", 64, 2)])
def test_spmm_max_min_f32(graph, device, reduce, op, feat, heads):
    name, g, arr = graph
    rng = np.random.default_rng(3)
    e = arr.COO_src.shape[0]
    rows = e if op == "copy_e" else arr.num_nodes
    x = rng.standard_normal((rows, feat), dtype=np.float32)
    w = rng.standard_normal((e, heads), dtype=np.float32) if op == "u_mul_e" else None
    got = ops.spmm(g, op, reduce, _dev(x, device),
                   None if w is None else _dev(w, device)).cpu().numpy()
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      x, w, op=op, reduce=reduce, heads=heads)
    # a max / min of fp32 products is exact: compare bit for bit
    assert np.array_equal(got, ref), f"{op} {reduce} {name}"


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("op,feat,heads,bf16", [("copy_u", 64, 1, False), ("copy_u", 5, 1, False),
                                                ("copy_e", 16, 1, False), ("u_mul_e", 32, 4, False),
                                                ("u_mul_e", 6, 2, False), ("copy_u", 64, 1, True)])
def test_spmm_arg_outputs_bit_exact(graph, device, reduce, op, feat, heads, bf16):
    """Positions of the extrema: small-integer data (exact products, many ties)
    so that "first extremum in adjacency order wins" decides most elements."""
    name, g, arr = graph
    rng = np.random.default_rng(feat + heads)
    e = arr.COO_src.shape[0]
    rows = e if op == "copy_e" else arr.num_nodes
    x = rng.integers(-3, 4, size=(rows, feat)).astype(np.float32)
    w = rng.integers(-2, 3, size=(e, heads)).astype(np.float32) if op == "u_mul_e" else None
    out, arg_u, arg_e = ops.spmm(g, op, reduce, _dev(x, device, bf16),
                                 None if w is None else _dev(w, device), return_arg=True)
    ref, ref_u, ref_e = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                                    x, w, op=op, reduce=reduce, heads=heads, want_arg=True)
    np.testing.assert_array_equal(out.float().cpu().numpy(), ref, err_msg=f"{name} values")
    assert (arg_u is None) == (op == "copy_e") and (arg_e is None) == (op == "copy_u")
    if arg_u is not None:
        assert arg_u.dtype == torch.int32
        np.testing.assert_array_equal(arg_u.cpu().numpy(), ref_u, err_msg=f"{name} arg_u")
    if arg_e is not None:
        np.testing.assert_array_equal(arg_e.cpu().numpy(), ref_e, err_msg=f"{name} arg_e")


def test_spmm_arg_rejects_sum(graph, device):
    name, g, arr = graph
    x = torch.zeros((arr.num_nodes, 4), device=device)
    with pytest.raises(RuntimeError, match="max or the min"):
        ops.spmm(g, "copy_u", "sum", x, return_arg=True)
    lib = capi.load()
    rc = lib.ga_spmm_csr_arg(g.in_pointer.data_ptr(), g.in_row_of_slot.data_ptr(),
                             g.in_node_indices.data_ptr(), None, x.data_ptr(), None,
                             x.data_ptr(), None, None, arr.num_nodes, g.num_edges, 4, 1,
                             capi.GA_COPY_U, capi.GA_SUM, capi.GA_F32, None, 0, None)
    assert rc == capi.GA_EINVAL


@pytest.mark.parametrize("feat,heads", [(64, 1), (128, 8), (256, 4), (24, 3),
                                        (7, 1)])
def test_spmm_bf16(graph, device, feat, heads):
    name, g, arr = graph
    rng = np.random.default_rng(feat)
    e = arr.COO_src.shape[0]
    x = to_bf16_f32(rng.standard_normal((arr.num_nodes, feat), dtype=np.float32))
    w = rng.standard_normal((e, heads), dtype=np.float32)
    got = ops.gspmm_src_mul_e_sum(_dev(x, device, True), _dev(w, device), [1],
                                  False, None, g)
    assert got.dtype == torch.bfloat16
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      x, w, op="u_mul_e", heads=heads)
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16,
                 f"bf16 u_mul_e {name} F={feat}")
    got = ops.SpMMSrc(_dev(x, device, True), [1], False, None, g)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      x, op="copy_u")
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16, f"bf16 copy_u {name}")


@pytest.mark.parametrize("feat", [1, 4, 8, 5])
@pytest.mark.parametrize("bf16", [False, True])
def test_sddmm_u_add_v_bit_exact(graph, device, feat, bf16):
    name, g, arr = graph
    rng = np.random.default_rng(feat)
    u = rng.standard_normal((arr.num_nodes, feat), dtype=np.float32)
    v = rng.standard_normal((arr.num_nodes, feat), dtype=np.float32)
    if bf16:
        u, v = to_bf16_f32(u), to_bf16_f32(v)
    got = ops.gsddmm_u_add_v_mul_alpha(_dev(u, device, bf16), _dev(v, device, bf16),
                                       1, g)
    assert got.dtype == torch.float32 and got.shape == (arr.COO_src.shape[0], feat)
    ref = oracle.sddmm_u_add_v(arr.COO_src, arr.COO_dst, u, v)
    assert np.array_equal(got.cpu().numpy(), ref), f"u_add_v {name} F={feat}"


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("feat", [1, 4, 5])
def test_sddmm_u_op_v_bit_exact(graph, device, op, feat):
    """One fp32 operation per element: the result must equal the oracle's bit
    for bit (division included: it is correctly rounded on both sides)."""
    name, g, arr = graph
    rng = np.random.default_rng(feat)
    u = rng.standard_normal((arr.num_nodes, feat), dtype=np.float32)
    v = rng.standard_normal((arr.num_nodes, feat), dtype=np.float32)
    v = np.where(np.abs(v) < 0.1, 1.0, v).astype(np.float32)
    got = ops.gsddmm_u_op_v(op, _dev(u, device), _dev(v, device), g).cpu().numpy()
    ref = oracle.sddmm_u_op_v(op, arr.COO_src, arr.COO_dst, u, v)
    assert np.array_equal(got, ref), f"{op} {name}"


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("feat", [1, 2, 4])
def test_sddmm_over_adjacency_bit_exact(device, op, feat):
    """Graphs stored by destination (edge ids = in-adjacency slots) take the kernel
    that walks the adjacency and finds each slot's row from the row pointer: rows of
    every length (a 150,000-edge row over many chunks, single edges), runs of nodes
    without in-edges at the start, in the middle and at the end, edge counts that do
    not fill the last chunk; operands at an offset (row-aligned only)."""
    from graphiler_amd.datasets import sort_by_dst
    rng = np.random.default_rng(feat * 13 + len(op))
    cases = []
    s, d, n = _hub_graph(feat)
    cases.append((s, d + 50, n + 120))                     # empty rows before and after
    s, d = skewed_graph(rng, 1000, 6000, 9000)
    cases.append((s, d, 1000))
    s, d = random_graph(rng, 40, 7)
    cases.append((s, d, 40))
    s, d = random_graph(rng, 5000, 1024 * 3 + 1)
    cases.append((s, np.sort(d) // 7 * 7, 5000))           # rows only at multiples of 7
    for src, dst, n in cases:
        src, dst = sort_by_dst(src, dst)
        g = prepare_graph(src, dst, n, device=device)
        assert g.in_eid_is_identity
        u = rng.standard_normal((n + 1, feat), dtype=np.float32)
        v = rng.standard_normal((n + 1, feat), dtype=np.float32)
        v = np.where(np.abs(v) < 0.1, 1.0, v).astype(np.float32)
        for lead in (0, 1):                                # lead 1: rows start feat*4 bytes in
            ud, vd = _dev(u, device)[lead:lead + n], _dev(v, device)[lead:lead + n]
            got = ops.gsddmm_u_op_v(op, ud, vd, g).cpu().numpy()
            ref = oracle.sddmm_u_op_v(op, src, dst, u[lead:lead + n], v[lead:lead + n])
            assert np.array_equal(got, ref), f"{op} F={feat} n={n} E={src.shape[0]} lead={lead}"


@pytest.mark.parametrize("heads,dim", [(1, 64), (8, 16), (4, 64), (3, 5),
                                       (1, 1), (2, 256), (8, 64), (1, 17), (2, 24),
                                       (1, 300), (5, 129)])
@pytest.mark.parametrize("bf16", [False, True])
def test_sddmm_u_dot_v(graph, device, heads, dim, bf16):
    name, g, arr = graph
    rng = np.random.default_rng(heads * 100 + dim)
    u = rng.standard_normal((arr.num_nodes, heads, dim), dtype=np.float32)
    v = rng.standard_normal((arr.num_nodes, heads, dim), dtype=np.float32)
    if bf16:
        u, v = to_bf16_f32(u), to_bf16_f32(v)
    got = ops.gsddmm_u_dot_v(_dev(u, device, bf16), _dev(v, device, bf16), g)
    ref = oracle.sddmm_u_dot_v(arr.COO_src, arr.COO_dst, u, v)
    # bf16 inputs are exact in fp32; the products are accumulated in fp32
    assert_close(got.cpu().numpy(), ref, TOL_F32, f"u_dot_v {name} {heads}x{dim}",
                 mag=oracle.sddmm_u_dot_v(arr.COO_src, arr.COO_dst, np.abs(u), np.abs(v)))


@pytest.mark.parametrize("heads", [1, 4, 8, 3, 64, 5, 6, 12, 33, 65, 100])
def test_segment_softmax(graph, device, heads):
    name, g, arr = graph
    rng = np.random.default_rng(heads)
    e = arr.COO_src.shape[0]
    x = (rng.standard_normal((e, heads)) * 4.0).astype(np.float32)
    got = ops.SegmentSoftmax(_dev(x, device), 1, None, g).cpu().numpy()
    ref = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, x)
    assert_close(got, ref, TOL_F32, f"softmax {name} H={heads}", mag=ref)
    if e:
        # each non-empty segment sums to one, per head
        sums = oracle.spmm(arr.in_pointer, arr.in_node_indices,
                           arr.in_edge_indices, got.astype(np.float32),
                           op="copy_e")
        nonempty = np.diff(arr.in_pointer) > 0
        assert np.abs(sums[nonempty] - 1.0).max() < 1e-5


def _hub_graph(seed):
    """400 nodes; node 7 has 150,000 in-edges, nodes 8 and 300 have 5,000 and 2,500,
    3,000 more fall anywhere; edge ids shuffled against the adjacency order."""
    rng = np.random.default_rng(seed)
    n = 400
    dst = np.concatenate([np.full(150_000, 7), np.full(5_000, 8), np.full(2_500, 300),
                          rng.integers(0, n, 3_000)]).astype(np.int64)
    dst = dst[rng.permutation(dst.shape[0])]
    src = rng.integers(0, n, dst.shape[0], dtype=np.int64)
    return src, dst, n


def _dot_attention_reference(arr, k, q, v, heads):
    """sum(k * q) -> segment softmax -> weighted sum on the oracle, and the rows' log-sum-exp."""
    n, e = arr.num_nodes, arr.COO_src.shape[0]
    score = oracle.sddmm_u_dot_v(arr.COO_src, arr.COO_dst, k, q).astype(np.float32)
    att = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, score)
    out = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      v.reshape(n, -1), att, op="u_mul_e", heads=heads)
    mag = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      np.abs(v).reshape(n, -1), att, op="u_mul_e", heads=heads)
    lse = np.full((n, heads), -np.inf)
    big = np.full((n, heads), -np.inf)
    np.maximum.at(big, arr.COO_dst, score.astype(np.float64))
    tot = np.zeros((n, heads))
    np.add.at(tot, arr.COO_dst, np.exp(score.astype(np.float64) - big[arr.COO_dst]))
    has = np.diff(arr.in_pointer) > 0
    lse[has] = big[has] + np.log(tot[has])
    return out, mag, lse


@pytest.mark.parametrize("heads,dim", [(8, 16), (1, 64), (4, 8), (2, 32), (1, 128), (16, 8),
                                       (16, 64), (8, 128)])     # more than one tile of 64 lanes per row
@pytest.mark.parametrize("bf16", [False, True])
def test_dot_attention_sum(graph, device, heads, dim, bf16):
    """ga_dot_attention_sum over the graph's in-adjacency (queries on the destinations)."""
    name, g, arr = graph
    rng = np.random.default_rng(heads * 1000 + dim)
    n = arr.num_nodes
    k, q, v = (rng.standard_normal((n, heads, dim), dtype=np.float32) for _ in range(3))
    k *= 0.5
    if bf16:
        k, q, v = to_bf16_f32(k), to_bf16_f32(q), to_bf16_f32(v)
    if dim // (8 if bf16 else 4) > 16:          # a head wider than 16 lanes of 16 bytes
        if arr.COO_src.shape[0]:
            with pytest.raises(capi.GraphilerError) as err:
                ops.dot_attention_sum(_dev(k, device, bf16), _dev(q, device, bf16),
                                      _dev(v, device, bf16), g)
            assert err.value.code == capi.GA_EUNSUPPORTED
        return
    out, lse = ops.dot_attention_sum(_dev(k, device, bf16), _dev(q, device, bf16),
                                     _dev(v, device, bf16), g, return_lse=True)
    assert out.shape == (n, heads, dim) and lse.shape == (n, heads)
    ref, mag, ref_lse = _dot_attention_reference(arr, k, q, v, heads)
    assert_close(out.float().cpu().numpy().reshape(n, -1), ref, TOL_BF16 if bf16 else TOL_F32,
                 f"dot attention {name} {heads}x{dim}", mag=mag)
    got_lse = lse.cpu().numpy()
    has = np.diff(arr.in_pointer) > 0
    assert np.all(np.isneginf(got_lse[~has])) and np.all(np.isfinite(got_lse[has]))
    if has.any():
        assert np.abs(got_lse[has] - ref_lse[has]).max() <= 2e-5 * max(1.0, np.abs(ref_lse[has]).max())
    only = ops.dot_attention_sum(_dev(k, device, bf16), _dev(q, device, bf16), _dev(v, device, bf16), g)
    assert torch.equal(only.view(torch.int16 if bf16 else torch.int32),
                       out.view(torch.int16 if bf16 else torch.int32))


@pytest.mark.parametrize("bf16", [False, True])
def test_dot_attention_sum_long_rows_and_rejects(device, bf16):
    """Rows of 150,000 / 5,000 / 2,500 slots (partial states chained across workgroups),
    and the shapes the kernel does not take."""
    src, dst, n = _hub_graph(11)
    g = prepare_graph(src, dst, n, device=device)
    arr = build_graph_arrays(src, dst, n)
    rng = np.random.default_rng(12)
    heads, dim = 4, 16
    k, q, v = (rng.standard_normal((n, heads, dim), dtype=np.float32) for _ in range(3))
    k *= 0.25
    if bf16:
        k, q, v = to_bf16_f32(k), to_bf16_f32(q), to_bf16_f32(v)
    out, lse = ops.dot_attention_sum(_dev(k, device, bf16), _dev(q, device, bf16),
                                     _dev(v, device, bf16), g, return_lse=True)
    ref, mag, ref_lse = _dot_attention_reference(arr, k, q, v, heads)
    assert_close(out.float().cpu().numpy().reshape(n, -1), ref, TOL_BF16 if bf16 else TOL_F32,
                 "dot attention, long rows", mag=mag)
    has = np.diff(arr.in_pointer) > 0
    assert np.abs(lse.cpu().numpy()[has] - ref_lse[has]).max() <= 2e-5 * np.abs(ref_lse[has]).max()
    bad = torch.randn(n, 2, 6, device=device)                    # heads of 6: not 4 (8) values wide
    if bf16:
        bad = bad.bfloat16()
    with pytest.raises(capi.GraphilerError) as err:
        ops.dot_attention_sum(bad, bad, bad, g)
    assert err.value.code == capi.GA_EUNSUPPORTED
    with pytest.raises(RuntimeError):
        ops.dot_attention_sum(_dev(k, device, bf16), _dev(q, device, bf16)[:, :2], _dev(v, device, bf16), g)


@pytest.mark.parametrize("bf16", [False, True])
def test_transpose_scale_blocks(device, bf16):
    """ga_transpose_scale_blocks: every D x D block transposed, times its scale and a
    constant, in fp32 with one rounding -- bit for bit the same arithmetic in ATen."""
    lib = capi.load()
    dt = torch.bfloat16 if bf16 else torch.float32
    stream = torch.cuda.current_stream().cuda_stream
    for t, h, d in ((5, 3, 8), (10, 8, 16), (1, 1, 1), (2, 1, 33)):
        w = torch.randn(t, h, d, d, device=device).to(dt)
        scale = torch.rand(t, h, device=device) + 0.5
        for sc, factor in ((scale, 0.25), (None, 1.0), (scale, 1.0 / 3.0)):
            out = torch.full_like(w, float("nan"))
            rc = lib.ga_transpose_scale_blocks(w.data_ptr(), None if sc is None else sc.data_ptr(),
                                               factor, out.data_ptr(), t * h, d,
                                               capi.GA_BF16 if bf16 else capi.GA_F32, stream)
            assert rc == 0, rc
            want = w.float().transpose(-1, -2)
            if sc is not None:
                want = want * sc[:, :, None, None]
            want = (want * torch.tensor(factor, dtype=torch.float32, device=device)).to(dt)
            assert torch.equal(out.view(torch.int16 if bf16 else torch.int32),
                               want.contiguous().view(torch.int16 if bf16 else torch.int32))
    w = torch.randn(2, 4, 4, device=device)
    assert lib.ga_transpose_scale_blocks(w.data_ptr(), None, 1.0, w.data_ptr(), 2, 4, capi.GA_F32,
                                         stream) == capi.GA_EINVAL           # in place
    assert lib.ga_transpose_scale_blocks(None, None, 1.0, None, 0, 4, capi.GA_F32, stream) == 0


@pytest.mark.parametrize("feat,heads,bf16", [(64, 1, False), (256, 4, True), (17, 1, False),
                                             (1, 1, False), (128, 8, False)])
def test_row_reductions_over_many_workgroups(device, feat, heads, bf16):
    """A 150,000-edge row spans hundreds to thousands of workgroups of the row
    reductions, so its partial states are combined by whole blocks (pieces of the
    chain in parallel, then in order); the 5,000- and 2,500-edge rows take the
    sequential chain.  Sums, extrema with their positions (small integers: exact, many
    ties), the fused GAT chain and the per-edge softmax sum against the oracle."""
    src, dst, n = _hub_graph(feat + heads)
    rng = np.random.default_rng(feat)
    e = src.shape[0]
    g = prepare_graph(src, dst, n, device=device)
    arr = build_graph_arrays(src, dst, n)
    adj = (arr.in_pointer, arr.in_node_indices, arr.in_edge_indices)
    tol = TOL_BF16 if bf16 else TOL_F32
    x = rng.standard_normal((n, feat), dtype=np.float32)
    w = rng.standard_normal((e, heads), dtype=np.float32)
    if bf16:
        x = to_bf16_f32(x)
    xd = _dev(x, device, bf16)
    got = ops.SpMMSrc(xd, [1], False, None, g).float().cpu().numpy()
    assert_close(got, oracle.spmm(*adj, x, op="copy_u"), tol, f"copy_u F={feat}",
                 mag=oracle.spmm(*adj, np.abs(x), op="copy_u"))
    got = ops.gspmm_src_mul_e_sum(xd, _dev(w, device), [1], False, None, g).float().cpu().numpy()
    assert_close(got, oracle.spmm(*adj, x, w, op="u_mul_e", heads=heads), tol, f"u_mul_e F={feat}",
                 mag=oracle.spmm(*adj, np.abs(x), np.abs(w), op="u_mul_e", heads=heads))

    xi = rng.integers(-3, 4, size=(n, feat)).astype(np.float32)
    out, arg_u, _ = ops.spmm(g, "copy_u", "max", _dev(xi, device, bf16), None, return_arg=True)
    ref, ref_u, _ = oracle.spmm(*adj, xi, None, op="copy_u", reduce="max", heads=1, want_arg=True)
    np.testing.assert_array_equal(out.float().cpu().numpy(), ref)
    np.testing.assert_array_equal(arg_u.cpu().numpy(), ref_u)

    dim = feat // heads
    el = rng.standard_normal((n, heads), dtype=np.float32) * 2
    er = rng.standard_normal((n, heads), dtype=np.float32) * 2
    got = ops.gat_aggregate(_dev(el, device), _dev(er, device), xd, g, 0.2).float().cpu().numpy()
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, x, heads=heads, slope=0.2)
    assert_close(got, ref, tol, f"fused GAT {heads}x{dim}",
                 mag=oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, np.abs(x),
                                          heads=heads, slope=0.2))

    logit = (rng.standard_normal((e, heads)) * 3).astype(np.float32)
    m = rng.standard_normal((e, feat), dtype=np.float32)
    if bf16:
        m = to_bf16_f32(m)
    att = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, logit)
    prod = (m.reshape(e, heads, dim).astype(np.float64) * att[:, :, None]).reshape(e, -1)
    got = ops.edge_softmax_sum(_dev(logit, device), _dev(m, device, bf16), g).float().cpu().numpy()
    assert_close(got, oracle.spmm(*adj, prod.astype(np.float32), op="copy_e"),
                 TOL_BF16 if bf16 else TOL_F32, f"edge_softmax_sum {heads}x{dim}")


@pytest.mark.parametrize("heads", [1, 8, 32, 3, 12, 100])
def test_segment_softmax_rows_over_many_chunks(device, heads):
    """A row of 150,000 edges next to ordinary ones: its statistics are merged from
    hundreds to thousands of per-chunk partials (once per row), and two more long
    rows share chunks with it.  Edge ids shuffled against the adjacency order."""
    rng = np.random.default_rng(heads + 77)
    src, dst, n = _hub_graph(heads + 77)
    g = prepare_graph(src, dst, n, device=device)
    arr = build_graph_arrays(src, dst, n)
    x = (rng.standard_normal((dst.shape[0], heads)) * 4.0).astype(np.float32)
    got = ops.SegmentSoftmax(_dev(x, device), 1, None, g).cpu().numpy()
    ref = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, x)
    assert_close(got, ref, TOL_F32, f"softmax long rows H={heads}", mag=ref)
    sums = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                       got.astype(np.float32), op="copy_e")
    assert np.abs(sums[np.diff(arr.in_pointer) > 0] - 1.0).max() < 2e-5


def test_segment_softmax_in_place(device):
    """y == x is allowed at the C boundary (rows over many chunks and short ones, heads
    on both kernel families) and gives the bits of the out-of-place call."""
    lib = capi.load()
    src, dst, n = _hub_graph(5)
    g = prepare_graph(src, dst, n, device=device)
    rng = np.random.default_rng(5)
    for heads in (1, 4, 3):
        x = _dev((rng.standard_normal((dst.shape[0], heads)) * 4.0).astype(np.float32), device)
        want = ops.SegmentSoftmax(x, 1, None, g)
        y = x.clone()
        ws = g.workspace(lib.ga_softmax_workspace_bytes(g.num_edges, heads))
        rc = lib.ga_segment_softmax(
            g.in_pointer.data_ptr(), g.in_row_of_slot.data_ptr(),
            None if g.in_eid_is_identity else g.in_edge_indices.data_ptr(),
            y.data_ptr(), y.data_ptr(), g.num_nodes, g.num_edges, heads,
            ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc
        assert torch.equal(y, want), f"in-place softmax differs at H={heads}"
        # an output that starts inside the input is refused before anything runs
        both = torch.empty(x.numel() + heads, device=device)
        rc = lib.ga_segment_softmax(
            g.in_pointer.data_ptr(), g.in_row_of_slot.data_ptr(),
            None if g.in_eid_is_identity else g.in_edge_indices.data_ptr(),
            both.data_ptr(), both.data_ptr() + 4 * heads, g.num_nodes, g.num_edges, heads,
            ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
        assert rc == capi.GA_EINVAL


def _mask_some_logits(rng, ptr, eid, x):
    """-inf on about a third of the logits, keeping one finite logit per row and head."""
    x = x.copy()
    mask = rng.random(x.shape) < 0.35
    for v in range(len(ptr) - 1):
        if ptr[v + 1] > ptr[v]:
            mask[eid[ptr[v] + rng.integers(0, ptr[v + 1] - ptr[v])]] = False
    x[mask] = -np.inf
    return x


@pytest.mark.parametrize("heads", [1, 8, 100])
def test_segment_softmax_masked_logits(device, heads):
    """-inf logits (masked edges) weigh exactly 0 and leave the other edges of their
    row untouched, as expf(-inf - max) = 0 does in segment_softmax_kernel.cu:22-45;
    rows of every length incl. the 150,000-edge one, leading -inf runs included."""
    rng = np.random.default_rng(heads + 5)
    src, dst, n = _hub_graph(heads + 5)
    g = prepare_graph(src, dst, n, device=device)
    arr = build_graph_arrays(src, dst, n)
    x = (rng.standard_normal((dst.shape[0], heads)) * 4.0).astype(np.float32)
    x = _mask_some_logits(rng, arr.in_pointer, arr.in_edge_indices, x)
    got = ops.SegmentSoftmax(_dev(x, device), 1, None, g).cpu().numpy()
    ref = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, x)
    assert np.isfinite(got).all()
    assert not got[np.isneginf(x)].any()
    assert_close(got, ref, TOL_F32, f"softmax with -inf logits H={heads}", mag=ref)


@pytest.mark.parametrize("feat,heads", [(64, 1), (128, 8), (17, 1)])
def test_fused_softmax_sums_masked_logits(device, feat, heads):
    """The fused GAT pass and the per-edge softmax sum with -inf logits: a source whose
    attention term is -inf contributes nothing, also when the -inf edges come first in
    a row (the running maximum is then still -inf)."""
    rng = np.random.default_rng(feat + heads)
    src, dst, n = _hub_graph(feat)
    src[:] = rng.integers(1, n, src.shape[0])      # node 0 is never the only source ...
    g = prepare_graph(src, dst, n, device=device)
    arr = build_graph_arrays(src, dst, n)
    e = src.shape[0]
    z = rng.standard_normal((n, feat), dtype=np.float32)
    el = rng.standard_normal((n, heads), dtype=np.float32) * 2
    er = rng.standard_normal((n, heads), dtype=np.float32) * 2
    el[rng.random(n) < 0.3] = -np.inf
    has_finite = np.zeros(n, bool)
    has_finite[dst[np.isfinite(el[src, 0])]] = True
    extra = np.flatnonzero(~has_finite & (np.diff(arr.in_pointer) > 0))
    el[src[arr.in_edge_indices[arr.in_pointer[extra]]]] = 0.5   # ... every row keeps a finite logit
    got = ops.gat_aggregate(_dev(el, device), _dev(er, device), _dev(z, device), g, 0.2).cpu().numpy()
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, z, heads=heads, slope=0.2)
    assert np.isfinite(got).all()
    assert_close(got, ref, TOL_F32, f"fused GAT with -inf terms {heads}x{feat // heads}")

    logit = (rng.standard_normal((e, heads)) * 3).astype(np.float32)
    logit = _mask_some_logits(rng, arr.in_pointer, arr.in_edge_indices, logit)
    m = rng.standard_normal((e, feat), dtype=np.float32)
    att = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, logit)
    prod = (m.reshape(e, heads, -1).astype(np.float64) * att[:, :, None]).reshape(e, -1)
    got = ops.edge_softmax_sum(_dev(logit, device), _dev(m, device), g).cpu().numpy()
    assert np.isfinite(got).all()
    assert_close(got, oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                                  prod.astype(np.float32), op="copy_e"),
                 TOL_F32, f"edge_softmax_sum with -inf logits {heads}x{feat // heads}")


def test_segment_softmax_1d_input(graph, device):
    name, g, arr = graph
    rng = np.random.default_rng(0)
    x = rng.standard_normal(arr.COO_src.shape[0]).astype(np.float32)
    got = ops.SegmentSoftmax(_dev(x, device), 1, None, g)
    assert got.shape == x.shape
    ref = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, x)
    assert_close(got.cpu().numpy(), ref, TOL_F32, f"softmax 1-D {name}", mag=ref)


@pytest.mark.parametrize("shape,dtype", [((64,), np.float32), ((1,), np.float32),
                                         ((3, 5), np.float32), ((7,), np.int64),
                                         ((128,), np.float16), ((3,), np.uint8),
                                         ((17,), np.float32), ((129,), np.float32),
                                         ((18,), np.float32), ((33,), np.float16),
                                         ((5,), np.uint8), ((100,), np.float64),
                                         ((67,), np.float32), ((258,), np.float16),
                                         ((1025,), np.float32)])
def test_broadcast_bit_exact(graph, device, shape, dtype):
    name, g, arr = graph
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((arr.num_nodes,) + shape) * 100).astype(dtype)
    dx = _dev(x, device)
    assert np.array_equal(ops.BroadcastSrcNode(dx, g).cpu().numpy(),
                          oracle.gather_rows(arr.COO_src, x))
    assert np.array_equal(ops.BroadcastDstNode(dx, g).cpu().numpy(),
                          oracle.gather_rows(arr.COO_dst, x))


def test_check_input_errors(device):
    dbg = datasets.debug_graph()
    g = prepare_graph(dbg.src, dbg.dst, 3, device=device)
    x = torch.ones(3, 4)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ops.SpMMSrc(x, [1], False, None, g)
    xt = torch.ones(4, 3, device=device).t()
    with pytest.raises(RuntimeError, match="must be contiguous"):
        ops.SpMMSrc(xt, [1], False, None, g)
    with pytest.raises(RuntimeError):
        ops.SegmentSoftmax(torch.ones(6, 1, device=device), 0, None, g)
    with pytest.raises(RuntimeError):
        ops.BroadcastEdgeType(torch.ones(2, 2, device=device), g)


@pytest.mark.parametrize("heads,dim", [(1, 64), (4, 64), (8, 16), (1, 1),
                                       (3, 5), (2, 100)])
@pytest.mark.parametrize("bf16", [False, True])
def test_gat_aggregate_fused(graph, device, heads, dim, bf16):
    name, g, arr = graph
    rng = np.random.default_rng(heads * 31 + dim)
    n = arr.num_nodes
    el = rng.standard_normal((n, heads), dtype=np.float32) * 2
    er = rng.standard_normal((n, heads), dtype=np.float32) * 2
    z = rng.standard_normal((n, heads * dim), dtype=np.float32)
    if bf16:
        z = to_bf16_f32(z)
    got = ops.gat_aggregate(_dev(el, device), _dev(er, device),
                            _dev(z, device, bf16), g, 0.2)
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, z,
                               heads=heads, slope=0.2)
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 f"fused GAT {name} {heads}x{dim} bf16={bf16}",
                 mag=oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, np.abs(z),
                                          heads=heads, slope=0.2))
    assert not got.float().cpu().numpy()[np.diff(arr.in_pointer) == 0].any()


@pytest.mark.parametrize("feat", [3, 7, 17, 41, 65, 130, 255])
@pytest.mark.parametrize("bf16", [False, True])
def test_one_head_rows_without_16_byte_tiles(graph, device, feat, bf16):
    """Feature rows that 16-byte accesses do not tile (odd widths, bf16 widths that
    are not multiples of 8), one head: the row reductions then give each lane four
    features a lane-group width apart.  Copy and weighted sums, a max, the fused GAT
    chain and the per-edge softmax sum against the oracle; the unaligned-base case
    takes the same kernels from a view that starts one element into a buffer."""
    name, g, arr = graph
    rng = np.random.default_rng(feat * 3 + bf16)
    n, e = arr.num_nodes, arr.COO_src.shape[0]
    tol = TOL_BF16 if bf16 else TOL_F32
    x = rng.standard_normal((n, feat), dtype=np.float32)
    m = rng.standard_normal((e, feat), dtype=np.float32)
    w = rng.standard_normal((e, 1), dtype=np.float32)
    if bf16:
        x, m = to_bf16_f32(x), to_bf16_f32(m)
    xd, md, wd = _dev(x, device, bf16), _dev(m, device, bf16), _dev(w, device)
    adj = (arr.in_pointer, arr.in_node_indices, arr.in_edge_indices)
    empty = np.diff(arr.in_pointer) == 0

    got = ops.SpMMSrc(xd, [1], False, None, g).float().cpu().numpy()
    assert_close(got, oracle.spmm(*adj, x, op="copy_u"), tol, f"copy_u {name} F={feat}")
    assert not got[empty].any()
    shifted = torch.empty(n * feat + 1, dtype=xd.dtype, device=device)[1:].view(n, feat)
    shifted.copy_(xd)
    got = ops.SpMMSrc(shifted, [1], False, None, g).float().cpu().numpy()
    assert_close(got, oracle.spmm(*adj, x, op="copy_u"), tol, f"copy_u shifted {name} F={feat}")
    got = ops.SpMMEdge(md, [1], False, None, g).float().cpu().numpy()
    assert_close(got, oracle.spmm(*adj, m, op="copy_e"), tol, f"copy_e {name} F={feat}")
    got = ops.gspmm_src_mul_e_sum(xd, wd, [1], False, None, g).float().cpu().numpy()
    assert_close(got, oracle.spmm(*adj, x, w, op="u_mul_e", heads=1), tol,
                 f"u_mul_e {name} F={feat}")
    got = ops.spmm(g, "copy_u", "max", xd).float().cpu().numpy()
    ref = oracle.spmm(*adj, x, op="copy_u", reduce="max")
    assert np.array_equal(np.isfinite(got), np.isfinite(ref))
    assert np.array_equal(got[~empty], ref[~empty]), f"max {name} F={feat}"

    el = rng.standard_normal((n, 1), dtype=np.float32) * 2
    er = rng.standard_normal((n, 1), dtype=np.float32) * 2
    got = ops.gat_aggregate(_dev(el, device), _dev(er, device), xd, g, 0.2).float().cpu().numpy()
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, x, heads=1, slope=0.2)
    assert_close(got, ref, tol, f"fused GAT {name} D={feat}")
    assert not got[empty].any()

    logit = (rng.standard_normal((e, 1)) * 3).astype(np.float32)
    att = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, logit)
    prod = (m.astype(np.float64) * att).astype(np.float32)
    got = ops.edge_softmax_sum(_dev(logit, device), md, g).float().cpu().numpy()
    assert_close(got, oracle.spmm(*adj, prod, op="copy_e"), TOL_BF16 if bf16 else TOL_F32,
                 f"edge_softmax_sum {name} D={feat}")


@pytest.mark.parametrize("heads,dim,bf16", [(1, 64, False), (4, 64, True), (8, 16, True),
                                            (2, 8, False), (3, 32, False), (1, 16, True)])
def test_gat_aggregate_from_z(graph, device, heads, dim, bf16):
    """Source term recomputed from the gathered row: equals the fused chain fed
    with el = z . a_l (oracle, float64 dot of the stored rows)."""
    name, g, arr = graph
    n = arr.num_nodes
    rng = np.random.default_rng(heads * 31 + dim)
    z = rng.standard_normal((n, heads * dim), dtype=np.float32)
    if bf16:
        z = to_bf16_f32(z)
    a_l = (rng.standard_normal((heads, dim)) / np.sqrt(dim)).astype(np.float32)
    er = rng.standard_normal((n, heads), dtype=np.float32)
    el = np.einsum("nhd,hd->nh", z.reshape(n, heads, dim).astype(np.float64), a_l).astype(np.float32)
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, z, heads=heads,
                               slope=0.2)
    got = ops.gat_aggregate_from_z(_dev(a_l, device), _dev(er, device), _dev(z, device, bf16),
                                   g, 0.2)
    assert_close(got.float().cpu().numpy().reshape(ref.shape), ref,
                 TOL_BF16 if bf16 else TOL_F32, f"gat from z on {name}")


@pytest.mark.parametrize("heads,dim", [(1, 64), (4, 16), (3, 5)])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("activation", ["elu", "relu"])
def test_gat_aggregate_with_activation(graph, device, heads, dim, bf16, activation):
    """The layer's activation applied by the fused pass to the rows it stores (the F.elu
    between the layers of examples/GAT/GAT.py): activation(oracle chain) in float64; relu
    also bit for bit against torch.relu of the plain result (it commutes with rounding)."""
    name, g, arr = graph
    n = arr.num_nodes
    rng = np.random.default_rng(heads * 17 + dim)
    z = rng.standard_normal((n, heads * dim), dtype=np.float32)
    if bf16:
        z = to_bf16_f32(z)
    el = rng.standard_normal((n, heads), dtype=np.float32)
    er = rng.standard_normal((n, heads), dtype=np.float32)
    ref = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, z, heads=heads,
                               slope=0.2).astype(np.float64)
    ref = np.where(ref > 0, ref, np.expm1(ref) if activation == "elu" else 0.0)
    args = (_dev(el, device), _dev(er, device), _dev(z, device, bf16), g, 0.2)
    got = ops.gat_aggregate(*args, activation=activation)
    assert_close(got.float().cpu().numpy().reshape(ref.shape), ref,
                 TOL_BF16 if bf16 else TOL_F32, f"gat + {activation} on {name}")
    if activation == "relu":
        assert torch.equal(got, torch.relu(ops.gat_aggregate(*args)))
    elif not bf16:
        # sums of about 1e-4: exp(o) - 1 would cancel to 1e-3 relative there, F.elu's expm1
        # does not; every element is held to the size of its row's terms
        zs = (z * np.float32(1e-4)).astype(np.float32)
        pre = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, zs, heads=heads,
                                   slope=0.2).astype(np.float64)
        mag = oracle.gat_aggregate(arr.in_pointer, arr.in_node_indices, el, er, np.abs(zs),
                                   heads=heads, slope=0.2)
        small = ops.gat_aggregate(_dev(el, device), _dev(er, device), _dev(zs, device), g, 0.2,
                                  activation="elu")
        assert_close(small.cpu().numpy().reshape(pre.shape), np.where(pre > 0, pre, np.expm1(pre)),
                     TOL_F32, f"gat + elu on sums near 1e-4, {name}", mag=mag)
    if dim in (16, 64):          # head widths the source-term variant takes
        a_l = (rng.standard_normal((heads, dim)) / np.sqrt(dim)).astype(np.float32)
        plain = ops.gat_aggregate_from_z(_dev(a_l, device), _dev(er, device), _dev(z, device, bf16), g, 0.2)
        fused = ops.gat_aggregate_from_z(_dev(a_l, device), _dev(er, device), _dev(z, device, bf16), g, 0.2,
                                         activation=activation)
        want = torch.relu(plain.float()) if activation == "relu" else torch.nn.functional.elu(plain.float())
        assert_close(fused.float().cpu().numpy(), want.cpu().numpy(), TOL_BF16 if bf16 else TOL_F32,
                     f"gat from z + {activation} on {name}")
    with pytest.raises(RuntimeError):
        ops.gat_aggregate(*args, activation="gelu")


def test_gat_aggregate_from_z_unsupported_head_width(device):
    g = prepare_graph(np.array([0, 1]), np.array([1, 0]), 2, device=device)
    with pytest.raises(capi.GraphilerError):          # 24 / 4 = 6 lanes per head
        ops.gat_aggregate_from_z(torch.ones(1, 24, device=device), torch.ones(2, 1, device=device),
                                 torch.ones(2, 24, device=device), g, 0.2)


def test_gat_layer_plan_equals_fused(graph, device):
    from graphiler_amd import layers
    name, g, arr = graph
    rng = np.random.default_rng(5)
    n = arr.num_nodes
    h = torch.from_numpy(rng.standard_normal((n, 40), dtype=np.float32)).to(device)
    w = torch.from_numpy(datasets.glorot(rng, (40, 32))).to(device)
    a = torch.from_numpy(datasets.glorot(rng, (2, 2, 16))).to(device)
    plan = layers.gat_layer(g, h, w, a, 2, 0.2, fused=False).cpu().numpy()
    fused = layers.gat_layer(g, h, w, a, 2, 0.2, fused=True).cpu().numpy()
    assert_close(fused, plan, TOL_F32, f"GAT layer plan vs fused {name}")


def _typed_rows(rng, counts):
    tp = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    return tp, int(tp[-1])


@pytest.mark.parametrize("K,M,heads", [(16, 64, 1), (64, 8, 1), (64, 64, 1),
                                       (128, 128, 1), (20, 12, 1), (6, 5, 1),
                                       (16, 16, 8), (32, 48, 2), (8, 3, 3),
                                       (256, 32, 1), (128, 200, 1), (256, 64, 1),
                                       (512, 64, 1), (256, 128, 1), (132, 16, 2)])
@pytest.mark.parametrize("bf16", [False, True])
def test_segment_mm(device, K, M, heads, bf16):
    rng = np.random.default_rng(K * 1000 + M + heads)
    counts = [70, 0, 1, 333, 0, 0, 64, 15, 129, 2000, 0]
    tp, rows = _typed_rows(rng, counts)
    X = rng.standard_normal((rows, heads * K), dtype=np.float32)
    W = (rng.standard_normal((len(counts), heads, K, M)) / np.sqrt(K)).astype(np.float32)
    if bf16:
        X, W = to_bf16_f32(X), to_bf16_f32(W)
    lib = capi.load()
    dX, dW = _dev(X, device, bf16), _dev(W, device, bf16)
    dtp = _dev(tp, device)
    Y = torch.full((rows, heads * M), float("nan"), dtype=dX.dtype, device=device)
    rc = lib.ga_segment_mm(dtp.data_ptr(), len(counts), dX.data_ptr(), dW.data_ptr(),
                           Y.data_ptr(), rows, heads, K, M,
                           capi.GA_BF16 if bf16 else capi.GA_F32,
                           torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    ref = oracle.segment_mm(tp, X, W, heads=heads)
    assert_close(Y.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 f"segment_mm K={K} M={M} H={heads} bf16={bf16}",
                 mag=oracle.segment_mm(tp, np.abs(X), np.abs(W), heads=heads))


def test_segment_mm_ops_and_rgcn_layer(device):
    """SegmentMMEdge / SegmentMMNode through the operator wrappers, and the
    RGCN plan BroadcastSrcNode -> SegmentMMEdge -> mul(norm) -> SpMMEdge."""
    from graphiler_amd import layers
    wl = datasets.rgcn_zipf(num_nodes=3000, n_edges=40_000, n_rel=60, seed=2)
    ntype = np.sort(np.random.default_rng(0).integers(0, 4, wl.num_nodes))
    g = prepare_graph(wl.src, wl.dst, wl.num_nodes, device=device,
                      ntype_of=ntype, num_ntypes=4, etype_of=wl.etype, num_etypes=60)
    arr = build_graph_arrays(wl.src, wl.dst, wl.num_nodes)
    rng = np.random.default_rng(2)
    h = rng.standard_normal((wl.num_nodes, 16), dtype=np.float32)
    W = datasets.glorot(rng, (60, 16, 64))
    deg = np.maximum(np.bincount(wl.dst, minlength=wl.num_nodes), 1)
    norm = (1.0 / deg[wl.dst]).astype(np.float32)[:, None]
    got = layers.rgcn_layer(g, _dev(h, device), _dev(W, device), _dev(norm, device))
    etp = oracle.type_pointer(wl.etype, 60)
    msg = oracle.segment_mm(etp, oracle.gather_rows(wl.src, h), W) * norm
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      msg.astype(np.float32), op="copy_e")
    assert_close(got.cpu().numpy(), ref, TOL_F32, "RGCN layer")
    Wn = datasets.glorot(rng, (4, 16, 32))
    got = ops.SegmentMMNode(_dev(h, device), _dev(Wn, device), g)
    ref = oracle.segment_mm(oracle.type_pointer(ntype, 4), h, Wn)
    assert_close(got.cpu().numpy(), ref, TOL_F32, "SegmentMMNode")
    with pytest.raises(RuntimeError, match="type pointer"):
        g2 = prepare_graph(wl.src, wl.dst, wl.num_nodes, device=device)
        ops.SegmentMMEdge(_dev(h[:1], device), _dev(W, device), g2)


@pytest.mark.parametrize("K,M,heads,bf16", [
    (16, 64, 1, False), (64, 64, 1, False), (16, 16, 8, False), (64, 8, 1, False),
    (12, 48, 2, False), (128, 128, 1, False), (200, 16, 1, False),
    (16, 16, 8, True), (64, 64, 1, True), (32, 32, 4, True), (16, 64, 1, True),
    (64, 48, 1, True), (32, 32, 3, True), (8, 16, 5, True), (8, 16, 3, False)])
def test_segment_mm_gather_and_dot(device, K, M, heads, bf16):
    """Y[e] = X[endpoint(e)] @ W[type(e)] read through the COO columns, and its
    reduction against a second gathered row; expected values: the oracle's
    segment_mm on numpy-gathered rows and a float64 einsum.  (200, 16) falls outside
    the fused kernel's shapes and (12, 48, 2 heads) / bf16 (64, 48) outside the dot
    form's: the entry point must say so and the operator wrapper must still give the
    result."""
    rng = np.random.default_rng(K * 131 + M * 7 + heads + 1000 * bf16)
    counts = [70, 0, 1, 333, 0, 64, 15, 129, 2001, 0]
    n_nodes, n_rel = 500, len(counts)
    etype = np.repeat(np.arange(n_rel), counts).astype(np.int64)
    e = etype.shape[0]
    src = rng.integers(0, n_nodes, e, dtype=np.int64)
    dst = rng.integers(0, n_nodes, e, dtype=np.int64)
    g = prepare_graph(src, dst, n_nodes, device=device, etype_of=etype, num_etypes=n_rel)
    X = rng.standard_normal((n_nodes, heads * K), dtype=np.float32)
    Q = rng.standard_normal((n_nodes, heads * M), dtype=np.float32)
    W = (rng.standard_normal((n_rel, heads, K, M)) / np.sqrt(K)).astype(np.float32)
    if bf16:
        X, Q, W = to_bf16_f32(X), to_bf16_f32(Q), to_bf16_f32(W)
    dX, dQ, dW = _dev(X, device, bf16), _dev(Q, device, bf16), _dev(W, device, bf16)
    tol = TOL_BF16 if bf16 else TOL_F32
    tp = oracle.type_pointer(etype, n_rel)
    lib = capi.load()
    stream = torch.cuda.current_stream().cuda_stream
    dt = capi.GA_BF16 if bf16 else capi.GA_F32
    kb = 32 if bf16 else 16
    fits = heads * K <= 8 * kb and heads * M <= 128 and K % (8 if bf16 else 4) == 0
    blocks = -(-heads * M // 16)
    cg = max(1 << (blocks - 1).bit_length(), 2 if bf16 else 1)     # column blocks, power of two
    dot_fits = fits and M % cg == 0 and M // cg in (1, 2, 4, 8, 16)
    for which, col in ((0, src), (1, dst)):
        ref = oracle.segment_mm(tp, X[col], W, heads=heads)
        Y = torch.full((e, heads * M), float("nan"), dtype=dX.dtype, device=device)
        rc = lib.ga_segment_mm_gather(
            g.etype_pointer.data_ptr(), n_rel, dX.data_ptr(),
            (g.COO_src if which == 0 else g.COO_dst).data_ptr(), dW.data_ptr(), Y.data_ptr(),
            None, None, None, None, None, e, heads, K, M, dt, stream)
        assert rc == (0 if fits else capi.GA_EUNSUPPORTED)
        if fits:
            assert_close(Y.float().cpu().numpy(), ref, tol, f"segment_mm_gather {which}")
        got = ops.SegmentMMEdgeGather(dX, dW, which, g)
        assert_close(got.float().cpu().numpy(), ref, tol, f"SegmentMMEdgeGather {which}")
        norm = rng.uniform(0.25, 2.0, (e, 1)).astype(np.float32)        # per-row factor
        got = ops.SegmentMMEdgeGather(dX, dW, which, g, row_scale=_dev(norm, device))
        assert_close(got.float().cpu().numpy(), ref * norm, tol, f"SegmentMMEdgeGather scaled {which}")
        # dot against the other endpoint's row of Q
        other = dst if which == 0 else src
        y64 = np.einsum("ehk,ehkm->ehm", X[col].reshape(e, heads, K).astype(np.float64),
                        W[etype].astype(np.float64))
        want = np.einsum("ehm,ehm->eh", y64, Q[other].reshape(e, heads, M).astype(np.float64))
        D = torch.full((e, heads), float("nan"), dtype=torch.float32, device=device)
        rc = lib.ga_segment_mm_gather(
            g.etype_pointer.data_ptr(), n_rel, dX.data_ptr(),
            (g.COO_src if which == 0 else g.COO_dst).data_ptr(), dW.data_ptr(), None,
            dQ.data_ptr(), (g.COO_dst if which == 0 else g.COO_src).data_ptr(), None,
            D.data_ptr(), None, e, heads, K, M, dt, stream)
        assert rc == (0 if dot_fits else capi.GA_EUNSUPPORTED)
        if dot_fits:
            assert_close(D.cpu().numpy(), want, tol, f"segment_mm dot {which}")
        got = ops.SegmentMMEdgeDot(dX, dW, which, dQ, 1 - which, g)
        assert got.shape == (e, heads) and got.dtype == torch.float32
        assert_close(got.cpu().numpy(), want, tol, f"SegmentMMEdgeDot {which}")
        scale = rng.uniform(0.5, 2.0, (n_rel, heads)).astype(np.float32)
        got = ops.SegmentMMEdgeDot(dX, dW, which, dQ, 1 - which, g, scale=_dev(scale, device))
        assert_close(got.cpu().numpy(), want * scale[etype], tol, f"SegmentMMEdgeDot scaled {which}")
    # identity index (NULL) = plain segment_mm on per-edge rows
    Xe = rng.standard_normal((e, heads * K), dtype=np.float32)
    if bf16:
        Xe = to_bf16_f32(Xe)
    dXe = _dev(Xe, device, bf16)
    if fits:
        Y = torch.full((e, heads * M), float("nan"), dtype=dX.dtype, device=device)
        assert lib.ga_segment_mm_gather(g.etype_pointer.data_ptr(), n_rel, dXe.data_ptr(), None,
                                        dW.data_ptr(), Y.data_ptr(), None, None, None, None, None,
                                        e, heads, K, M, dt, stream) == 0
        assert_close(Y.float().cpu().numpy(), oracle.segment_mm(tp, Xe, W, heads=heads), tol,
                     "segment_mm_gather identity")
    # argument errors: neither result; both results; scale without a dot operand
    args = (g.etype_pointer.data_ptr(), n_rel, dX.data_ptr(), None, dW.data_ptr())
    tail = (e, heads, K, M, dt, stream)
    Y = torch.empty((e, heads * M), dtype=dX.dtype, device=device)
    D = torch.empty((e, heads), dtype=torch.float32, device=device)
    none = (None,) * 6
    assert lib.ga_segment_mm_gather(*args, *none, *tail) == capi.GA_EINVAL
    assert lib.ga_segment_mm_gather(*args, Y.data_ptr(), dQ.data_ptr(), None, None,
                                    D.data_ptr(), None, *tail) == capi.GA_EINVAL
    assert lib.ga_segment_mm_gather(*args, Y.data_ptr(), None, None, D.data_ptr(), None, None,
                                    *tail) == capi.GA_EINVAL
    assert lib.ga_segment_mm_gather(*args, None, dQ.data_ptr(), None, None, D.data_ptr(),
                                    D.data_ptr(), *tail) == capi.GA_EINVAL      # row factor without Y


def test_segment_mm_dot_factor_of_another_shape(device):
    """A per-type factor that is not one value per head (here (T, 3) against a
    one-head dot) multiplies the result the way the unfused plan's
    ``* BroadcastEdgeType(p)`` would: by broadcasting, after the kernel."""
    rng = np.random.default_rng(9)
    etype = np.repeat(np.arange(4), [30, 0, 50, 21]).astype(np.int64)
    e, n = etype.shape[0], 40
    src, dst = rng.integers(0, n, e, dtype=np.int64), rng.integers(0, n, e, dtype=np.int64)
    g = prepare_graph(src, dst, n, device=device, etype_of=etype, num_etypes=4)
    X = rng.standard_normal((n, 16), dtype=np.float32)
    Q = rng.standard_normal((n, 32), dtype=np.float32)
    W = rng.standard_normal((4, 16, 32)).astype(np.float32) / 4
    p = rng.uniform(0.5, 2.0, (4, 3)).astype(np.float32)
    want = np.einsum("em,em->e", np.einsum("ek,ekm->em", X[src].astype(np.float64), W[etype]),
                     Q[dst].astype(np.float64))[:, None] * p[etype]
    got = ops.SegmentMMEdgeDot(_dev(X, device), _dev(W, device), 0, _dev(Q, device), 1, g,
                               scale=_dev(p, device))
    assert got.shape == (e, 3)
    assert_close(got.cpu().numpy(), want, TOL_F32, "dot with a (T, 3) factor")


@pytest.mark.parametrize("heads,dim,bf16", [(1, 64, False), (8, 16, True), (4, 5, False),
                                            (2, 24, True), (1, 1, False)])
def test_edge_softmax_sum(device, heads, dim, bf16):
    """softmax over the in-edges of per-edge logits times per-edge rows, summed:
    expected = the oracle's segment softmax, a numpy product and the oracle's
    copy_e sum.  Edge ids are shuffled against the adjacency order, one node
    owns a third of the edges and half the nodes have none."""
    rng = np.random.default_rng(heads * 100 + dim)
    src, dst = skewed_graph(rng, 600, 9000, 4000)
    n, e = 600, src.shape[0]
    g = prepare_graph(src, dst, n, device=device)
    arr = build_graph_arrays(src, dst, n)
    logit = (rng.standard_normal((e, heads)) * 3).astype(np.float32)
    m = rng.standard_normal((e, heads * dim), dtype=np.float32)
    if bf16:
        m = to_bf16_f32(m)
    att = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, logit)
    prod = (m.reshape(e, heads, dim).astype(np.float64) * att[:, :, None]).reshape(e, -1)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      prod.astype(np.float32), op="copy_e")
    got = ops.edge_softmax_sum(_dev(logit, device), _dev(m, device, bf16), g)
    assert got.shape == (n, heads * dim)
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 f"edge_softmax_sum H={heads} D={dim}")
    assert not got[n // 2:].float().abs().sum().item()         # rows without edges: 0
    # edge ids already in adjacency order (no edge-id column passed)
    s2, d2 = datasets.sort_by_dst(src, dst)
    g2 = prepare_graph(s2, d2, n, device=device)
    assert g2.in_eid_is_identity
    order = np.argsort(dst, kind="stable")
    got2 = ops.edge_softmax_sum(_dev(logit[order], device), _dev(m[order], device, bf16), g2)
    assert_close(got2.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 "edge_softmax_sum identity order")


@pytest.mark.parametrize("heads,dim", [(1, 64), (4, 8)])
def test_edge_reductions_on_every_graph(graph, device, heads, dim):
    """edge_softmax_sum and e_mul_e on the debug graph, the graph without edges,
    the single busy row, the skewed and the R-MAT graphs."""
    name, g, arr = graph
    e, n = int(arr.in_node_indices.shape[0]), arr.num_nodes
    rng = np.random.default_rng(5)
    logit = (rng.standard_normal((e, heads)) * 2).astype(np.float32)
    m = rng.standard_normal((e, heads * dim), dtype=np.float32)
    got = ops.edge_softmax_sum(_dev(logit, device), _dev(m, device), g)
    att = oracle.segment_softmax(arr.in_pointer, arr.in_edge_indices, logit)
    prod = (m.reshape(e, heads, dim).astype(np.float64) * att[:, :, None]).reshape(e, heads * dim)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      prod.astype(np.float32), op="copy_e")
    assert got.shape == (n, heads * dim)
    assert_close(got.cpu().numpy(), ref, TOL_F32, f"edge_softmax_sum on {name}")
    w = rng.uniform(0.1, 1.0, (e, 1)).astype(np.float32)
    got = ops.gspmm_e_mul_e_sum(_dev(m, device), _dev(w, device), g)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      (m * w).astype(np.float32), op="copy_e")
    assert_close(got.cpu().numpy(), ref, TOL_F32, f"e_mul_e on {name}")


def test_fused_typed_products_without_rows(device):
    """Zero edges / zero rows: the entry points return GA_OK and touch nothing."""
    g = prepare_graph(np.zeros(0, np.int64), np.zeros(0, np.int64), 9, device=device,
                      etype_of=np.zeros(0, np.int64), num_etypes=3)
    x = torch.randn(9, 16, device=device)
    w = torch.randn(3, 16, 32, device=device)
    assert ops.SegmentMMEdgeGather(x, w, 0, g).shape == (0, 32)
    assert ops.SegmentMMEdgeDot(x, w, 0, torch.randn(9, 32, device=device), 1, g).shape == (0, 1)
    z, el, er = ops.linear_attn(torch.zeros(0, 16, device=device, dtype=torch.bfloat16),
                                torch.zeros(16, 32, device=device, dtype=torch.bfloat16),
                                torch.zeros(1, 32, device=device), torch.zeros(1, 32, device=device))
    assert z.shape == (0, 32) and el.shape == (0, 1) and er.shape == (0, 1)


def test_e_mul_e_sum(device):
    """out[v] = sum over in-edges of m[e] * a[e]: SpMMEdge of the product without
    forming it; edge ids shuffled against the adjacency order."""
    rng = np.random.default_rng(77)
    src, dst = skewed_graph(rng, 400, 6000, 1500)
    n, e = 400, src.shape[0]
    g = prepare_graph(src, dst, n, device=device)
    arr = build_graph_arrays(src, dst, n)
    m = rng.standard_normal((e, 64), dtype=np.float32)
    a = rng.uniform(0.1, 1.0, (e, 1)).astype(np.float32)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      (m * a).astype(np.float32), op="copy_e")
    for x, y in ((m, a), (a, m)):
        got = ops.gspmm_e_mul_e_sum(_dev(x, device), _dev(y, device), g)
        assert_close(got.cpu().numpy(), ref, TOL_F32, "e_mul_e")
    # per-head weights on shaped operands, bf16 messages
    mh = to_bf16_f32(rng.standard_normal((e, 4, 16), dtype=np.float32))
    ah = rng.uniform(0.1, 1.0, (e, 4, 1)).astype(np.float32)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      (mh * ah).reshape(e, 64).astype(np.float32), op="copy_e")
    got = ops.gspmm_e_mul_e_sum(_dev(mh, device, True), _dev(ah, device), g)
    assert got.shape == (n, 4, 16)
    assert_close(got.float().cpu().numpy().reshape(n, 64), ref, TOL_BF16, "e_mul_e heads bf16")
    # two full-width operands: product first
    m2 = rng.standard_normal((e, 64), dtype=np.float32)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices,
                      (m * m2).astype(np.float32), op="copy_e")
    got = ops.gspmm_e_mul_e_sum(_dev(m, device), _dev(m2, device), g)
    assert_close(got.cpu().numpy(), ref, TOL_F32, "e_mul_e full width")


@pytest.mark.parametrize("rows,K,M,heads", [(1000, 602, 64, 1), (333, 77, 64, 2),
                                            (777, 64, 64, 4),
                                            (300, 100, 256, 4), (5000, 16, 32, 2),
                                            (50, 8, 16, 1), (1, 4, 64, 1),
                                            (70001, 40, 64, 2), (200000, 33, 32, 1),
                                            # K % 4 == 2: rows start 0 or 8 bytes past a
                                            # 16-byte boundary, alternately (8-byte vectors)
                                            (257, 6, 16, 1), (300, 34, 64, 2),
                                            (513, 98, 64, 4), (131, 30, 32, 1)])
def test_linear_attn(device, rows, K, M, heads):
    rng = np.random.default_rng(K + M)
    x = rng.standard_normal((rows, K), dtype=np.float32)
    w = datasets.glorot(rng, (K, M))
    a = rng.standard_normal((2, heads, M // heads), dtype=np.float32)
    z, el, er = ops.linear_attn(_dev(x, device), _dev(w, device), _dev(a[0], device),
                                _dev(a[1], device))
    zr = x.astype(np.float64) @ w.astype(np.float64)
    assert_close(z.cpu().numpy(), zr, TOL_F32, "linear z")
    zh = zr.reshape(rows, heads, -1)
    assert_close(el.cpu().numpy(), (zh * a[0]).sum(-1), TOL_F32, "linear el")
    assert_close(er.cpu().numpy(), (zh * a[1]).sum(-1), TOL_F32, "linear er")
    z2 = ops.linear_attn(_dev(x, device), _dev(w, device))
    assert np.array_equal(z2.cpu().numpy(), z.cpu().numpy())


@pytest.mark.parametrize("rows,K,M", [(20000, 50, 64), (16384, 128, 41), (40000, 602, 16),
                                      (1000, 50, 64), (20000, 50, 128)])
def test_linear_dispatch(device, rows, K, M):
    """ops.linear: own kernel at tall-and-narrow fp32 shapes, the vendor GEMM
    elsewhere; the same product either way."""
    rng = np.random.default_rng(rows + K + M)
    x = rng.standard_normal((rows, K), dtype=np.float32)
    w = datasets.glorot(rng, (K, M))
    got = ops.linear(_dev(x, device), _dev(w, device))
    assert_close(got.cpu().numpy(), x.astype(np.float64) @ w.astype(np.float64), TOL_F32, "linear")
    own = rows >= ops.LINEAR_MIN_ROWS and M <= ops.LINEAR_MAX_COLS
    same = np.array_equal(got.cpu().numpy(), ops.linear_attn(_dev(x, device), _dev(w, device)).cpu().numpy())
    assert same or not own


@pytest.mark.parametrize("rows,K,M", [(20000, 50, 64), (16500, 500, 16), (17000, 37, 3),
                                      (1000, 50, 64), (20000, 50, 128)])
def test_linear_with_row_factor(device, rows, K, M):
    """The factor per row in the projection's store is the product rounded to fp32 and
    then multiplied: bit for bit ``linear(x, w) * s``, on the kernel's shapes and on the
    vendor GEMM's."""
    rng = np.random.default_rng(rows + K + M)
    x = _dev(rng.standard_normal((rows, K), dtype=np.float32), device)
    w = _dev(datasets.glorot(rng, (K, M)), device)
    s = _dev(rng.uniform(0.1, 2.0, (rows, 1)).astype(np.float32), device)
    s[5] = float("nan")
    want = ops.linear(x, w) * s
    for sc in (s, s.view(-1)):
        got = ops.linear(x, w, row_scale=sc)
        assert got.shape == (rows, M)
        assert torch.equal(torch.nan_to_num(got, nan=7.0), torch.nan_to_num(want, nan=7.0))
    assert torch.isnan(got[5]).all()
    with pytest.raises(RuntimeError, match="row_scale"):
        ops.linear(x, w, row_scale=s[:-1])
    with pytest.raises(RuntimeError, match="row_scale"):
        ops.linear(x, w, row_scale=s.double())


@pytest.mark.parametrize("rows,K,M", [(19717, 500, 16), (16385, 1433, 16), (16400, 128, 3), (20001, 131, 7),
                                      (17000, 130, 1), (30000, 4096, 16), (16384, 127, 16), (33000, 500, 16)])
def test_plain_projection_onto_few_columns(device, rows, K, M):
    """At most 16 columns: the build that multiplies and stores one column block.  Against
    float64, with and without the row factor, row counts that are no multiple of a tile."""
    rng = np.random.default_rng(rows + K + M)
    x = rng.standard_normal((rows, K), dtype=np.float32)
    w = datasets.glorot(rng, (K, M))
    sc = rng.uniform(0.5, 1.5, (rows, 1)).astype(np.float32)
    ref = x.astype(np.float64) @ w.astype(np.float64)
    xd, wd, sd = _dev(x, device), _dev(w, device), _dev(sc, device)
    got = ops.linear_attn(xd, wd)
    assert got.shape == (rows, M)
    assert_close(got.cpu().numpy(), ref, TOL_F32, f"projection {rows}x{K}x{M}")
    assert torch.equal(ops.linear(xd, wd, row_scale=sd), got * sd)
    assert torch.equal(ops.linear_attn(xd, wd), got)          # the same bits every time


@pytest.mark.parametrize("offset", [1, 2, 3, 4])
@pytest.mark.parametrize("K", [66, 602, 64, 37])
def test_linear_attn_row_alignment(device, K, offset):
    """The feature matrix at every 4-byte offset from a 16-byte boundary (a view
    into a larger buffer): each offset selects another vector width of the row
    loads."""
    rows, M = 300, 64
    rng = np.random.default_rng(K + offset)
    x = rng.standard_normal((rows, K), dtype=np.float32)
    w = datasets.glorot(rng, (K, M))
    a = rng.standard_normal((2, 1, M), dtype=np.float32)
    buf = torch.zeros(rows * K + 8, device=device)
    xd = buf[offset:offset + rows * K].view(rows, K)
    xd.copy_(_dev(x, device))
    assert xd.data_ptr() % 16 == (4 * offset) % 16
    z, el, er = ops.linear_attn(xd, _dev(w, device), _dev(a[0], device), _dev(a[1], device))
    zr = x.astype(np.float64) @ w.astype(np.float64)
    assert_close(z.cpu().numpy(), zr, TOL_F32, "linear z")
    assert_close(el.cpu().numpy(), (zr * a[0]).sum(-1, keepdims=True), TOL_F32, "linear el")
    assert_close(er.cpu().numpy(), (zr * a[1]).sum(-1, keepdims=True), TOL_F32, "linear er")


@pytest.mark.parametrize("rows,K,M,heads,bf16", [
    (3000, 100, 256, 4, True),      # the larger GAT configuration's first layer (K % 8 != 0)
    (1500, 256, 256, 4, True),      # ... and its hidden layers
    (777, 64, 128, 8, True),        # heads of width 16: two per column-block pair
    (500, 32, 96, 3, True), (129, 8, 32, 1, True), (1, 16, 64, 2, True),
    (1000, 100, 128, 1, False),     # fp32 head of width 128: tile kernel, not linear.hip
    (640, 128, 256, 2, False)])
def test_project_attn_tile_kernel(device, rows, K, M, heads, bf16):
    """Projection + attention terms through the typed-linear tile kernel (bf16
    storage, and the fp32 head widths the dedicated fp32 kernel does not take)."""
    rng = np.random.default_rng(K * 3 + M + heads)
    x = rng.standard_normal((rows, K), dtype=np.float32)
    w = datasets.glorot(rng, (K, M))
    a = rng.standard_normal((2, heads, M // heads), dtype=np.float32)
    if bf16:
        x, w = to_bf16_f32(x), to_bf16_f32(w)
    z, el, er = ops.linear_attn(_dev(x, device, bf16), _dev(w, device, bf16),
                                _dev(a[0], device), _dev(a[1], device))
    assert el.dtype == torch.float32 and z.dtype == (torch.bfloat16 if bf16 else torch.float32)
    zr = x.astype(np.float64) @ w.astype(np.float64)
    assert_close(z.float().cpu().numpy(), zr, TOL_BF16 if bf16 else TOL_F32, "project z")
    zh = zr.reshape(rows, heads, -1)
    # el / er come from the fp32 accumulators, not from the rounded z
    assert_close(el.cpu().numpy(), (zh * a[0]).sum(-1), TOL_F32, "project el")
    assert_close(er.cpu().numpy(), (zh * a[1]).sum(-1), TOL_F32, "project er")


def test_linear_attn_unsupported_shapes(device):
    x = torch.ones(8, 8, device=device)          # head width 8
    with pytest.raises(capi.GraphilerError):
        ops.linear_attn(x, torch.ones(8, 16, device=device),
                        torch.ones(2, 8, device=device), torch.ones(2, 8, device=device))


def test_graph_without_nodes(device):
    """Zero nodes and zero edges: every operator returns a tensor with no rows."""
    none = np.zeros(0, np.int64)
    g = prepare_graph(none, none, 0, device=device)
    assert g.num_nodes == 0 and g.num_edges == 0 and g.in_pointer.cpu().tolist() == [0]
    x = torch.zeros(0, 8, device=device)
    e1 = torch.zeros(0, 1, device=device)
    assert ops.SpMMSrc(x, [1], False, None, g).shape == (0, 8)
    assert ops.SpMMEdge(x, [1], False, None, g).shape == (0, 8)
    assert ops.gspmm_src_mul_e_sum(x, e1, [1], False, None, g).shape == (0, 8)
    assert ops.spmm_scaled(x, g, row_scale=e1, activation="relu").shape == (0, 8)
    assert ops.spmm(g, "copy_u", "max", x).shape == (0, 8)
    assert ops.gsddmm_u_add_v_mul_alpha(e1, e1, 1, g).shape == (0, 1)
    assert ops.gsddmm_u_dot_v(x, x, g).shape[0] == 0
    assert ops.SegmentSoftmax(e1, 1, None, g).shape == (0, 1)
    assert ops.BroadcastSrcNode(x, g).shape == (0, 8)
    assert ops.gat_aggregate(e1, e1, x, g, 0.2).shape == (0, 8)
    assert ops.edge_softmax_sum(e1, x, g).shape == (0, 8)
