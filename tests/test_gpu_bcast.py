"""The general forms of the two binary graph operators -- operands whose feature
shapes broadcast (the offset tables of bcast.cc:19-71 consumed on the device) and,
for SDDMM, operands on source nodes, edges or destination nodes in any combination
(selector.h:30-60) -- against plain numpy broadcasting and fancy indexing, which is
what the tables encode.  fp32; sums in float64 on the host, held to 1e-5; single
operations and max / min with their positions bit for bit."""
import numpy as np
import pytest
import torch

from graphiler_amd import ops, prepare_graph
from graphiler_amd.graph import build_graph_arrays
from helpers import TOL_F32, assert_close, random_graph, skewed_graph

pytestmark = pytest.mark.gpu

NP_OPS = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}


@pytest.fixture(scope="module", params=["uniform", "skewed_shuffled_ids"])
def graph(request, device):
    rng = np.random.default_rng(21)
    if request.param == "uniform":
        src, dst = random_graph(rng, 200, 1500)
        n = 200
    else:
        src, dst = skewed_graph(rng, 300, 1200, 2500)     # a hub, nodes without in-edges
        n = 300
    return prepare_graph(src, dst, n, device=device), build_graph_arrays(src, dst, n), src, dst, n


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _aligned(a, b):
    """The two operands with their feature dimensions (all but the first) aligned at
    the right, as the reference's tables align them: numpy would otherwise line the row
    dimension of the operand with fewer dimensions up with a feature dimension."""
    nd = max(a.ndim, b.ndim)
    pad = lambda t: t.reshape((t.shape[0],) + (1,) * (nd - t.ndim) + t.shape[1:])
    return pad(a), pad(b)


SPMM_SHAPES = [((4, 1), (1, 8)), ((3,), (1,)), ((2, 3), (3,)), ((5,), (5,)), ((1, 6), (4, 1)),
               ((2, 1, 3), (4, 1))]


@pytest.mark.parametrize("u_feat,e_feat", SPMM_SHAPES)
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_spmm_broadcast_sum(graph, device, u_feat, e_feat, op):
    g, arr, src, dst, n = graph
    rng = np.random.default_rng(len(u_feat) * 7 + len(op))
    e = src.shape[0]
    u = rng.standard_normal((n,) + u_feat).astype(np.float32)
    w = rng.uniform(0.5, 2.0, (e,) + e_feat).astype(np.float32)
    got = ops.gspmm(g, op, "sum", _dev(u, device), _dev(w, device)).cpu().numpy()
    msg = NP_OPS[op](*_aligned(u[src].astype(np.float64), w.astype(np.float64)))   # numpy broadcasting
    want = np.zeros((n,) + msg.shape[1:])
    np.add.at(want, dst, msg)
    mag = np.zeros_like(want)
    np.add.at(mag, dst, np.abs(msg))
    assert got.shape == want.shape
    assert_close(got, want, TOL_F32, f"gspmm {op} {u_feat} x {e_feat}", mag=mag)


@pytest.mark.parametrize("reduce", ["max", "min"])
def test_spmm_broadcast_extrema_with_positions(graph, device, reduce):
    """Small integers: exact values, many ties; the first extremum in adjacency order
    wins and rows without edges keep -inf / +inf with positions 0."""
    g, arr, src, dst, n = graph
    rng = np.random.default_rng(5)
    e = src.shape[0]
    u = rng.integers(-3, 4, (n, 3, 1)).astype(np.float32)
    w = rng.integers(1, 3, (e, 1, 2)).astype(np.float32)
    out, arg_u, arg_e = ops.gspmm(g, "mul", reduce, _dev(u, device), _dev(w, device), return_arg=True)
    out, arg_u, arg_e = out.cpu().numpy(), arg_u.cpu().numpy(), arg_e.cpu().numpy()
    ptr, nbr, eid = arr.in_pointer, arr.in_node_indices, arr.in_edge_indices
    better = np.greater if reduce == "max" else np.less
    for v in range(n):
        acc = np.full((3, 2), -np.inf if reduce == "max" else np.inf, np.float32)
        au = np.zeros((3, 2), np.int32)
        ae = np.zeros((3, 2), np.int32)
        for i in range(ptr[v], ptr[v + 1]):
            m = u[nbr[i]] * w[eid[i]]
            hit = better(m, acc)
            acc = np.where(hit, m, acc)
            au = np.where(hit, nbr[i], au)
            ae = np.where(hit, eid[i], ae)
        assert np.array_equal(out[v], acc) and np.array_equal(arg_u[v], au) and np.array_equal(arg_e[v], ae), v


def test_spmm_copies_and_out_adjacency(graph, device):
    g, arr, src, dst, n = graph
    rng = np.random.default_rng(6)
    e = src.shape[0]
    w = rng.standard_normal((e, 2, 2)).astype(np.float32)
    got = ops.gspmm(g, "copy_rhs", "sum", None, _dev(w, device)).cpu().numpy()
    want = np.zeros((n, 2, 2))
    np.add.at(want, dst, w.astype(np.float64))
    assert_close(got, want, TOL_F32, "gspmm copy_rhs")
    u = rng.standard_normal((n, 2, 1)).astype(np.float32)
    got = ops.gspmm(g, "mul", "sum", _dev(u, device), _dev(w, device), reverse=True).cpu().numpy()
    want = np.zeros((n, 2, 2))
    np.add.at(want, src, u[dst].astype(np.float64) * w)       # out-adjacency: rows by source
    assert_close(got, want, TOL_F32, "gspmm over the out-adjacency")
    # the shaped call of the tuned wrapper falls through to the general kernel
    got = ops.spmm(g, "u_mul_e", "sum", _dev(u, device).expand(n, 2, 1).contiguous(),
                   _dev(w, device))
    want = np.zeros((n, 2, 2))
    np.add.at(want, dst, u[src].astype(np.float64) * w)
    assert_close(got.cpu().numpy(), want, TOL_F32, "spmm with a general broadcast")


TARGET_ROWS = {"u": lambda s, d, e: s, "e": lambda s, d, e: np.arange(e), "v": lambda s, d, e: d}


@pytest.mark.parametrize("lhs_target,rhs_target", [("u", "v"), ("u", "e"), ("e", "v"), ("v", "u"),
                                                   ("e", "e"), ("u", "u")])
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_sddmm_targets_and_broadcast_bit_exact(graph, device, lhs_target, rhs_target, op):
    g, arr, src, dst, n = graph
    rng = np.random.default_rng(11)
    e = src.shape[0]
    rows = {"u": n, "e": e, "v": n}
    for l_feat, r_feat in (((4,), (4,)), ((3, 1), (1, 5)), ((2, 3), (3,)), ((1,), (6,))):
        lhs = rng.standard_normal((rows[lhs_target],) + l_feat).astype(np.float32)
        rhs = rng.uniform(0.5, 2.0, (rows[rhs_target],) + r_feat).astype(np.float32)
        got = ops.gsddmm(g, op, _dev(lhs, device), _dev(rhs, device), lhs_target, rhs_target)
        want = NP_OPS[op](*_aligned(lhs[TARGET_ROWS[lhs_target](src, dst, e)],
                                    rhs[TARGET_ROWS[rhs_target](src, dst, e)]))
        assert got.shape == want.shape
        assert np.array_equal(got.cpu().numpy(), want), (op, lhs_target, rhs_target, l_feat, r_feat)


@pytest.mark.parametrize("lhs_target,rhs_target", [("u", "v"), ("e", "v"), ("u", "e")])
def test_sddmm_dot_general(graph, device, lhs_target, rhs_target):
    g, arr, src, dst, n = graph
    rng = np.random.default_rng(12)
    e = src.shape[0]
    rows = {"u": n, "e": e, "v": n}
    for l_feat, r_feat in (((4, 8), (4, 8)), ((4, 8), (1, 8)), ((16,), (16,)), ((2, 1, 5), (3, 5))):
        lhs = rng.standard_normal((rows[lhs_target],) + l_feat).astype(np.float32)
        rhs = rng.standard_normal((rows[rhs_target],) + r_feat).astype(np.float32)
        got = ops.gsddmm(g, "dot", _dev(lhs, device), _dev(rhs, device), lhs_target, rhs_target)
        a, b = _aligned(lhs[TARGET_ROWS[lhs_target](src, dst, e)].astype(np.float64),
                        rhs[TARGET_ROWS[rhs_target](src, dst, e)].astype(np.float64))
        want = (a * b).sum(-1)
        mag = (np.abs(a) * np.abs(b)).sum(-1)
        if want.ndim == 1:
            want, mag = want[:, None], mag[:, None]
        assert got.shape == want.shape, (got.shape, want.shape)
        assert_close(got.cpu().numpy(), want, TOL_F32, f"dot {l_feat} . {r_feat}", mag=mag)


def test_general_forms_reject_bad_arguments(graph, device):
    g, arr, src, dst, n = graph
    x = torch.zeros(n, 3, device=device)
    with pytest.raises(RuntimeError, match="number of rows"):
        ops.gsddmm(g, "add", x, x, "e", "v")
    with pytest.raises(RuntimeError, match="targets"):
        ops.gsddmm(g, "add", x, x, "u", "w")
    with pytest.raises(RuntimeError, match="float32"):
        ops.gsddmm(g, "add", x.bfloat16(), x, "u", "v")
    with pytest.raises(ValueError):
        ops.gspmm(g, "mul", "sum", torch.zeros(n, 3, device=device),
                  torch.zeros(g.num_edges, 4, device=device))        # shapes do not broadcast
