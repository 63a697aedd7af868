"""Operator wrappers: the reference's ``torch.ops.my_ops.*`` surface over the C ABI.

Every function keeps the name, argument order and argument meaning of the
operator it replaces (schemas in src/ops/dgl_primitives/spmm.cu:391-406,
sddmm.cu:131-134, segment_softmax/segment_softmax.cu:27-30,
segment_mm/segment_mm.cu:35-42, broadcast/broadcast.cu:102-122).  The unused
``dim / keep_dim / dtype`` arguments exist in the reference because its builder
relabels an ``aten::sum`` / ``aten::softmax`` node (src/builder/builder.cpp:141-143);
they are accepted and ignored here too, except ``dim == 1`` for the softmax.

The wrappers own allocation and argument checking (CUDA + contiguous, raising
``RuntimeError`` like the reference's CHECK_INPUT, src/ops/ops.cuh:14-20) and
hand raw device pointers plus the current HIP stream to the library.  There is
no CPU path: tensors that are not on the GPU are rejected.
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np
import torch

from . import capi
from .bcast import calc_bcast_off
from .graph import DGLGraph

_DTYPES = {torch.float32: capi.GA_F32, torch.bfloat16: capi.GA_BF16}
_REDUCE = {"sum": capi.GA_SUM, "max": capi.GA_MAX, "min": capi.GA_MIN}


def _check_input(x: torch.Tensor, name: str) -> None:
    if not x.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not x.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _feat_dtype(x: torch.Tensor, name: str) -> int:
    if x.dtype not in _DTYPES:
        raise RuntimeError(f"{name} must be float32 or bfloat16")
    return _DTYPES[x.dtype]


def _stream(x: torch.Tensor) -> int:
    return torch.cuda.current_stream(x.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def get_feat_dim(features: torch.Tensor) -> int:
    """broadcast.cu:3-9: product of the sizes of all dimensions after the first."""
    d = 1
    for s in features.shape[1:]:
        d *= int(s)
    return d


def _out_shape(rows: int, x: torch.Tensor):
    return (rows,) + (tuple(x.shape[1:]) if x.dim() > 1 else (1,))


# ----------------------------------------------------------------- SpMM ----
def spmm(g: DGLGraph, op: str, reduce: str, u: torch.Tensor,
         w: Optional[torch.Tensor] = None, reverse: bool = False,
         return_arg: bool = False):
    """Generalised SpMM over the in-adjacency (``reverse``: the out-adjacency).

    op: "copy_u" (u is (N, ...)), "copy_e" (u is (E, ...)), "u_mul_e" /
    "u_add_e" / "u_sub_e" / "u_div_e" (functor.cuh:19-72; w is (E,), (E, 1) or
    (E, H) fp32), "e_mul_e" (u is (E, ...) in edge-id order, times w: the rows
    are read through the edge-id column in place of the neighbour column).
    reduce: "sum" | "max" | "min".
    ``return_arg`` (max / min only): also return ``(arg_u, arg_e)``, the int32
    neighbour id and edge id that supplied each output element (spmm.cuh:30-71);
    the one the operator has no use for is None.
    """
    _check_input(u, "features")
    dt = _feat_dtype(u, "features")
    if reverse:
        pointer, nbr, eid = g.out_pointer, g.out_node_indices, g.out_edge_indices
        rows, ident = g.out_row_of_slot, g.out_eid_is_identity
    else:
        pointer, nbr, eid = g.in_pointer, g.in_node_indices, g.in_edge_indices
        rows, ident = g.in_row_of_slot, g.in_eid_is_identity
    feat = get_feat_dim(u)
    heads = 1
    edge_rows = op in ("copy_e", "e_mul_e")
    if op == "e_mul_e":
        nbr = eid            # "neighbour" row of a slot = its edge id
    code = {"copy_u": capi.GA_COPY_U, "copy_e": capi.GA_COPY_E,
            "e_mul_e": capi.GA_U_MUL_E,
            "u_mul_e": capi.GA_U_MUL_E, "u_add_e": capi.GA_U_ADD_E,
            "u_sub_e": capi.GA_U_SUB_E, "u_div_e": capi.GA_U_DIV_E}[op]
    if code >= capi.GA_U_MUL_E:
        _check_input(w, "edge weights")
        if w.dtype != torch.float32:
            raise RuntimeError("edge weights must be float32")
        if w.shape[0] != g.num_edges:
            raise RuntimeError("edge weights must have one row per edge")
        heads = get_feat_dim(w)
        shaped = w.dim() == u.dim() and u.dim() >= 3
        if feat % heads and not shaped:
            raise RuntimeError("feature width is not a multiple of the heads")
        if shaped:
            # shaped operands, e.g. (N, H, D) * (E, H, 1): the row-reduction kernels
            # take exactly the broadcasts that are "one weight per head" (tables of
            # bcast.cc:19-71); any other shape pair goes to the general kernel
            b = calc_bcast_off("mul", tuple(u.shape), tuple(w.shape))
            per_head = np.arange(feat, dtype=np.int64) // max(feat // heads, 1)
            if feat % heads or b.out_len != feat \
                    or not np.array_equal(b.lhs_offset, np.arange(feat)) \
                    or not np.array_equal(b.rhs_offset, per_head):
                return gspmm(g, {"u_mul_e": "mul", "e_mul_e": "mul", "u_add_e": "add",
                                 "u_sub_e": "sub", "u_div_e": "div"}[op], reduce, u, w,
                             reverse=reverse, return_arg=return_arg, edge_rows=edge_rows)
    n_src = g.num_edges if edge_rows else g.num_nodes
    if u.shape[0] != n_src:
        raise RuntimeError("features have the wrong number of rows")
    out = torch.empty(_out_shape(g.num_nodes, u), dtype=u.dtype, device=u.device)
    lib = capi.load()
    if return_arg:
        if reduce not in ("max", "min"):
            raise RuntimeError("return_arg needs the max or the min reducer")
        arg_u = arg_e = None
        if op != "copy_e":
            arg_u = torch.empty(out.shape, dtype=torch.int32, device=u.device)
        if op != "copy_u":
            arg_e = torch.empty(out.shape, dtype=torch.int32, device=u.device)
        ws = g.workspace(lib.ga_spmm_arg_workspace_bytes(g.num_edges, feat))
        capi.check(lib.ga_spmm_csr_arg(
            pointer.data_ptr(), rows.data_ptr(), nbr.data_ptr(),
            None if ident else eid.data_ptr(), u.data_ptr(), _ptr(w),
            out.data_ptr(), _ptr(arg_u), _ptr(arg_e), g.num_nodes, g.num_edges,
            feat, heads, code, _REDUCE[reduce], dt, ws.data_ptr(), ws.numel(),
            _stream(u)), "ga_spmm_csr_arg")
        return out, arg_u, arg_e
    ws_bytes = lib.ga_spmm_workspace_bytes(g.num_edges, feat)
    ws = g.workspace(ws_bytes)
    capi.check(lib.ga_spmm_csr(
        pointer.data_ptr(), rows.data_ptr(), nbr.data_ptr(),
        None if ident else eid.data_ptr(), u.data_ptr(), _ptr(w),
        out.data_ptr(), g.num_nodes, g.num_edges, feat, heads, code,
        _REDUCE[reduce], dt, ws.data_ptr(), ws.numel(), _stream(u)),
        "ga_spmm_csr")
    return out


def SpMMSrc(features, dims: Sequence[int], keep_dim: bool, dtype,
            graph: DGLGraph) -> torch.Tensor:
    """spmm.cu:375-389: out[v] = sum over in-edges of features[src]."""
    return spmm(graph, "copy_u", "sum", features)


def SpMMEdge(features, dims: Sequence[int], keep_dim: bool, dtype,
             graph: DGLGraph) -> torch.Tensor:
    """spmm.cu:359-373: out[v] = sum over in-edges of features[edge id]."""
    return spmm(graph, "copy_e", "sum", features)


# A row factor / activation in the sum's store is free on the lanes-per-slot kernel (rows
# of up to four features; five to seven features on graphs of up to 300,000 edges, the
# library's own rule) and cheap for rows that 16-byte accesses tile.  For the other
# widths (the one-feature-per-lane layout of the run schedule) it pays from a result of
# SPMM_TAIL_MIN_BYTES on: measured on 19,717 nodes, the 9-wide sum with the tail takes
# 24 us against 16 us without and 24 us with two elementwise kernels after it; from
# 232,965 nodes on the tail in the store wins for every width (4-8 % of the sum).
SPMM_TAIL_MIN_BYTES = 8 << 20
SPMM_SLOTS_MAX_EDGES_5_TO_7 = 300_000


def spmm_tail_preferred(features, graph: DGLGraph) -> bool:
    """Whether ``spmm_scaled`` beats the sum followed by elementwise operators."""
    feat = get_feat_dim(features)
    row_bytes = feat * features.element_size()
    on_slots = feat <= 4 or (feat <= 7 and graph.num_edges <= SPMM_SLOTS_MAX_EDGES_5_TO_7)
    return on_slots or row_bytes % 16 == 0 or graph.num_nodes * row_bytes >= SPMM_TAIL_MIN_BYTES


def spmm_scaled(features, graph: DGLGraph, row_scale=None, activation=None,
                edge_rows: bool = False) -> torch.Tensor:
    """SpMMSrc (``edge_rows``: SpMMEdge) with the row-wise tail of a layer applied
    where the sums are stored: out[v] = act(row_scale[v] * sum over in-edges), the
    reduce of examples/GCN/GCN.py:26 (``torch.relu(torch.sum(mailbox, 1))``) with
    an optional destination-side norm.  row_scale: (N,) or (N, 1) fp32 or None;
    activation: None | "relu" | "elu".  Bit for bit what the separate operators
    give (sum, multiplication in fp32, activation, one rounding to the storage type)."""
    _check_input(features, "features")
    dt = _feat_dtype(features, "features")
    act = _activation(activation)
    n = graph.num_nodes
    if features.shape[0] != (graph.num_edges if edge_rows else n):
        raise RuntimeError("features have the wrong number of rows")
    if row_scale is not None:
        _check_input(row_scale, "row_scale")
        if row_scale.dtype != torch.float32 or row_scale.numel() != n \
                or row_scale.shape[0] != n:
            raise RuntimeError("row_scale must be (N,) or (N, 1) float32")
    feat = get_feat_dim(features)
    out = torch.empty(_out_shape(n, features), dtype=features.dtype, device=features.device)
    lib = capi.load()
    ws = graph.workspace(lib.ga_spmm_scaled_workspace_bytes(graph.num_edges, feat))
    capi.check(lib.ga_spmm_csr_scaled(
        graph.in_pointer.data_ptr(), graph.in_row_of_slot.data_ptr(),
        graph.in_node_indices.data_ptr(),
        None if graph.in_eid_is_identity else graph.in_edge_indices.data_ptr(),
        features.data_ptr(), out.data_ptr(), _ptr(row_scale), act, n, graph.num_edges, feat,
        capi.GA_COPY_E if edge_rows else capi.GA_COPY_U, dt, ws.data_ptr(), ws.numel(),
        _stream(features)), "ga_spmm_csr_scaled")
    return out


def gspmm_src_mul_e_sum(ufeature, efeature, dims: Sequence[int], keep_dim: bool,
                        dtype, graph: DGLGraph) -> torch.Tensor:
    """spmm.cu:286-320: out[v] = sum over in-edges of ufeature[src] * efeature[e]."""
    return spmm(graph, "u_mul_e", "sum", ufeature, efeature)


def gspmm_dst_mul_e_sum(ufeature, efeature, dims: Sequence[int], keep_dim: bool,
                        dtype, graph: DGLGraph) -> torch.Tensor:
    """spmm.cu:322-356: the same contraction over the out-adjacency:
    out[v] = sum over out-edges of ufeature[dst] * efeature[e]."""
    return spmm(graph, "u_mul_e", "sum", ufeature, efeature, reverse=True)


def gspmm_e_mul_e_sum(x, y, graph: DGLGraph) -> torch.Tensor:
    """out[v] = sum over in-edges e of x[e] * y[e] for two per-edge operands,
    the ``SpMMEdge(x * y)`` of the reference's plans (reduce of
    examples/HGT/HGT.py:50-53, message of examples/RGCN/RGCN.py:29) without the
    product tensor.  One operand must be a per-edge (or per-head) fp32 weight;
    two full-width operands are multiplied first and summed with copy_e."""
    for a, b in ((x, y), (y, x)):
        if b.dtype != torch.float32 or a.dim() < 2 or a.shape[0] != b.shape[0]:
            continue
        scalar = b.dim() <= 2 and get_feat_dim(b) == 1                  # (E,) / (E, 1)
        per_head = (b.dim() == a.dim() >= 3 and b.shape[-1] == 1
                    and b.shape[:-1] == a.shape[:-1])                   # (E, H, 1)
        if scalar or per_head:
            return spmm(graph, "e_mul_e", "sum", a, b)
    return spmm(graph, "copy_e", "sum", (x * y).contiguous())


# ---------------------------------------------------------------- SDDMM ----
def _edge_columns(g: DGLGraph):
    """(lhs, rhs, bits) giving source and destination of every edge in edge-id
    order: the int32 in-adjacency columns when edge ids are slot numbers (half
    the index traffic), the int64 COO columns otherwise."""
    if g.in_eid_is_identity:
        return g.in_node_indices, g.in_row_of_slot, 32
    return g.COO_src, g.COO_dst, 64


# Operand widths (fp32 values per node) at which the SDDMM that walks the adjacency
# beats the two-column kernel on an MI355X: with one value per node both are bound by
# the rate of the 4-byte gathers of the source term (about two cycles per gather and
# compute unit: 44 us against 61 us for 11.6 M edges); from two values on the walk
# wins (4 values, 64.3 M edges: 0.78 against 0.90 ms).
_ADJ_SDDMM_WIDTHS = (2, 4)


def gsddmm_u_add_v_mul_alpha(src_feature, dst_feature, alpha: int,
                             graph: DGLGraph) -> torch.Tensor:
    """sddmm.cu:118-129: out[e] = src_feature[src[e]] + dst_feature[dst[e]]
    in edge-id order, fp32 (E, feat).  ``alpha`` is ignored, as in the reference."""
    return gsddmm_u_op_v("add", src_feature, dst_feature, graph)


def gsddmm_u_op_v(op: str, src_feature, dst_feature, graph: DGLGraph) -> torch.Tensor:
    """Generic SDDMM of the reference (sddmm.cuh:34-71 with the add / sub / mul /
    div functors, functor.cuh:19-72): out[e] = src_feature[src[e]] (op)
    dst_feature[dst[e]] in edge-id order, fp32 (E, feat).  fp32 operands of width
    2 or 4 on a graph whose edge ids are in-adjacency slots walk the adjacency
    (rows from the row pointer: one index column read instead of two)."""
    code = {"add": capi.GA_SDDMM_ADD, "sub": capi.GA_SDDMM_SUB, "mul": capi.GA_SDDMM_MUL,
            "div": capi.GA_SDDMM_DIV}[op]
    if (src_feature.dtype == torch.float32 and dst_feature.dtype == torch.float32
            and src_feature.is_cuda and dst_feature.is_cuda
            and src_feature.is_contiguous() and dst_feature.is_contiguous()
            and get_feat_dim(src_feature) == get_feat_dim(dst_feature)
            and get_feat_dim(src_feature) in _ADJ_SDDMM_WIDTHS and graph.num_edges > 0
            and graph.in_eid_is_identity):
        feat = get_feat_dim(src_feature)
        out = torch.empty(_out_shape(graph.num_edges, src_feature),
                          dtype=torch.float32, device=src_feature.device)
        rc = capi.load().ga_sddmm_u_op_v_adj(
            graph.in_pointer.data_ptr(), graph.in_row_of_slot.data_ptr(),
            graph.in_node_indices.data_ptr(), src_feature.data_ptr(),
            dst_feature.data_ptr(), out.data_ptr(), graph.num_nodes, graph.num_edges,
            feat, code, _stream(out))
        if rc not in (capi.GA_EALIGN, capi.GA_EUNSUPPORTED):   # else: the two-column kernel
            capi.check(rc, "ga_sddmm_u_op_v_adj")
            return out
    _check_input(src_feature, "src_feature")
    _check_input(dst_feature, "dst_feature")
    dt = _feat_dtype(src_feature, "src_feature")
    if dst_feature.dtype != src_feature.dtype:
        raise RuntimeError("src_feature and dst_feature must share a dtype")
    feat = get_feat_dim(src_feature)
    if get_feat_dim(dst_feature) != feat:
        raise RuntimeError("src_feature and dst_feature must share a width")
    out = torch.empty(_out_shape(graph.num_edges, src_feature),
                      dtype=torch.float32, device=src_feature.device)
    lhs, rhs, bits = _edge_columns(graph)
    capi.check(capi.load().ga_sddmm_u_op_v(
        lhs.data_ptr(), rhs.data_ptr(), bits, src_feature.data_ptr(),
        dst_feature.data_ptr(), out.data_ptr(), graph.num_edges, feat, code, dt,
        _stream(out)), "ga_sddmm_u_op_v")
    return out


def gsddmm_u_dot_v(src_feature, dst_feature, graph: DGLGraph) -> torch.Tensor:
    """u_dot_v over the last dimension (functor.cuh:103-116, sddmm.cuh:80-120):
    (N, H, D) x (N, H, D) -> (E, H) fp32; 2-D inputs are one head."""
    _check_input(src_feature, "src_feature")
    _check_input(dst_feature, "dst_feature")
    dt = _feat_dtype(src_feature, "src_feature")
    if dst_feature.dtype != src_feature.dtype or \
            dst_feature.shape[1:] != src_feature.shape[1:]:
        raise RuntimeError("src_feature and dst_feature must share dtype and shape")
    if src_feature.dim() == 2:
        heads, dim = 1, int(src_feature.shape[1])
    elif src_feature.dim() == 3:
        heads, dim = int(src_feature.shape[1]), int(src_feature.shape[2])
    else:
        raise RuntimeError("u_dot_v expects (N, D) or (N, H, D) features")
    out = torch.empty((graph.num_edges, heads), dtype=torch.float32,
                      device=src_feature.device)
    lhs, rhs, bits = _edge_columns(graph)
    capi.check(capi.load().ga_sddmm_u_dot_v(
        lhs.data_ptr(), rhs.data_ptr(), bits, src_feature.data_ptr(),
        dst_feature.data_ptr(), out.data_ptr(), graph.num_edges, heads, dim, dt,
        _stream(out)), "ga_sddmm_u_dot_v")
    return out


# ------------------------------------------------- general (broadcasting) forms ----
_BCAST_OPS = {"add": capi.GA_BCAST_ADD, "sub": capi.GA_BCAST_SUB, "mul": capi.GA_BCAST_MUL,
              "div": capi.GA_BCAST_DIV, "copy_lhs": capi.GA_BCAST_COPY_LHS,
              "copy_rhs": capi.GA_BCAST_COPY_RHS, "dot": capi.GA_BCAST_DOT}


def _bcast_shape(lhs_shape, rhs_shape, drop_last: bool):
    """Feature shape of op(lhs, rhs) under numpy broadcasting of the dimensions after
    the first (``drop_last``: the dot product consumes the last one)."""
    ls = tuple(lhs_shape[1:-1] if drop_last else lhs_shape[1:])
    rs = tuple(rhs_shape[1:-1] if drop_last else rhs_shape[1:])
    return tuple(np.broadcast_shapes(ls, rs))


def _offsets(table: np.ndarray, device) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(table, dtype=np.int64)).to(device)


def gspmm(g: DGLGraph, op: str, reduce: str, u: Optional[torch.Tensor],
          e: Optional[torch.Tensor], reverse: bool = False, return_arg: bool = False,
          edge_rows: bool = False):
    """The reference's general SpMM (SpMMCsrKernel with UseBcast, spmm.cuh:30-71):
    out[v] = reduce over the in-edges i of v of ``op(u[src_i], e[edge_i])`` where the
    feature shapes of ``u`` (N, ...) and ``e`` (E, ...) broadcast against each other by
    numpy's rules (offset tables: :func:`graphiler_amd.bcast.calc_bcast_off`, the
    reference's CalcBcastOff, bcast.cc:19-71).  op: add | sub | mul | div | copy_lhs |
    copy_rhs; reduce: sum | max | min; fp32.  ``reverse``: over the out-adjacency.
    ``edge_rows``: ``u`` is per-edge too (read through the edge-id column).
    The general path: one thread per output element, no tuning; shapes the benchmark
    models use (equal shapes, one weight per head) are served by :func:`spmm`."""
    code = _BCAST_OPS[op]
    if op == "dot":
        raise RuntimeError("dot is an SDDMM operator")
    use_u, use_e = op != "copy_rhs", op != "copy_lhs"
    for t, name, used in ((u, "u", use_u), (e, "e", use_e)):
        if used:
            _check_input(t, name)
            if t.dtype != torch.float32:
                raise RuntimeError("the general SpMM is float32 only")
    if reverse:
        pointer, nbr, eid, ident = g.out_pointer, g.out_node_indices, g.out_edge_indices, \
            g.out_eid_is_identity
    else:
        pointer, nbr, eid, ident = g.in_pointer, g.in_node_indices, g.in_edge_indices, \
            g.in_eid_is_identity
    if edge_rows:
        nbr = eid
    if use_u and u.shape[0] != (g.num_edges if edge_rows else g.num_nodes):
        raise RuntimeError("u has the wrong number of rows")
    if use_e and e.shape[0] != g.num_edges:
        raise RuntimeError("e must have one row per edge")
    ref = u if use_u else e
    lhs_shape = tuple(u.shape) if use_u else (1,) + tuple(e.shape[1:])
    rhs_shape = tuple(e.shape) if use_e else (1,) + tuple(u.shape[1:])
    b = calc_bcast_off(op, lhs_shape, rhs_shape)
    feat_shape = _bcast_shape(lhs_shape, rhs_shape, False) if b.use_bcast else \
        tuple((e if op == "copy_rhs" else u).shape[1:])
    out = torch.empty((g.num_nodes,) + feat_shape, dtype=torch.float32, device=ref.device)
    arg_u = arg_e = None
    if return_arg:
        if reduce not in ("max", "min"):
            raise RuntimeError("return_arg needs the max or the min reducer")
        if use_u:
            arg_u = torch.empty(out.shape, dtype=torch.int32, device=ref.device)
        if use_e:
            arg_e = torch.empty(out.shape, dtype=torch.int32, device=ref.device)
    u_off = _offsets(b.lhs_offset, ref.device) if b.use_bcast else None
    e_off = _offsets(b.rhs_offset, ref.device) if b.use_bcast else None
    capi.check(capi.load().ga_spmm_csr_bcast(
        pointer.data_ptr(), nbr.data_ptr(), None if ident else eid.data_ptr(), _ptr(u), _ptr(e),
        out.data_ptr(), _ptr(arg_u), _ptr(arg_e), g.num_nodes, g.num_edges, _ptr(u_off),
        _ptr(e_off), max(b.lhs_len, 1), max(b.rhs_len, 1), b.out_len, code, _REDUCE[reduce],
        _stream(ref)), "ga_spmm_csr_bcast")
    return (out, arg_u, arg_e) if return_arg else out


_TARGETS = {"u": 0, "e": 1, "v": 2}


def gsddmm(g: DGLGraph, op: str, lhs: torch.Tensor, rhs: torch.Tensor,
           lhs_target: str = "u", rhs_target: str = "v") -> torch.Tensor:
    """The reference's general SDDMM (SDDMMCooKernel / the dot-product kernel,
    sddmm.cuh:34-120): out[e] = ``op(lhs[id_l(e)], rhs[id_r(e)])`` in edge-id order with
    each operand on the source nodes ("u"), on the edges ("e") or on the destination
    nodes ("v") (selector.h:30-60) and feature shapes that broadcast by numpy's rules
    (bcast.cc:19-71); ``dot`` sums the products over the last dimension.  fp32.
    The general path; ``u (op) v`` on equal shapes and ``u_dot_v`` per head are served
    by :func:`gsddmm_u_op_v` / :func:`gsddmm_u_dot_v`."""
    code = _BCAST_OPS[op]
    _check_input(lhs, "lhs")
    _check_input(rhs, "rhs")
    if lhs.dtype != torch.float32 or rhs.dtype != torch.float32:
        raise RuntimeError("the general SDDMM is float32 only")
    for t, target, name in ((lhs, lhs_target, "lhs"), (rhs, rhs_target, "rhs")):
        if target not in _TARGETS:
            raise RuntimeError("targets are 'u' (source), 'e' (edge) or 'v' (destination)")
        if t.shape[0] != (g.num_edges if target == "e" else g.num_nodes):
            raise RuntimeError(f"{name} has the wrong number of rows for target {target!r}")
    if op == "dot" and lhs.shape[-1] != rhs.shape[-1]:
        raise RuntimeError("dot needs operands with the same last dimension")
    b = calc_bcast_off(op, tuple(lhs.shape), tuple(rhs.shape))
    if b.use_bcast:
        feat_shape = _bcast_shape(lhs.shape, rhs.shape, op == "dot")
    else:
        src = rhs if op == "copy_rhs" else lhs
        feat_shape = tuple(src.shape[1:-1] if op == "dot" else src.shape[1:])
    out = torch.empty((g.num_edges,) + (feat_shape or (1,)), dtype=torch.float32, device=lhs.device)
    l_off = _offsets(b.lhs_offset, lhs.device) if b.use_bcast else None
    r_off = _offsets(b.rhs_offset, lhs.device) if b.use_bcast else None
    capi.check(capi.load().ga_sddmm_bcast(
        g.COO_src.data_ptr(), g.COO_dst.data_ptr(), lhs.data_ptr(), rhs.data_ptr(),
        out.data_ptr(), g.num_edges, _TARGETS[lhs_target], _TARGETS[rhs_target], _ptr(l_off),
        _ptr(r_off), max(b.lhs_len, 1), max(b.rhs_len, 1), b.out_len, b.reduce_size, code,
        _stream(out)), "ga_sddmm_bcast")
    return out


# -------------------------------------------------------------- softmax ----
def SegmentSoftmax(features, dim: int, dtype, graph: DGLGraph) -> torch.Tensor:
    """segment_softmax.cu:3-24: softmax of the per-edge logits over each
    destination's in-edges; (E,), (E, 1) or (E, H) fp32."""
    _check_input(features, "features")
    if dim != 1:
        raise RuntimeError("SegmentSoftmax reduces over dim 1 of the mailbox")
    if features.dtype != torch.float32:
        raise RuntimeError("features must be float32")
    if features.shape[0] != graph.num_edges:
        raise RuntimeError("features must have one row per edge")
    heads = get_feat_dim(features)
    ident = graph.in_eid_is_identity
    # every edge id occurs in exactly one segment, so all of y is written
    y = torch.empty_like(features)
    lib = capi.load()
    ws = graph.workspace(lib.ga_softmax_workspace_bytes(graph.num_edges, heads))
    capi.check(lib.ga_segment_softmax(
        graph.in_pointer.data_ptr(), graph.in_row_of_slot.data_ptr(),
        None if ident else graph.in_edge_indices.data_ptr(),
        features.data_ptr(), y.data_ptr(), graph.num_nodes, graph.num_edges,
        heads, ws.data_ptr(), ws.numel(), _stream(y)), "ga_segment_softmax")
    return y


# ----------------------------------------------------------- segment_mm ----
def _segment_mm(features, weights, type_pointer, num_types, rows_expected, row_scale=None):
    _check_input(features, "features")
    _check_input(weights, "weights")
    dt = _feat_dtype(features, "features")
    if weights.dtype != features.dtype:
        raise RuntimeError("features and weights must share a dtype")
    if type_pointer is None:
        raise RuntimeError("the graph has no type pointer for this operator")
    if weights.dim() == 3:
        heads = 1
    elif weights.dim() == 4:
        heads = int(weights.shape[1])
    else:
        raise RuntimeError("weights must be (T, K, M) or (T, H, K, M)")
    K, M = int(weights.shape[-2]), int(weights.shape[-1])
    if int(weights.shape[0]) != num_types:
        raise RuntimeError("weights must have one matrix per type")
    rows = int(features.shape[0])
    if rows != rows_expected or get_feat_dim(features) != heads * K:
        raise RuntimeError("features must be (rows, heads*K)")
    out = torch.empty((rows, heads * M), dtype=features.dtype,
                      device=features.device)
    if row_scale is not None:
        _check_input(row_scale, "row_scale")
        if row_scale.dtype != torch.float32 or row_scale.numel() != rows:
            raise RuntimeError("row_scale must be one float32 per row")
        rc = capi.load().ga_segment_mm_gather(
            type_pointer.data_ptr(), num_types, features.data_ptr(), None,
            weights.data_ptr(), out.data_ptr(), None, None, None, None,
            row_scale.data_ptr(), rows, heads, K, M, dt, _stream(out))
        if rc != capi.GA_EUNSUPPORTED:
            capi.check(rc, "ga_segment_mm_gather")
            return out
    capi.check(capi.load().ga_segment_mm(
        type_pointer.data_ptr(), num_types, features.data_ptr(),
        weights.data_ptr(), out.data_ptr(), rows, heads, K, M, dt,
        _stream(out)), "ga_segment_mm")
    if row_scale is not None:       # a shape outside the kernels that take the factor
        out = (out.float() * row_scale.reshape(-1, 1)).to(out.dtype)
    return out


def SegmentMMNode(features, weights, graph: DGLGraph, row_scale=None) -> torch.Tensor:
    """segment_mm.cu:23-27: per-node-type linear, nodes sorted by type.  ``row_scale``
    (N,) or (N, 1) fp32 multiplies row r of the result, applied to the fp32 sums before
    they are rounded (the ``trans_out * alpha.unsqueeze(1)`` of examples/HGT/HGT.py:58-60)."""
    return _segment_mm(features, weights, graph.ntype_pointer,
                       graph.num_ntypes, graph.num_nodes, row_scale)


def SegmentMMNodeGated(features, weights, gate, graph: DGLGraph, sigmoid: bool = True) -> torch.Tensor:
    """``SegmentMMNode(features, weights) * g(BroadcastNodeType(gate))`` with g the sigmoid
    (or the identity): the output projection of an HGT layer with its per-node-type gate
    (examples/HGT/HGT.py:58-60).  ``gate`` (T,) fp32.  The factor is applied to the fp32 sums
    in the product's kernel where that kernel takes it (bf16, wide outputs); otherwise it is
    formed per row first and goes in as ``row_scale`` of SegmentMMNode."""
    _check_input(features, "features")
    _check_input(weights, "weights")
    _check_input(gate, "gate")
    if graph.ntype_pointer is None:
        raise RuntimeError("the graph has no type pointer for this operator")
    if gate.dtype != torch.float32 or gate.numel() != graph.num_ntypes:
        raise RuntimeError("gate must be one float32 per node type")
    if features.dtype == torch.bfloat16 and weights.dtype == torch.bfloat16 and weights.dim() == 3 \
            and int(weights.shape[0]) == graph.num_ntypes and features.dim() == 2 \
            and int(features.shape[0]) == graph.num_nodes \
            and int(features.shape[1]) == int(weights.shape[1]):
        K, M = int(weights.shape[1]), int(weights.shape[2])
        out = torch.empty((graph.num_nodes, M), dtype=features.dtype, device=features.device)
        rc = capi.load().ga_segment_mm_gated(
            graph.ntype_pointer.data_ptr(), graph.num_ntypes, features.data_ptr(),
            weights.data_ptr(), out.data_ptr(), gate.data_ptr(), 1 if sigmoid else 0,
            graph.num_nodes, K, M, capi.GA_BF16, _stream(out))
        if rc != capi.GA_EUNSUPPORTED:
            capi.check(rc, "ga_segment_mm_gated")
            return out
    factor = torch.sigmoid(gate) if sigmoid else gate
    alpha = BroadcastNodeType(factor.reshape(-1, 1).contiguous(), graph)
    return SegmentMMNode(features, weights, graph, row_scale=alpha)


def SegmentMMNodeStacked(features, weights: Sequence[torch.Tensor], graph: DGLGraph):
    """``[SegmentMMNode(features, w, graph) for w in weights]`` (1 to 4 weight tensors
    of one shape (T, K, M)) with the rows of ``features`` read once: the K, Q and V
    projections of an HGT layer (examples/HGT/HGT.py:35-44).  Returns the list of
    (N, M) results, the same values as separate calls."""
    import ctypes
    if not 1 <= len(weights) <= 4:
        raise RuntimeError("one to four weight tensors")
    _check_input(features, "features")
    dt = _feat_dtype(features, "features")
    if graph.ntype_pointer is None:
        raise RuntimeError("the graph has no type pointer for this operator")
    shape = tuple(weights[0].shape)
    for w in weights:
        _check_input(w, "weights")
        if w.dtype != features.dtype or tuple(w.shape) != shape or w.dim() != 3:
            raise RuntimeError("weights must be (T, K, M) tensors of one shape and the features' dtype")
    K, M = int(shape[1]), int(shape[2])
    if int(shape[0]) != graph.num_ntypes:
        raise RuntimeError("weights must have one matrix per type")
    rows = int(features.shape[0])
    if rows != graph.num_nodes or get_feat_dim(features) != K:
        raise RuntimeError("features must be (rows, K)")
    outs = [torch.empty((rows, M), dtype=features.dtype, device=features.device)
            for _ in weights]
    n = len(weights)
    wp = (ctypes.c_void_p * n)(*[w.data_ptr() for w in weights])
    yp = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    capi.check(capi.load().ga_segment_mm_stacked(
        graph.ntype_pointer.data_ptr(), graph.num_ntypes, features.data_ptr(), wp, yp, n,
        rows, K, M, dt, _stream(features)), "ga_segment_mm_stacked")
    return outs


def SegmentMMEdge(features, weights, graph: DGLGraph) -> torch.Tensor:
    """segment_mm.cu:29-33: per-edge-type linear, edges sorted by type."""
    return _segment_mm(features, weights, graph.etype_pointer,
                       graph.num_etypes, graph.num_edges)


def _endpoint(graph: DGLGraph, which: int) -> torch.Tensor:
    if which not in (0, 1):
        raise RuntimeError("endpoint must be 0 (source) or 1 (destination)")
    return graph.COO_src if which == 0 else graph.COO_dst


def _mm_shapes(features, weights, graph: DGLGraph):
    _check_input(features, "features")
    _check_input(weights, "weights")
    if weights.dtype != features.dtype:
        raise RuntimeError("features and weights must share a dtype")
    if graph.etype_pointer is None:
        raise RuntimeError("the graph has no type pointer for this operator")
    if weights.dim() not in (3, 4):
        raise RuntimeError("weights must be (T, K, M) or (T, H, K, M)")
    heads = 1 if weights.dim() == 3 else int(weights.shape[1])
    K, M = int(weights.shape[-2]), int(weights.shape[-1])
    if int(weights.shape[0]) != graph.num_etypes:
        raise RuntimeError("weights must have one matrix per type")
    if int(features.shape[0]) != graph.num_nodes or get_feat_dim(features) != heads * K:
        raise RuntimeError("features must be (nodes, heads*K)")
    return heads, K, M


def SegmentMMEdgeGather(features, weights, endpoint: int, graph: DGLGraph,
                        row_scale=None) -> torch.Tensor:
    """``SegmentMMEdge(BroadcastSrcNode(features), weights)`` (endpoint 0) or
    the same with ``BroadcastDstNode`` (endpoint 1) as one pass: row e of the
    result is features[endpoint(e)] @ weights[type(e)] (broadcast.cu:58-69 +
    segment_mm.cu:29-33); the (E, heads*K) copy of the node rows is never made.
    ``row_scale`` (E,) or (E, 1) fp32 multiplies row e (RGCN's per-edge norm)."""
    heads, K, M = _mm_shapes(features, weights, graph)
    index = _endpoint(graph, endpoint)
    if row_scale is not None:
        _check_input(row_scale, "row_scale")
        if row_scale.dtype != torch.float32 or row_scale.numel() != graph.num_edges:
            raise RuntimeError("row_scale must be one float32 per edge")
    out = torch.empty((graph.num_edges, heads * M), dtype=features.dtype,
                      device=features.device)
    rc = capi.load().ga_segment_mm_gather(
        graph.etype_pointer.data_ptr(), graph.num_etypes, features.data_ptr(),
        index.data_ptr(), weights.data_ptr(), out.data_ptr(), None, None, None, None,
        _ptr(row_scale), graph.num_edges, heads, K, M, _feat_dtype(features, "features"),
        _stream(out))
    if rc == capi.GA_EUNSUPPORTED:      # shape outside the matrix-core tile
        out = SegmentMMEdge(_gather(features, index), weights, graph)
        if row_scale is not None:
            out = (out * row_scale.reshape(-1, 1)).to(out.dtype)
        return out
    capi.check(rc, "ga_segment_mm_gather")
    return out


def _typed_tiles(graph: DGLGraph):
    """The (destination tile, relation) ordering of the in-edges that TypedSpMMEdge
    walks, and its tile height; built on the device at first use and kept with the
    graph."""
    t = graph._cache.get("typed_tiles")
    if t is None:
        lib = capi.load()
        n, e, r = graph.num_nodes, graph.num_edges, graph.num_etypes
        rows = int(lib.ga_typed_tile_rows(n))
        cap = int(lib.ga_typed_tiles_chunk_capacity(n, e, r, rows))
        tiles = -(-n // rows)
        dev = graph.device
        i32 = dict(dtype=torch.int32, device=dev)
        t = (torch.empty(tiles + 1, **i32), torch.empty(max(cap, 1), **i32),
             torch.empty(max(16 * cap, 1), **i32),
             torch.empty(max(16 * cap, 4), dtype=torch.uint8, device=dev),
             torch.empty(max(16 * cap, 4), **i32), rows)
        nbytes = int(lib.ga_typed_tiles_workspace_bytes(n, e, r, rows))
        if nbytes == 0:
            raise RuntimeError("graph too large for the typed tile layout")
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        ident = graph.in_eid_is_identity
        capi.check(lib.ga_typed_tiles_build(
            graph.in_row_of_slot.data_ptr(), graph.in_node_indices.data_ptr(),
            None if ident else graph.in_edge_indices.data_ptr(),
            graph.etype_pointer.data_ptr(), n, e, r, rows, t[0].data_ptr(), t[1].data_ptr(),
            t[2].data_ptr(), t[3].data_ptr(), t[4].data_ptr(), ws.data_ptr(), ws.numel(),
            torch.cuda.current_stream(dev).cuda_stream), "ga_typed_tiles_build")
        graph._cache["typed_tiles"] = t
    return t


def typed_spmm_supported(features, weights) -> bool:
    """Shapes TypedSpMMEdge takes: 16 / 32 / 48 / 64 input features, 8 / 16 / 32 / 64
    output features."""
    return weights.dim() == 3 and int(weights.shape[2]) in (8, 16, 32, 64) \
        and int(weights.shape[1]) in (16, 32, 48, 64) \
        and get_feat_dim(features) == int(weights.shape[1])


# The one-pass kernel adds the messages of a destination chunk after chunk into one fp32
# accumulator: its rounding error grows with the in-degree (2.5e-6 of the sum at 4,000
# in-edges of one sign, 6.4e-6 at 16,000, 2.2e-5 at 256,000), where the run-wise sums of
# SpMMEdge stay at 3e-7.  Above this in-degree fp32 layers take the operator pair.
TYPED_SPMM_MAX_IN_DEGREE_F32 = 8192


def typed_spmm_preferred(features, weights, graph: Optional[DGLGraph] = None) -> bool:
    """Shapes at which the one-pass kernel beats SegmentMMEdgeGather + SpMMEdge: the
    small products (K * M up to 2048; at 64 x 64 the pair is the faster one) -- and, for
    fp32 on a given graph, only while no node has more than
    ``TYPED_SPMM_MAX_IN_DEGREE_F32`` in-edges (accuracy, see above)."""
    if not typed_spmm_supported(features, weights) \
            or int(weights.shape[1]) * int(weights.shape[2]) > 2048:
        return False
    if graph is not None and features.dtype == torch.float32 \
            and graph.max_in_degree > TYPED_SPMM_MAX_IN_DEGREE_F32:
        return False
    return True


def TypedSpMMEdge(features, weights, graph: DGLGraph, row_scale=None,
                  activation=None) -> torch.Tensor:
    """``SpMMEdge(SegmentMMEdge(BroadcastSrcNode(features), weights) * row_scale)``
    in one pass (examples/RGCN/RGCN.py:25-33; broadcast.cu:58-63, segment_mm.cu:29-33,
    spmm.cu:359-373): out[v] = sum over the in-edges e of v of
    row_scale[e] * features[src(e)] @ weights[type(e)].  No per-edge tensor is written.
    features (N, K), weights (R, K, M) with K in 16, 32, 48, 64 and M in 8, 16, 32, 64;
    ``row_scale`` (E,) or
    (E, 1) fp32.  The additions of a row happen in the order of the prepared layout
    (by relation, then adjacency order), the same in every call.  ``activation``
    ("relu" | "elu"): applied to the fp32 sums before they are stored.
    This is the kernel itself, whatever the graph: a destination's messages go into one
    fp32 accumulator, so the rounding error of its sum grows with its in-degree (relative
    to the sum of magnitudes 3e-7 at 1,000 in-edges, 6e-6 at 16,000, 1.1e-5 at 40,000);
    ``typed_spmm_preferred(features, weights, graph)`` is the rule the layer, the
    TorchScript operator and the compiled plans apply before they take it."""
    _check_input(features, "features")
    _check_input(weights, "weights")
    dt = _feat_dtype(features, "features")
    if weights.dtype != features.dtype:
        raise RuntimeError("features and weights must have one dtype")
    if graph.etype_pointer is None:
        raise RuntimeError("the graph has no edge type pointer")
    if weights.dim() != 3 or int(weights.shape[0]) != graph.num_etypes \
            or get_feat_dim(features) != int(weights.shape[1]):
        raise RuntimeError("weights must be (edge types, K, M) with K the feature width")
    if int(features.shape[0]) != graph.num_nodes:
        raise RuntimeError("features must have one row per node")
    if row_scale is not None:
        _check_input(row_scale, "row_scale")
        if row_scale.dtype != torch.float32 or row_scale.numel() != graph.num_edges:
            raise RuntimeError("row_scale must be one float32 per edge")
    K, M = int(weights.shape[1]), int(weights.shape[2])
    tcp, ctype, ssrc, sdst, sedge, tile_rows = _typed_tiles(graph)
    out = torch.empty((graph.num_nodes, M), dtype=features.dtype, device=features.device)
    capi.check(capi.load().ga_typed_spmm_act(
        tcp.data_ptr(), ctype.data_ptr(), ssrc.data_ptr(), sdst.data_ptr(), sedge.data_ptr(),
        features.data_ptr(), weights.data_ptr(), _ptr(row_scale), out.data_ptr(),
        graph.num_nodes, int(features.shape[0]), graph.num_edges, graph.num_etypes, tile_rows,
        K, M, _activation(activation), dt, _stream(out)), "ga_typed_spmm_act")
    return out


def SegmentMMEdgeDot(features, weights, endpoint: int, other, other_endpoint: int,
                     graph: DGLGraph, scale=None) -> torch.Tensor:
    """out[e, h] = <features[endpoint(e)] @ weights[type(e)], other[other_endpoint(e)]>
    per head, fp32 (E, heads): the ``sum(bmm(k, W) * q, dim=1, keepdim=True)`` of
    examples/HGT/HGT.py:42-45 with neither per-edge operand materialised.
    ``scale`` (T, heads) or (T,) multiplies row e by scale[type(e)] (the
    ``* relation_pri`` of HGT.py:45)."""
    heads, K, M = _mm_shapes(features, weights, graph)
    late = None            # a per-type factor of another shape: broadcast afterwards
    if scale is not None:
        _check_input(scale, "scale")
        if scale.numel() == graph.num_etypes * heads:
            scale = scale.float().contiguous()
        else:
            late, scale = BroadcastEdgeType(scale, graph), None
    _check_input(other, "other")
    if other.dtype != features.dtype or int(other.shape[0]) != graph.num_nodes \
            or get_feat_dim(other) != heads * M:
        raise RuntimeError("other must be (nodes, heads*M) of the features' dtype")
    xi, qi = _endpoint(graph, endpoint), _endpoint(graph, other_endpoint)
    out = torch.empty((graph.num_edges, heads), dtype=torch.float32, device=features.device)
    rc = capi.load().ga_segment_mm_gather(
        graph.etype_pointer.data_ptr(), graph.num_etypes, features.data_ptr(),
        xi.data_ptr(), weights.data_ptr(), None, other.data_ptr(), qi.data_ptr(),
        _ptr(scale), out.data_ptr(), None, graph.num_edges, heads, K, M,
        _feat_dtype(features, "features"), _stream(out))
    if rc == capi.GA_EUNSUPPORTED:
        y = SegmentMMEdgeGather(features, weights, endpoint, graph)
        prod = y.float() * _gather(other, qi).float().reshape(y.shape)
        out = prod.reshape(graph.num_edges, heads, M).sum(-1)
        if scale is not None:
            out = out * BroadcastEdgeType(scale.reshape(graph.num_etypes, heads), graph)
        return out if late is None else out * late
    capi.check(rc, "ga_segment_mm_gather")
    return out if late is None else out * late


# ------------------------------------------------------------ broadcast ----
def _gather(features: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    _check_input(features, "features")
    row_bytes = get_feat_dim(features) * features.element_size()
    out = torch.empty((index.shape[0],) + tuple(features.shape[1:]),
                      dtype=features.dtype, device=features.device)
    capi.check(capi.load().ga_gather_rows(
        index.data_ptr(), 64 if index.dtype == torch.int64 else 32,
        features.data_ptr(), out.data_ptr(), index.shape[0], row_bytes,
        _stream(out)), "ga_gather_rows")
    return out


def BroadcastSrcNode(features, graph: DGLGraph) -> torch.Tensor:
    """broadcast.cu:58-63: features[COO_src]."""
    return _gather(features, graph.COO_src)


def BroadcastDstNode(features, graph: DGLGraph) -> torch.Tensor:
    """broadcast.cu:64-69: features[COO_dst]."""
    return _gather(features, graph.COO_dst)


def BroadcastNodeType(features, graph: DGLGraph) -> torch.Tensor:
    """broadcast.cu:71-79: features[ntype_COO]."""
    if graph.ntype_COO is None:
        raise RuntimeError("the graph has no node-type column")
    return _gather(features, graph.ntype_COO)


def BroadcastSrcNodeType(features, graph: DGLGraph) -> torch.Tensor:
    """broadcast.cu:81-84."""
    return BroadcastSrcNode(BroadcastNodeType(features, graph), graph)


def BroadcastDstNodeType(features, graph: DGLGraph) -> torch.Tensor:
    """broadcast.cu:86-89."""
    return BroadcastDstNode(BroadcastNodeType(features, graph), graph)


def BroadcastEdgeType(features, graph: DGLGraph) -> torch.Tensor:
    """broadcast.cu:91-100: features[etype_COO]."""
    if graph.etype_COO is None:
        raise RuntimeError("the graph has no edge-type column")
    return _gather(features, graph.etype_COO)


# ----------------------------------------------------------- fused GAT ----
_ACTIVATIONS = {None: capi.GA_ACT_NONE, "relu": capi.GA_ACT_RELU, "elu": capi.GA_ACT_ELU}


def _activation(name) -> int:
    if name not in _ACTIVATIONS:
        raise RuntimeError("activation must be None, 'relu' or 'elu'")
    return _ACTIVATIONS[name]


def gat_aggregate(el, er, z, graph: DGLGraph, negative_slope: float = 0.01, activation=None):
    """u_add_v -> leaky_relu -> edge softmax -> u_mul_e sum in one pass
    (the four-operator chain of examples/GAT/GAT.py:25-36 at opt level 2).
    el, er: (N, H) fp32 attention terms of source / destination; z: (N, H*D).
    ``activation`` ("relu" | "elu"): the layer's activation, applied to the fp32
    rows before they are stored instead of by a pass of its own."""
    act = _activation(activation)
    _check_input(el, "el")
    _check_input(er, "er")
    _check_input(z, "z")
    dt = _feat_dtype(z, "z")
    if not (el.is_floating_point() and er.is_floating_point()):
        raise RuntimeError("el and er must be floating point")
    # bf16 attention terms (a bf16 plan's mm(z, attn_weight)): the logits are fp32 either way
    el, er = el.float().contiguous(), er.float().contiguous()
    heads = get_feat_dim(el)
    feat = get_feat_dim(z)
    if get_feat_dim(er) != heads or feat % heads:
        raise RuntimeError("inconsistent head count")
    out = torch.empty(_out_shape(graph.num_nodes, z), dtype=z.dtype,
                      device=z.device)
    lib = capi.load()
    ws_bytes = lib.ga_gat_workspace_bytes(graph.num_edges, feat, heads)
    ws = graph.workspace(ws_bytes)
    capi.check(lib.ga_gat_aggregate_act(
        graph.in_pointer.data_ptr(), graph.in_row_of_slot.data_ptr(),
        graph.in_node_indices.data_ptr(), el.data_ptr(), er.data_ptr(),
        z.data_ptr(), out.data_ptr(), graph.num_nodes, graph.num_edges, heads,
        feat // heads, float(negative_slope), act, dt, ws.data_ptr(), ws.numel(),
        _stream(out)), "ga_gat_aggregate")
    return out


def gat_aggregate_from_z(a_l, er, z, graph: DGLGraph, negative_slope: float = 0.01,
                         activation=None):
    """``gat_aggregate`` with the source term recomputed from the gathered row:
    logits leaky_relu(<z[src, h], a_l[h]> + er[dst, h]).  a_l: (H, D) fp32;
    er: (N, H) fp32; z: (N, H*D).  For node counts whose (N, H) table of source
    terms no longer fits the caches this saves one memory sector per edge."""
    act = _activation(activation)
    _check_input(a_l, "a_l")
    _check_input(er, "er")
    _check_input(z, "z")
    dt = _feat_dtype(z, "z")
    if a_l.dtype != torch.float32 or er.dtype != torch.float32:
        raise RuntimeError("a_l and er must be float32")
    heads = get_feat_dim(er)
    feat = get_feat_dim(z)
    if feat % heads or a_l.numel() != feat:
        raise RuntimeError("inconsistent head count")
    out = torch.empty(_out_shape(graph.num_nodes, z), dtype=z.dtype, device=z.device)
    lib = capi.load()
    ws = graph.workspace(lib.ga_gat_workspace_bytes(graph.num_edges, feat, heads))
    capi.check(lib.ga_gat_aggregate_from_z_act(
        graph.in_pointer.data_ptr(), graph.in_row_of_slot.data_ptr(),
        graph.in_node_indices.data_ptr(), a_l.data_ptr(), er.data_ptr(), z.data_ptr(),
        out.data_ptr(), graph.num_nodes, graph.num_edges, heads, feat // heads,
        float(negative_slope), act, dt, ws.data_ptr(), ws.numel(), _stream(out)),
        "ga_gat_aggregate_from_z")
    return out


def edge_softmax_sum(logits, messages, graph: DGLGraph) -> torch.Tensor:
    """out[v] = sum over in-edges e of softmax_v(logits)[e] * messages[e]: the
    SegmentSoftmax -> mul -> SpMMEdge tail of the reference's HGT plan
    (examples/HGT/HGT.py:50-53) in one pass.  logits (E,), (E, 1) or (E, H) fp32;
    messages (E, H*D) or (E, H, D), both in edge-id order."""
    _check_input(logits, "logits")
    _check_input(messages, "messages")
    dt = _feat_dtype(messages, "messages")
    if logits.dtype != torch.float32:
        raise RuntimeError("logits must be float32")
    heads, feat = get_feat_dim(logits), get_feat_dim(messages)
    if logits.shape[0] != graph.num_edges or messages.shape[0] != graph.num_edges:
        raise RuntimeError("logits and messages must have one row per edge")
    if feat % heads:
        raise RuntimeError("message width is not a multiple of the heads")
    out = torch.empty(_out_shape(graph.num_nodes, messages), dtype=messages.dtype,
                      device=messages.device)
    lib = capi.load()
    ws = graph.workspace(lib.ga_gat_workspace_bytes(graph.num_edges, feat, heads))
    capi.check(lib.ga_edge_softmax_sum(
        graph.in_pointer.data_ptr(), graph.in_row_of_slot.data_ptr(),
        None if graph.in_eid_is_identity else graph.in_edge_indices.data_ptr(),
        logits.data_ptr(), messages.data_ptr(), out.data_ptr(), graph.num_nodes,
        graph.num_edges, heads, feat // heads, dt, ws.data_ptr(), ws.numel(),
        _stream(out)), "ga_edge_softmax_sum")
    return out


def dot_attention_sum(k, q, v, graph: DGLGraph, return_lse: bool = False):
    """out[v] = sum over the in-edges e of v of softmax_v(<k[src], q[v]>)[e] * v[src], per
    head: ``sum(k * q)`` -> SegmentSoftmax -> mul -> SpMM (examples/HGT/HGT.py:44-53
    without its relation matrices) in one pass, nothing per edge written.  k, q, v
    (N, H, D) or (N, D) (one head).  ``return_lse``: also the (N, H) fp32 log of every
    destination's sum of exponentials (-inf without in-edges)."""
    for name, x in (("k", k), ("q", q), ("v", v)):
        _check_input(x, name)
    dt = _feat_dtype(k, "k")
    if q.dtype != k.dtype or v.dtype != k.dtype or q.shape != k.shape or v.shape != k.shape \
            or k.dim() not in (2, 3) or int(k.shape[0]) != graph.num_nodes:
        raise RuntimeError("k, q and v must be (nodes, heads, D) or (nodes, D) of one dtype")
    heads = 1 if k.dim() == 2 else int(k.shape[1])
    d = int(k.shape[-1])
    out = torch.empty_like(v)
    lse = torch.empty((graph.num_nodes, heads), dtype=torch.float32, device=k.device) \
        if return_lse else None
    lib = capi.load()
    ws = graph.workspace(lib.ga_gat_workspace_bytes(graph.num_edges, heads * d, heads))
    capi.check(lib.ga_dot_attention_sum(
        graph.in_pointer.data_ptr(), graph.in_row_of_slot.data_ptr(),
        graph.in_node_indices.data_ptr(), graph.in_row_of_slot.data_ptr(), k.data_ptr(),
        q.data_ptr(), v.data_ptr(), out.data_ptr(), _ptr(lse), None, graph.num_nodes,
        graph.num_edges, heads, d, dt, ws.data_ptr(), ws.numel(), _stream(out)),
        "ga_dot_attention_sum")
    return (out, lse) if return_lse else out


def relation_pair_attention(k, q, v, relation_att, relation_msg, relation_scale,
                            graph: DGLGraph, factor: float = 1.0) -> torch.Tensor:
    """The message and reduce stages of an HGT layer (examples/HGT/HGT.py:35-53) with
    the per-relation matrices applied once per (destination, relation) pair instead
    of once per edge -- both stages are linear in them:

      score[e, h] = <k[src] @ A[t], q[dst]> * s[t, h] = <k[src], q[dst] @ (s A[t])^T>
      out[v]      = sum_e a[e] * (v[src] @ M[t])      = sum_{pairs (v, t)} (sum_{e in pair} a[e] * v[src]) @ M[t]

    with a = softmax of the scores over the in-edges of v.  k, q, v (N, H*D);
    relation_att, relation_msg (T, H, D, D); relation_scale (T, H) fp32 or bf16 (the prior)
    or None, ``factor`` a further constant on the scores (1 / sqrt(D)): s = scale * factor.  The typed products run over P pairs, the scores are a
    plain dot product per edge and the weighted sum gathers rows of v: no (E, H*D)
    tensor is written.  Returns (N, H*D).  Raises GraphilerError(GA_EUNSUPPORTED) for
    shapes the typed-product kernel does not take and RuntimeError when the graph has
    no pair layout (DGLGraph.relation_pairs)."""
    for name, x in (("k", k), ("q", q), ("v", v), ("relation_att", relation_att),
                    ("relation_msg", relation_msg)):
        _check_input(x, name)
    dt = _feat_dtype(k, "k")
    if relation_att.dim() != 4 or relation_att.shape != relation_msg.shape \
            or int(relation_att.shape[0]) != graph.num_etypes \
            or relation_att.shape[2] != relation_att.shape[3]:
        raise RuntimeError("relation matrices must be (edge types, heads, D, D)")
    heads, d = int(relation_att.shape[1]), int(relation_att.shape[2])
    n, e, hid, n_types = graph.num_nodes, graph.num_edges, heads * d, graph.num_etypes
    for x in (k, q, v):
        if x.dtype != k.dtype or tuple(x.shape) != (n, hid):
            raise RuntimeError("k, q and v must be (nodes, heads*D) of one dtype")
    if relation_att.dtype != k.dtype or relation_msg.dtype != k.dtype:
        raise RuntimeError("relation matrices must have the features' dtype")
    pairs = graph.relation_pairs()
    if pairs is None:
        raise RuntimeError("the in-adjacency of this graph is not grouped by relation")
    lib, stream, dev, P = capi.load(), _stream(k), k.device, pairs.num_pairs
    if relation_scale is not None:
        _check_input(relation_scale, "relation_scale")
        if tuple(relation_scale.shape) != (n_types, heads) \
                or relation_scale.dtype not in (torch.float32, torch.bfloat16):
            raise RuntimeError("relation_scale must be (edge types, heads) float32 or bfloat16")
    # the matrices as the query side needs them: transposed, times the scale (an fp32
    # product rounded once to the features' dtype)
    att_t = torch.empty_like(relation_att)
    scale_dt = capi.GA_BF16 if relation_scale is not None and relation_scale.dtype == torch.bfloat16 \
        else capi.GA_F32
    capi.check(lib.ga_transpose_scale_blocks_as(
        relation_att.data_ptr(), _ptr(relation_scale), scale_dt, float(factor), att_t.data_ptr(),
        n_types * heads, d, dt, stream), "ga_transpose_scale_blocks_as")

    def typed_rows(x, index, w):        # row r = x[index[r]] @ w[relation of pair by_type[r]]
        y = torch.empty((P, hid), dtype=x.dtype, device=dev)
        capi.check(lib.ga_segment_mm_gather(
            pairs.type_pointer.data_ptr(), n_types, x.data_ptr(), index.data_ptr(),
            w.data_ptr(), y.data_ptr(), None, None, None, None, None, P, heads, d, d, dt,
            stream), "ga_segment_mm_gather")
        return y

    q_pair = typed_rows(q, pairs.dst_by_type, att_t)
    ws = graph.workspace(max(lib.ga_softmax_workspace_bytes(e, heads),
                             lib.ga_spmm_workspace_bytes(e, hid),
                             lib.ga_gat_workspace_bytes(e, hid, heads)))
    # scores, softmax inside every pair and the pair's weighted sum of value rows in one
    # pass; the pairs of a destination are then weighed by the softmax of their
    # log-sum-exps (the softmax-weighted sum of per-"edge" rows, with the pairs as the
    # edges), which makes the weights the softmax over all its in-edges
    v_pair = torch.empty((P, hid), dtype=v.dtype, device=dev)            # pair order
    lse = torch.empty((P, heads), dtype=torch.float32, device=dev)       # by_type order, like m_pair
    rc = lib.ga_dot_attention_sum(
        pairs.pair_pointer.data_ptr(), pairs.pair_of_slot.data_ptr(),
        graph.in_node_indices.data_ptr(), pairs.rank_of_slot.data_ptr(), k.data_ptr(),
        q_pair.data_ptr(), v.data_ptr(), v_pair.data_ptr(), lse.data_ptr(), pairs.rank.data_ptr(),
        P, e, heads, d, dt, ws.data_ptr(), ws.numel(), stream)
    if rc != capi.GA_EUNSUPPORTED:
        capi.check(rc, "ga_dot_attention_sum")
        m_pair = typed_rows(v_pair, pairs.by_type, relation_msg)         # by_type order
        out = torch.empty((n, hid), dtype=v.dtype, device=dev)
        capi.check(lib.ga_edge_softmax_sum(
            pairs.dst_pointer.data_ptr(), pairs.pair_dst.data_ptr(), pairs.rank.data_ptr(),
            lse.data_ptr(), m_pair.data_ptr(), out.data_ptr(), n, P, heads, d, dt, ws.data_ptr(),
            ws.numel(), stream), "ga_edge_softmax_sum")
        return out
    # head widths outside that kernel: the three steps as separate operators
    score = torch.empty((e, heads), dtype=torch.float32, device=dev)      # slot order
    capi.check(lib.ga_sddmm_u_dot_v(
        graph.in_node_indices.data_ptr(), pairs.rank_of_slot.data_ptr(), 32, k.data_ptr(),
        q_pair.data_ptr(), score.data_ptr(), e, heads, d, dt, stream), "ga_sddmm_u_dot_v")
    capi.check(lib.ga_segment_softmax(
        graph.in_pointer.data_ptr(), graph.in_row_of_slot.data_ptr(), None, score.data_ptr(),
        score.data_ptr(), n, e, heads, ws.data_ptr(), ws.numel(), stream), "ga_segment_softmax")
    capi.check(lib.ga_spmm_csr(
        pairs.pair_pointer.data_ptr(), pairs.pair_of_slot.data_ptr(),
        graph.in_node_indices.data_ptr(), None, v.data_ptr(), score.data_ptr(),
        v_pair.data_ptr(), P, e, hid, heads, capi.GA_U_MUL_E, capi.GA_SUM, dt, ws.data_ptr(),
        ws.numel(), stream), "ga_spmm_csr")
    m_pair = typed_rows(v_pair, pairs.by_type, relation_msg)             # by_type order
    out = torch.empty((n, hid), dtype=v.dtype, device=dev)
    capi.check(lib.ga_spmm_csr(
        pairs.dst_pointer.data_ptr(), pairs.pair_dst.data_ptr(), pairs.rank.data_ptr(),
        pairs.rank.data_ptr(), m_pair.data_ptr(), None, out.data_ptr(), n, P, hid, 1,
        capi.GA_COPY_E, capi.GA_SUM, dt, ws.data_ptr(), ws.numel(), stream), "ga_spmm_csr")
    return out


# ------------------------------------------------------ dense projection ----
# fp32 projections with at most this many output columns and at least this many rows
# run on the library's own kernel (one pass over the rows, 1.2-2.1x the rate of the
# vendor GEMM on an MI355X at these tall-and-narrow shapes); wider or shorter ones
# are the vendor GEMM's ground (several column passes / too few workgroups here).
LINEAR_MAX_COLS = 64
LINEAR_MIN_ROWS = 16384


def linear(x, weight, row_scale=None):
    """x @ weight for a (rows, K) node feature matrix and a (K, M) weight: the
    dense operator in front of the graph operators of a layer
    (examples/GCN/GCN.py:39 ``torch.mm(feature, self.weight)``).  ``row_scale``
    ((rows,) or (rows, 1) fp32): a factor per row of the product, the source-side
    norm of the GCN message (GCN.py:22-23), applied by the library's kernel to the
    rows it stores and by a multiplication afterwards on the ``torch.mm`` route."""
    if row_scale is not None and (row_scale.dtype != torch.float32
                                  or row_scale.numel() != x.shape[0]
                                  or row_scale.shape[0] != x.shape[0]):
        raise RuntimeError("row_scale must be (rows,) or (rows, 1) float32")
    if (x.dtype == torch.float32 and weight.dtype == torch.float32 and x.dim() == 2
            and weight.dim() == 2 and x.is_cuda and x.is_contiguous() and weight.is_contiguous()
            and weight.shape[1] <= LINEAR_MAX_COLS and x.shape[0] >= LINEAR_MIN_ROWS):
        if row_scale is None:
            return linear_attn(x, weight)
        _check_input(row_scale, "row_scale")
        if int(weight.shape[0]) != int(x.shape[1]):
            raise RuntimeError("weight must be (K, M)")
        z = torch.empty((x.shape[0], weight.shape[1]), dtype=x.dtype, device=x.device)
        capi.check(capi.load().ga_linear_rows_scaled(
            x.data_ptr(), weight.data_ptr(), row_scale.data_ptr(), z.data_ptr(),
            int(x.shape[0]), int(x.shape[1]), int(weight.shape[1]), _stream(x)),
            "ga_linear_rows_scaled")
        return z
    z = torch.mm(x, weight)
    return z if row_scale is None else z * row_scale.view(-1, 1).to(z.dtype)


def linear_attn(x, weight, a_l=None, a_r=None):
    """z = x @ weight and, when a_l / a_r (heads, D) fp32 are given, the GAT
    attention terms el = <z_h, a_l[h]>, er = <z_h, a_r[h]> (fp32) from the same
    kernel.  Returns z or (z, el, er).  fp32 or bf16 storage with the attention
    terms; fp32 only without them.  A shape the kernels do not take raises
    GraphilerError with GA_EUNSUPPORTED."""
    _check_input(x, "x")
    _check_input(weight, "weight")
    dt = _feat_dtype(x, "x")
    if weight.dtype != x.dtype:
        raise RuntimeError("x and weight must share a dtype")
    if x.dim() != 2 or weight.dim() != 2:
        raise RuntimeError("x must be (rows, K) and weight (K, M)")
    rows, K = int(x.shape[0]), int(x.shape[1])
    if int(weight.shape[0]) != K:
        raise RuntimeError("weight must be (K, M)")
    M = int(weight.shape[1])
    z = torch.empty((rows, M), dtype=x.dtype, device=x.device)
    if a_l is None:
        if x.dtype != torch.float32:
            raise RuntimeError("the plain projection is float32 only")
        capi.check(capi.load().ga_linear_attn(
            x.data_ptr(), weight.data_ptr(), None, None, z.data_ptr(), None, None,
            rows, K, M, 1, _stream(x)), "ga_linear_attn")
        return z
    _check_input(a_l, "a_l")
    _check_input(a_r, "a_r")
    if a_l.dtype != torch.float32 or a_r.dtype != torch.float32:
        raise RuntimeError("a_l and a_r must be float32")
    heads = int(a_l.shape[0])
    if a_l.numel() != M or a_r.numel() != M or M % heads:
        raise RuntimeError("a_l and a_r must be (heads, M / heads)")
    el = torch.empty((rows, heads), dtype=torch.float32, device=x.device)
    er = torch.empty((rows, heads), dtype=torch.float32, device=x.device)
    capi.check(capi.load().ga_project_attn(
        x.data_ptr(), weight.data_ptr(), a_l.data_ptr(), a_r.data_ptr(), z.data_ptr(),
        el.data_ptr(), er.data_ptr(), rows, K, M, heads, dt, _stream(x)), "ga_project_attn")
    return z, el, er
