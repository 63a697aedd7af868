"""Layer forwards as the operator sequences the reference's compiled plans run.

The reference turns DGL-style message / reduce / update functions into a
TorchScript graph of ``my_ops::*`` nodes (python/graphiler/mpdfg_builder.py:35-75,
src/optimizer/fusion.cpp:15-145) and executes it in ``update_all``
(python/graphiler/update_all.py:1-5).  The functions below are those
opt-level-2 operator sequences written out by hand for the four example models,
calling :mod:`graphiler_amd.ops`; the GAT projection uses the kernel that also
produces the attention terms, the GCN projection :func:`graphiler_amd.ops.linear`
(the library's kernel at tall-and-narrow fp32 shapes, ``torch.mm`` otherwise).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import capi, ops
from .graph import DGLGraph


def gcn_layer(g: DGLGraph, h: torch.Tensor, weight: torch.Tensor,
              norm_src: torch.Tensor, norm_dst: torch.Tensor | None = None,
              relu: bool = True) -> torch.Tensor:
    """examples/GCN/GCN.py:21-27,39: h' = act(SpMMSrc((h @ W) * norm_src)),
    optionally scaled by ``norm_dst`` for the symmetric normalisation."""
    if norm_src.dtype != torch.float32 or (norm_dst is not None and norm_dst.dtype != torch.float32):
        m = ops.linear(h, weight) * norm_src
        out = ops.SpMMSrc(m, [1], False, None, g)
        if norm_dst is not None:
            out = out * norm_dst
        return torch.relu(out) if relu else out
    # the norms and the relu ride on the rows the two kernels store
    m = ops.linear(h, weight, row_scale=norm_src.contiguous())
    if ops.spmm_tail_preferred(m, g):
        return ops.spmm_scaled(m, g, row_scale=None if norm_dst is None else norm_dst.contiguous(),
                               activation="relu" if relu else None)
    out = ops.SpMMSrc(m, [1], False, None, g)
    if norm_dst is not None:
        out = out * norm_dst
    return torch.relu(out) if relu else out


def gat_project(h, fc_weight, attn_weight, heads: int = 1):
    """Dense part of the GAT plan (GAT.py:25-29 after the split and reorder
    passes): z = h @ W, el = <z, a_l>, er = <z, a_r> per head."""
    try:        # one kernel: the GEMM with the attention terms in its epilogue
        return ops.linear_attn(h, fc_weight, attn_weight[0].float().contiguous(),
                               attn_weight[1].float().contiguous())
    except capi.GraphilerError as err:
        if err.code != capi.GA_EUNSUPPORTED:
            raise
    z = torch.mm(h, fc_weight)                               # (N, H*D)
    # per-head dot products as two skinny GEMMs with block-diagonal (H*D, H)
    # matrices: the reference's mm(z2, attn_weight) after its split pass
    el = torch.mm(z, _head_blocks(attn_weight[0].to(z.dtype)))           # (N, H)
    er = torch.mm(z, _head_blocks(attn_weight[1].to(z.dtype)))
    return z, el.float(), er.float()                         # fp32 terms, as the kernel returns them


def _head_blocks(a: torch.Tensor) -> torch.Tensor:
    """(H, D) per-head vectors -> (H*D, H) block-diagonal matrix."""
    heads, d = a.shape
    m = torch.zeros(heads * d, heads, dtype=a.dtype, device=a.device)
    for hd in range(heads):
        m[hd * d:(hd + 1) * d, hd] = a[hd]
    return m


# An (N, heads) fp32 table above this size (about what the 8 x 4 MB L2s hold
# besides the feature rows) makes the separate gather of the source term cost a
# memory sector per edge; measured: no difference at 0.9 MB, 17 % at 39 MB.
SOURCE_TERM_TABLE_LIMIT = 16 << 20


def gat_aggregate_plan(g: DGLGraph, z, el, er, negative_slope: float = 0.01):
    """The four graph operators of the reference's GAT plan, one after another."""
    e = ops.gsddmm_u_add_v_mul_alpha(el, er, 1, g)
    e = F.leaky_relu_(e, negative_slope)
    a = ops.SegmentSoftmax(e, 1, None, g)
    return ops.gspmm_src_mul_e_sum(z, a, [1], False, None, g)


def gat_layer(g: DGLGraph, h, fc_weight, attn_weight, heads: int = 1,
              negative_slope: float = 0.01, fused: bool = True, activation=None):
    """One GAT layer forward; ``fused`` runs the chain as a single pass.  When
    the (N, heads) table of source terms is too large to stay cached
    (``SOURCE_TERM_TABLE_LIMIT`` bytes), the pass recomputes them from the
    gathered rows instead of gathering them as well.  ``activation`` ("relu" |
    "elu"; the ``F.elu`` between the layers of examples/GAT/GAT.py) is applied by
    the fused pass to the rows it stores, by a separate call otherwise."""
    z, el, er = gat_project(h, fc_weight, attn_weight, heads)
    if fused:
        if el.numel() * el.element_size() >= SOURCE_TERM_TABLE_LIMIT:
            try:
                return ops.gat_aggregate_from_z(attn_weight[0].float().contiguous(), er.float(),
                                                z, g, negative_slope, activation)
            except capi.GraphilerError as err:      # head width the variant does not take
                if err.code != capi.GA_EUNSUPPORTED:
                    raise
        return ops.gat_aggregate(el.float(), er.float(), z, g, negative_slope, activation)
    out = gat_aggregate_plan(g, z, el, er, negative_slope)
    if activation == "elu":
        return F.elu(out)
    if activation == "relu":
        return torch.relu(out)
    if activation is not None:
        raise RuntimeError("activation must be None, 'relu' or 'elu'")
    return out


def rgcn_layer(g: DGLGraph, h, weight, norm, fused=True, activation=None):
    """examples/RGCN/RGCN.py:25-33.  weight (R, K, M); norm (E, 1) fp32; edges
    sorted by type.

    ``fused=True``: the typed product reads the source rows through the COO column
    and applies the norm to the rows it produces, then the neighbour sum (two
    passes over an (E, M) message tensor); for the small products where it is the
    faster one (ops.typed_spmm_preferred: 16 -> 64, 64 -> 8, ...; fp32 only on graphs
    without very large in-degrees, where its one accumulator per destination would
    lose accuracy), the single pass of ``fused="tiles"``.
    ``fused="pair"``: always the two passes.
    ``fused="tiles"``: ops.TypedSpMMEdge, one pass without the message tensor
    (K in 16, 32, 48, 64; M in 8, 16, 32, 64).
    ``fused=False``: the reference's plan BroadcastSrcNode -> SegmentMMEdge ->
    mul(norm) -> SpMMEdge.
    ``activation`` ("relu" | "elu"; the ``relu`` between the layers of
    examples/RGCN/RGCN.py:69): applied by the single pass to the sums it stores, by a
    separate call otherwise."""
    if activation not in (None, "relu", "elu"):
        raise RuntimeError("activation must be None, 'relu' or 'elu'")
    if fused == "tiles" or (fused is True and h.dim() == 2
                            and ops.typed_spmm_preferred(h, weight, g)):
        return ops.TypedSpMMEdge(h, weight, g, row_scale=norm.float().contiguous(),
                                 activation=activation)
    if fused:
        msg = ops.SegmentMMEdgeGather(h, weight, 0, g, row_scale=norm.float().contiguous())
        out = ops.SpMMEdge(msg, [1], False, None, g)
    else:
        hs = ops.BroadcastSrcNode(h, g)
        msg = ops.SegmentMMEdge(hs, weight, g)
        msg = msg * norm.to(msg.dtype)
        out = ops.SpMMEdge(msg, [1], False, None, g)
    if activation == "relu":
        return torch.relu(out)
    return F.elu(out) if activation == "elu" else out


# Edges per (destination, relation) pair from which an HGT layer applies its relation
# matrices per pair: the pair form replaces two typed products over E rows by two over
# P rows plus two passes over the pairs.
PAIRS_MIN_EDGES_PER_PAIR = 2.0


def hgt_layer(g: DGLGraph, h, k_weight, q_weight, v_weight, a_weight,
              relation_att, relation_msg, relation_pri, skip, heads: int = 1,
              fused=True):
    """examples/HGT/HGT.py:28-60 as the operator sequence of its optimised plan,
    generalised from one head to ``heads`` heads of width D = hidden / heads:

      K, V, Q   = SegmentMMNode(h, W_k | W_v | W_q)            per node type, h read once
      k_e, v_e  = BroadcastSrcNode(K | V);  q_e = BroadcastDstNode(Q)
      k_e, v_e  = SegmentMMEdge(k_e, relation_att | relation_msg)   per edge type,
                                                         one (D x D) block per head
      attn      = sum_D(k_e * q_e) * BroadcastEdgeType(relation_pri) / sqrt(D)
      t         = SpMMEdge(SegmentSoftmax(attn) * v_e)
      out       = SegmentMMNode(t, W_a) * sigmoid(BroadcastNodeType(skip))

    k/q/v/a_weight: (T_n, hidden, hidden); relation_att / relation_msg:
    (T_e, heads, D, D); relation_pri: (T_e, heads); skip: (T_n,).

    ``fused="edges"`` replaces the per-edge copies and products by
      attn = SegmentMMEdgeDot(K, relation_att, src, Q, dst) * pri / sqrt(D)
      t    = edge_softmax_sum(attn, SegmentMMEdgeGather(V, relation_msg, src))
    so the only per-edge tensors are the scores and the transformed values.
    ``fused="pairs"`` applies the relation matrices once per (destination, relation)
    pair instead (ops.relation_pair_attention): no per-edge tensor but the scores.
    ``fused=True`` takes the pairs when the graph has at least ``PAIRS_MIN_EDGES_PER_PAIR``
    edges per pair (config 4: 7.4) and the per-edge form otherwise.
    """
    n, hidden = h.shape
    d = hidden // heads
    e = g.num_edges
    # the three projections of h in one pass over its rows
    k, v, q = ops.SegmentMMNodeStacked(h, [k_weight, v_weight, q_weight], g)
    t = None
    if fused == "pairs" or fused is True:
        pairs = g.relation_pairs()
        if fused == "pairs" and pairs is None:
            raise RuntimeError("the in-adjacency of this graph is not grouped by relation")
        if pairs is not None and (fused == "pairs"
                                  or e >= PAIRS_MIN_EDGES_PER_PAIR * pairs.num_pairs):
            try:
                pri = relation_pri if relation_pri.dtype in (torch.float32, torch.bfloat16) \
                    else relation_pri.float()
                t = ops.relation_pair_attention(k, q, v, relation_att, relation_msg,
                                                pri.contiguous(), g,
                                                factor=1.0 / (d ** 0.5))
            except capi.GraphilerError as err:      # head width outside the typed product
                if err.code != capi.GA_EUNSUPPORTED or fused == "pairs":
                    raise
    if t is None and fused:
        attn = ops.SegmentMMEdgeDot(k, relation_att, 0, q, 1, g,
                                    scale=relation_pri.float() / (d ** 0.5))
        v_e = ops.SegmentMMEdgeGather(v, relation_msg, 0, g)
        t = ops.edge_softmax_sum(attn, v_e, g)
    elif t is None:
        pri = ops.BroadcastEdgeType(relation_pri.float(), g) / (d ** 0.5)
        k_e = ops.SegmentMMEdge(ops.BroadcastSrcNode(k, g), relation_att, g)
        v_e = ops.SegmentMMEdge(ops.BroadcastSrcNode(v, g), relation_msg, g)
        q_e = ops.BroadcastDstNode(q, g)
        attn = (k_e.view(e, heads, d).float() * q_e.view(e, heads, d).float()).sum(-1) * pri
        a = ops.SegmentSoftmax(attn.contiguous(), 1, None, g)      # (E, heads) fp32
        m = (v_e.view(e, heads, d).float() * a.unsqueeze(-1)).to(h.dtype).view(e, hidden)
        t = ops.SpMMEdge(m, [1], False, None, g)
    if fused:       # the gate goes into the product's epilogue, sigmoid and copy to the nodes included
        return ops.SegmentMMNodeGated(t, a_weight, skip.float().contiguous(), g, sigmoid=True)
    alpha = ops.BroadcastNodeType(torch.sigmoid(skip.float()).unsqueeze(1), g)
    out = ops.SegmentMMNode(t, a_weight, g)
    return (out.float() * alpha).to(h.dtype)
