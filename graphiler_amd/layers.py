"""Layer forwards as the operator sequences the reference's compiled plans run.

The reference turns DGL-style message / reduce / update functions into a
TorchScript graph of ``my_ops::*`` nodes (python/graphiler/mpdfg_builder.py:35-75,
src/optimizer/fusion.cpp:15-145) and executes it in ``update_all``
(python/graphiler/update_all.py:1-5).  The functions below are those
opt-level-2 operator sequences written out by hand for the four example models,
calling :mod:`graphiler_amd.ops`; dense per-node linears stay on ``torch.mm``
exactly as in the reference plans.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import ops
from .graph import DGLGraph


def gcn_layer(g: DGLGraph, h: torch.Tensor, weight: torch.Tensor,
              norm_src: torch.Tensor, norm_dst: torch.Tensor | None = None,
              relu: bool = True) -> torch.Tensor:
    """examples/GCN/GCN.py:21-27,39: h' = act(SpMMSrc((h @ W) * norm_src)),
    optionally scaled by ``norm_dst`` for the symmetric normalisation."""
    m = torch.mm(h, weight) * norm_src
    out = ops.SpMMSrc(m, [1], False, None, g)
    if norm_dst is not None:
        out = out * norm_dst
    return torch.relu(out) if relu else out


def gat_project(h, fc_weight, attn_weight, heads: int = 1):
    """Dense part of the GAT plan (GAT.py:25-29 after the split and reorder
    passes): z = h @ W, el = <z, a_l>, er = <z, a_r> per head."""
    z = torch.mm(h, fc_weight)                               # (N, H*D)
    # per-head dot products as two skinny GEMMs with block-diagonal (H*D, H)
    # matrices: the reference's mm(z2, attn_weight) after its split pass
    el = torch.mm(z, _head_blocks(attn_weight[0]))           # (N, H)
    er = torch.mm(z, _head_blocks(attn_weight[1]))
    return z, el, er


def _head_blocks(a: torch.Tensor) -> torch.Tensor:
    """(H, D) per-head vectors -> (H*D, H) block-diagonal matrix."""
    heads, d = a.shape
    m = torch.zeros(heads * d, heads, dtype=a.dtype, device=a.device)
    for hd in range(heads):
        m[hd * d:(hd + 1) * d, hd] = a[hd]
    return m


def gat_aggregate_plan(g: DGLGraph, z, el, er, negative_slope: float = 0.01):
    """The four graph operators of the reference's GAT plan, one after another."""
    e = ops.gsddmm_u_add_v_mul_alpha(el, er, 1, g)
    e = F.leaky_relu_(e, negative_slope)
    a = ops.SegmentSoftmax(e, 1, None, g)
    return ops.gspmm_src_mul_e_sum(z, a, [1], False, None, g)


def gat_layer(g: DGLGraph, h, fc_weight, attn_weight, heads: int = 1,
              negative_slope: float = 0.01, fused: bool = True):
    """One GAT layer forward; ``fused`` runs the chain as a single pass."""
    z, el, er = gat_project(h, fc_weight, attn_weight, heads)
    if fused:
        return ops.gat_aggregate(el, er, z, g, negative_slope)
    return gat_aggregate_plan(g, z, el, er, negative_slope)


def rgcn_layer(g: DGLGraph, h, weight, norm):
    """examples/RGCN/RGCN.py:25-33: BroadcastSrcNode -> SegmentMMEdge ->
    mul(norm) -> SpMMEdge.  weight (R, K, M); norm (E, 1); edges sorted by type."""
    hs = ops.BroadcastSrcNode(h, g)
    msg = ops.SegmentMMEdge(hs, weight, g)
    msg = msg * norm.to(msg.dtype)
    return ops.SpMMEdge(msg, [1], False, None, g)
