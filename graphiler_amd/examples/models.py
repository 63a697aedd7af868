"""The four example models as two-layer networks over compiled plans, with an
eager PyTorch baseline of the same user-defined functions.

Structure follows the reference's examples (examples/GCN/GCN.py:33-58,
examples/GAT/GAT.py:43-84, examples/RGCN/RGCN.py:39-77,
examples/HGT/HGT.py:63-190): a layer stores its inputs in the graph's feature
dictionaries and calls ``update_all`` with the plan of the requested
optimisation level.  ``mode`` is 0 / 1 / 2 (plan compiled at that level, the
reference's "+compile", "+reorder", "+fusion") or ``"eager"``: the same
message / reduce / update arithmetic written with ``index_select`` /
``index_add_`` / ``scatter_reduce`` on materialised per-edge tensors, which is
what a message-passing framework without a compiler executes; ``"eager64"`` is
the same with the per-destination sums accumulated in float64 (fp32 atomic adds
lose two to three digits on rows with 10^5-10^6 in-edges, so the plain eager
result cannot serve as the expected value on power-law graphs).  Weights are
positive uniform draws from a seeded generator (the reference draws ``torch.rand``).
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

from .. import ops
from ..mpdfg import GraphData, mpdfg_builder, update_all
from . import udf

_PLANS = {}


def plan(name: str, level: int):
    """Compiled plan of model ``name`` at optimisation level ``level`` (cached)."""
    key = (name, level)
    if key not in _PLANS:
        fns = {
            "GCN": (udf.gcn_message, udf.gcn_reduce, None),
            "GAT": (udf.gat_message, udf.gat_reduce, None),
            "RGCN": (udf.rgcn_message, udf.rgcn_reduce, None),
            "HGT": (udf.hgt_message, udf.hgt_reduce, udf.hgt_update),
        }[name]
        _PLANS[key] = mpdfg_builder(*fns, opt_level=level)
    return _PLANS[key]


def _param(rng, shape, device):
    """U(0, 2 / fan_in): positive like the reference's ``torch.rand`` weights (no
    cancellation, so a purely relative comparison of two results is meaningful),
    scaled so that activations stay of order one through both layers."""
    w = rng.random(shape, dtype=np.float32) * np.float32(2.0 / shape[-2])
    return torch.from_numpy(w).to(device)


# ---- eager building blocks ---------------------------------------------------------
EAGER = ("eager", "eager64")


def _sum_by_dst(g: GraphData, msg: torch.Tensor, mode="eager") -> torch.Tensor:
    dst = g.graph.COO_dst
    shape = (g.graph.num_nodes,) + tuple(msg.shape[1:])
    if mode != "eager64":
        return torch.zeros(shape, dtype=msg.dtype, device=msg.device).index_add_(0, dst, msg)
    out = torch.zeros(shape, dtype=torch.float64, device=msg.device)
    step = 1 << 24                      # bounds the float64 copy of the messages
    for lo in range(0, dst.numel(), step):
        out.index_add_(0, dst[lo:lo + step], msg[lo:lo + step].double())
    return out.to(msg.dtype)


def _softmax_by_dst(g: GraphData, score: torch.Tensor, mode="eager") -> torch.Tensor:
    dst = g.graph.COO_dst
    idx = dst.unsqueeze(1).expand_as(score)
    top = torch.full((g.graph.num_nodes, score.shape[1]), -math.inf, dtype=score.dtype,
                     device=score.device).scatter_reduce_(0, idx, score, "amax")
    p = torch.exp(score - top[dst])
    return p / _sum_by_dst(g, p, mode)[dst]


def _typed_rows(x: torch.Tensor, weight: torch.Tensor, type_of: torch.Tensor) -> torch.Tensor:
    return torch.bmm(x.unsqueeze(1), weight[type_of]).squeeze(1)


# ---- GCN ---------------------------------------------------------------------------
class GCN:
    def __init__(self, in_dim, hidden_dim, out_dim, device, seed=0):
        rng = np.random.default_rng(seed)
        self.w1 = _param(rng, (in_dim, hidden_dim), device)
        self.w2 = _param(rng, (hidden_dim, out_dim), device)

    def _layer(self, g, x, w, mode):
        g.ndata['h'] = torch.mm(x, w) if mode in EAGER else ops.linear(x, w)
        if mode in EAGER:
            src = g.graph.COO_src
            m = g.ndata['h'][src] * torch.pow(g.ndata['degree'][src], -0.5)
            g.ndata['h'] = torch.relu(_sum_by_dst(g, m, mode))
        else:
            update_all(g, plan("GCN", mode))
        return g.ndata.pop('h')

    def __call__(self, g: GraphData, features, mode=2):
        ptr = g.graph.in_pointer
        g.ndata['degree'] = (ptr[1:] - ptr[:-1]).float().clamp(min=1).unsqueeze(1)
        x = F.relu(self._layer(g, features, self.w1, mode))
        return self._layer(g, x, self.w2, mode)


# ---- GAT (one head) ------------------------------------------------------------------
class GAT:
    def __init__(self, in_dim, hidden_dim, out_dim, device, seed=0):
        rng = np.random.default_rng(seed)
        self.layers = []
        for a, b in ((in_dim, hidden_dim), (hidden_dim, out_dim)):
            self.layers.append((_param(rng, (a, b), device),
                                _param(rng, (2 * b, 1), device)))

    def _layer(self, g, x, fc, attn, mode):
        g.ndata['h'] = x
        if mode in EAGER:
            z = torch.mm(x, fc)
            z_src, z_dst = z[g.graph.COO_src], z[g.graph.COO_dst]
            e = F.leaky_relu(torch.mm(torch.cat([z_src, z_dst], dim=1), attn), 0.2)
            g.ndata['h'] = _sum_by_dst(g, _softmax_by_dst(g, e, mode) * z_src, mode)
        else:
            update_all(g, plan("GAT", mode), msg_params=(fc, attn))
        return g.ndata.pop('h')

    def __call__(self, g: GraphData, features, mode=2):
        h = F.elu(self._layer(g, features, *self.layers[0], mode))
        return self._layer(g, h, *self.layers[1], mode)


# ---- RGCN ------------------------------------------------------------------------------
class RGCN:
    def __init__(self, in_dim, hidden_dim, out_dim, num_rels, device, seed=0):
        rng = np.random.default_rng(seed)
        self.w1 = _param(rng, (num_rels, in_dim, hidden_dim), device)
        self.w2 = _param(rng, (num_rels, hidden_dim, out_dim), device)

    def _layer(self, g, x, w, norm, mode):
        g.ndata['h'], g.edata['norm'], g.etype_data['weight'] = x, norm, w
        if mode in EAGER:
            msg = _typed_rows(x[g.graph.COO_src], w, g.graph.etype_COO) * norm
            g.ndata['h'] = _sum_by_dst(g, msg, mode)
        else:
            update_all(g, plan("RGCN", mode))
        return g.ndata.pop('h')

    def __call__(self, g: GraphData, features, norm, mode=2):
        x = F.relu(self._layer(g, features, self.w1, norm, mode))
        return self._layer(g, x, self.w2, norm, mode)


# ---- HGT (single head) -------------------------------------------------------------------
class HGTLayer:
    def __init__(self, rng, in_dim, out_dim, num_ntypes, num_rels, device):
        self.sqrt_dk = math.sqrt(out_dim)
        self.k, self.q, self.v = (_param(rng, (num_ntypes, in_dim, out_dim), device)
                                  for _ in range(3))
        self.a = _param(rng, (num_ntypes, out_dim, out_dim), device)
        self.rel_att, self.rel_msg = (_param(rng, (num_rels, out_dim, out_dim), device)
                                      for _ in range(2))
        self.rel_pri = torch.ones(num_rels, 1, device=device)
        self.skip = torch.ones(num_ntypes, device=device)

    def __call__(self, g: GraphData, h, mode):
        g.ndata['h'] = h
        g.ntype_data.update(k_weight=self.k, q_weight=self.q, v_weight=self.v,
                            a_weight=self.a, skip=self.skip)
        g.etype_data.update(relation_att=self.rel_att, relation_msg=self.rel_msg,
                            relation_pri=self.rel_pri)
        if mode in EAGER:
            G = g.graph
            src, dst, et, nt = G.COO_src, G.COO_dst, G.etype_COO, G.ntype_COO
            k = _typed_rows(h[src], self.k, nt[src])
            v = _typed_rows(h[src], self.v, nt[src])
            q = _typed_rows(h[dst], self.q, nt[dst])
            k = _typed_rows(k, self.rel_att, et)
            v = _typed_rows(v, self.rel_msg, et)
            score = torch.sum(k * q, dim=1, keepdim=True) * self.rel_pri[et] / self.sqrt_dk
            t = _sum_by_dst(g, _softmax_by_dst(g, score, mode) * v, mode)
            out = _typed_rows(t, self.a, nt)
            g.ndata['h'] = out * torch.sigmoid(self.skip[nt]).unsqueeze(1)
        else:
            update_all(g, plan("HGT", mode), msg_params=(self.sqrt_dk,))
        return g.ndata.pop('h')


class HGT:
    def __init__(self, in_dim, hidden_dim, out_dim, num_ntypes, num_rels, device, seed=0):
        rng = np.random.default_rng(seed)
        self.layer1 = HGTLayer(rng, in_dim, hidden_dim, num_ntypes, num_rels, device)
        self.layer2 = HGTLayer(rng, hidden_dim, out_dim, num_ntypes, num_rels, device)

    def __call__(self, g: GraphData, features, mode=2):
        return self.layer2(g, self.layer1(g, features, mode), mode)
