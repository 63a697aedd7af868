"""Rewrites of a built plan: split, reorder, fusion (src/optimizer/split.cpp,
reorder.cpp, fusion.cpp, dedup.cpp), written as direct graph surgery so that a
rewrite can ask where a value lives (the reference matches on operator names
only and notes residency as a to-do, reorder.cpp:14-15, split.cpp:8).

* split:   ``mm(cat([a, b], 1), w)`` -> ``mm(a, w[:fa]) + mm(b, w[fa:])`` so each
  half can move to node data on its own (the GAT attention product).
* reorder: an operator that acts row by row commutes with a broadcast: ``op(
  Broadcast(x))`` -> ``Broadcast(op(x))`` does the work once per node instead of
  once per edge.  Allowed when every other operand is shared (a weight, a
  constant); two broadcasts of the same kind under one binary operator merge.
* fusion:  broadcast + compute + reduce chains into the fused graph operators:
  ``SpMMSrc``, ``gspmm_{src,dst}_mul_e_sum``, ``gsddmm_u_add_v_mul_alpha``,
  ``SegmentMMNode/Edge`` for per-type ``bmm``, and (not in the reference) the
  whole attention chain into ``gat_aggregate``.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .builder import EDGE, ETYPE, MPDFG, NODE, NTYPE, SHARED

_BCAST = {"my_ops::BroadcastSrcNode", "my_ops::BroadcastDstNode", "my_ops::BroadcastSrcNodeType",
          "my_ops::BroadcastDstNodeType", "my_ops::BroadcastEdgeType", "my_ops::BroadcastNodeType"}
# row-wise operators whose first operand is the data and the rest are shared
_ROWWISE = {"aten::relu", "aten::sigmoid", "aten::tanh", "aten::exp", "aten::neg",
            "aten::leaky_relu", "aten::squeeze", "aten::mm", "aten::pow", "aten::unsqueeze",
            "aten::view", "aten::reshape", "aten::sum", "aten::elu"}
_INPLACE = {"aten::relu_": "aten::relu", "aten::leaky_relu_": "aten::leaky_relu",
            "aten::sigmoid_": "aten::sigmoid", "aten::tanh_": "aten::tanh"}
_PAIRWISE = {"aten::mul", "aten::add", "aten::sub", "aten::div"}


def dedup(graph: torch._C.Graph) -> None:
    """Dead code, pooled constants, common subexpressions; the graph operators
    are pure functions of their inputs too, which TorchScript cannot know."""
    torch._C._jit_pass_dce(graph)
    torch._C._jit_pass_constant_pooling(graph)
    torch._C._jit_pass_cse(graph)
    # repeated reads of one feature (ndata["h"] for the source and again for the
    # destination): TorchScript keeps both because dictionaries are mutable; they
    # are the same tensor as long as no _set_item on that dictionary lies between
    known = {}
    for n in list(graph.nodes()):
        if n.kind() == "aten::_set_item":
            d = n.inputsAt(0).unique()
            known = {k: v for k, v in known.items() if k[0] != d}
        elif n.kind() == "aten::__getitem__" and n.inputsAt(1).node().kind() == "prim::Constant":
            key = (n.inputsAt(0).unique(), n.inputsAt(1).unique())
            if key in known:
                n.output().replaceAllUsesWith(known[key])
                n.destroy()
            else:
                known[key] = n.output()
    torch._C._jit_pass_cse(graph)

    mutated = _mutated
    changed = True
    while changed:
        changed = False
        seen = {}
        for n in list(graph.nodes()):
            ours = n.kind().startswith("my_ops::")
            # TorchScript's own pass will not merge two equal aten nodes once a
            # custom operator reads their results (it must assume it writes them)
            pure_aten = (n.kind().startswith("aten::") and not n.kind().endswith("_")
                         and n.kind() not in ("aten::__getitem__", "aten::_set_item")
                         and n.outputsSize() == 1 and not n.attributeNames()
                         and not any(mutated(i) for i in n.inputs())
                         and not mutated(n.output()))
            if not ours and not pure_aten:
                continue
            if ours and not any(o.uses() for o in n.outputs()):
                n.destroy()
                changed = True
                continue
            # a result that an in-place operator (leaky_relu_, relu_, ...) later
            # overwrites, or an operand that one does, is not the same value twice
            if ours and (any(mutated(o) for o in n.outputs()) or any(mutated(i) for i in n.inputs())):
                continue
            key = (n.kind(), tuple(i.unique() for i in n.inputs()))
            if key in seen:
                n.replaceAllUsesWith(seen[key])
                n.destroy()
                changed = True
            else:
                seen[key] = n
    torch._C._jit_pass_dce(graph)


def _mutated(v) -> bool:
    """True when an in-place operator (aten::*_) or a dictionary store uses ``v``."""
    return any(u.user.kind().endswith("_") or u.user.kind() == "aten::_set_item"
               for u in v.uses())


class _Rewriter:
    def __init__(self, plan: MPDFG):
        self.plan = plan
        self.G = plan.graph
        self.res = plan.residency
        self.dglgraph = list(self.G.inputs())[0]

    def where(self, v) -> str:
        return self.res.get(v.unique(), SHARED)

    def make(self, kind, inputs, before, residency, ty=None, like=None):
        node = self.G.create(kind, list(inputs), 1)
        if like is not None:
            node.copyAttributes(like)
            node.output().copyMetadata(like.output())
        node.insertBefore(before)
        node.output().setType(ty if ty is not None else
                              (like.output().type() if like is not None
                               else torch._C.TensorType.get()))
        self.res[node.output().unique()] = residency
        return node.output()

    def const(self, value, before):
        with self.G.insert_point_guard(before):
            v = self.G.insertConstant(value)
        self.res[v.unique()] = SHARED
        return v

    @staticmethod
    def single_use(v) -> bool:
        return len(v.uses()) == 1

    @staticmethod
    def const_of(v):
        from .builder import _const_of
        return _const_of(v)

    # ------------------------------------------------------------- split ----
    def split(self) -> bool:
        changed = False
        for n in list(self.G.nodes()):
            if n.kind() != "aten::mm":
                continue
            cat = n.inputsAt(0).node()
            if cat.kind() != "aten::cat" or self.const_of(cat.inputsAt(1)) != 1:
                continue
            lst = cat.inputsAt(0).node()
            if lst.kind() != "prim::ListConstruct" or lst.inputsSize() != 2:
                continue
            a, b = lst.inputsAt(0), lst.inputsAt(1)
            w = n.inputsAt(1)
            if self.where(w) != SHARED:
                continue
            r = self.where(n.output())
            int_t = torch._C.IntType.get()
            fa = self.make("my_ops::get_feat_dim", [a], n, SHARED, ty=int_t)
            zero, one = self.const(0, n), self.const(1, n)
            none = self.const(None, n)
            w_a = self.make("aten::slice", [w, zero, zero, fa, one], n, SHARED)
            w_b = self.make("aten::slice", [w, zero, fa, none, one], n, SHARED)
            m_a = self.make("aten::mm", [a, w_a], n, self.where(a))
            m_b = self.make("aten::mm", [b, w_b], n, self.where(b))
            out = self.make("aten::add", [m_a, m_b, one], n, r)
            n.output().replaceAllUsesWith(out)
            n.destroy()
            changed = True
        return changed

    # ----------------------------------------------------------- reorder ----
    def _target_residency(self, bkind: str, src_res: str) -> str:
        return NODE if bkind == "my_ops::BroadcastNodeType" else EDGE

    def reorder(self) -> bool:
        changed = False
        for n in list(self.G.nodes()):
            kind = _INPLACE.get(n.kind(), n.kind())
            if n.inputsSize() == 0:
                continue
            first = n.inputsAt(0).node()
            if kind == "my_ops::get_feat_dim" and first.kind() in _BCAST:
                n.replaceInput(0, first.inputsAt(0))
                changed = True
                continue
            if kind == "my_ops::get_feat_dim" and first.kind() == "aten::mm":
                # width of a product = columns of its right operand: frees the
                # consumer (a weight slice) from depending on the product itself
                one = self.const(1, n)
                cols = self.make("aten::size", [first.inputsAt(1), one], n, SHARED,
                                 ty=torch._C.IntType.get())
                n.output().replaceAllUsesWith(cols)
                n.destroy()
                changed = True
                continue
            if kind in _PAIRWISE and n.inputsSize() >= 2:
                second = n.inputsAt(1).node()
                if (first.kind() in _BCAST and second.kind() == first.kind()
                        and first.inputsAt(1).unique() == second.inputsAt(1).unique()
                        and self.where(first.inputsAt(0)) == self.where(second.inputsAt(0))
                        and all(self.where(i) == SHARED for i in list(n.inputs())[2:])):
                    src_res = self.where(first.inputsAt(0))
                    ins = [first.inputsAt(0), second.inputsAt(0)] + list(n.inputs())[2:]
                    small = self.make(kind, ins, n, src_res, like=n)
                    back = self.make(first.kind(), [small, self.dglgraph], n,
                                     self.where(n.output()))
                    n.output().replaceAllUsesWith(back)
                    n.destroy()
                    changed = True
                    continue
            if kind in _PAIRWISE and n.inputsSize() >= 2 and self._hop_pairwise(n, kind):
                changed = True
                continue
            if kind not in _ROWWISE or first.kind() not in _BCAST:
                continue
            if any(self.where(i) != SHARED for i in list(n.inputs())[1:]):
                continue
            if kind in ("aten::view", "aten::reshape"):
                # row-wise when the rows stay the leading dimension: a leading -1
                # (a view of per-edge data that regroups rows has no meaning as
                # per-edge data, so the others are taken to describe one row)
                shape = self.const_of(n.inputsAt(1))
                if not isinstance(shape, list) or len(shape) < 2 or shape[0] != -1 \
                        or any(not isinstance(d, int) or d <= 0 for d in shape[1:]):
                    continue
            if kind == "aten::sum":
                # only reductions inside a row: every listed dimension >= 1
                dims = self.const_of(n.inputsAt(1)) if n.inputsSize() == 4 else None
                if not isinstance(dims, list) or not dims or \
                        any(not isinstance(d, int) or d < 1 for d in dims):
                    continue
            if kind == "aten::unsqueeze" and self.const_of(n.inputsAt(1)) in (0, None):
                continue                      # a new leading dimension is not row-wise
            if kind == "aten::squeeze" and n.inputsSize() > 1 and self.const_of(n.inputsAt(1)) in (0, None):
                continue
            src = first.inputsAt(0)
            small = self.make(kind, [src] + list(n.inputs())[1:], n, self.where(src), like=n)
            back = self.make(first.kind(), [small, self.dglgraph], n, self.where(n.output()))
            n.output().replaceAllUsesWith(back)
            n.destroy()
            changed = True
        return changed

    def _hop_pairwise(self, n, kind) -> bool:
        """``op(Broadcast(x), w)`` / ``op(w, Broadcast(x))`` with a shared tensor or
        constant ``w`` (a weight that broadcasts against every row alike) ->
        ``Broadcast(op(x, w))``."""
        ins = list(n.inputs())
        for pos in (0, 1):
            bc, other = ins[pos].node(), ins[1 - pos]
            if bc.kind() not in _BCAST or self.where(other) != SHARED:
                continue
            if any(self.where(i) != SHARED for i in ins[2:]):
                continue
            src = bc.inputsAt(0)
            new_ins = list(ins)
            new_ins[pos] = src
            small = self.make(kind, new_ins, n, self.where(src), like=n)
            back = self.make(bc.kind(), [small, self.dglgraph], n, self.where(n.output()))
            n.output().replaceAllUsesWith(back)
            n.destroy()
            return True
        return False

    # ------------------------------------------------------------ fusion ----
    def fusion(self) -> bool:
        changed = False
        for n in list(self.G.nodes()):
            kind = n.kind()
            if kind == "my_ops::SpMMEdge":
                changed |= self._fuse_spmm(n)
            elif kind == "aten::add":
                changed |= self._fuse_u_add_v(n)
            elif kind == "aten::squeeze" and n.inputsSize() == 1:
                inner = n.input().node()
                if inner.kind() == "aten::unsqueeze":
                    n.output().replaceAllUsesWith(inner.inputsAt(0))
                    n.destroy()
                    changed = True
            elif kind == "aten::bmm":
                changed |= self._fuse_bmm(n)
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::gspmm_src_mul_e_sum":
                changed |= self._fuse_gat_chain(n)
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::gat_aggregate":
                changed |= self._fuse_gat_project(n)
        return changed

    def _fuse_spmm(self, n) -> bool:
        x = n.inputsAt(0).node()
        rest = list(n.inputs())[1:]                 # dims, keep, dtype, graph
        if x.kind() == "my_ops::BroadcastSrcNode":
            out = self.make("my_ops::SpMMSrc", [x.inputsAt(0)] + rest, n, NODE)
        elif x.kind() == "aten::mul":
            a, b = x.inputsAt(0), x.inputsAt(1)
            for msg, bc in ((a, b), (b, a)):
                k = bc.node().kind()
                if k in ("my_ops::BroadcastSrcNode", "my_ops::BroadcastDstNode") \
                        and self.where(msg) == EDGE:
                    op = "my_ops::gspmm_src_mul_e_sum" if "Src" in k else "my_ops::gspmm_dst_mul_e_sum"
                    out = self.make(op, [bc.node().inputsAt(0), msg] + rest, n, NODE)
                    break
            else:
                return False
        else:
            return False
        n.output().replaceAllUsesWith(out)
        n.destroy()
        return True

    def _fuse_u_add_v(self, n) -> bool:
        if n.inputsSize() != 3:
            return False
        a, b = n.inputsAt(0).node(), n.inputsAt(1).node()
        if a.kind() != "my_ops::BroadcastSrcNode" or b.kind() != "my_ops::BroadcastDstNode":
            return False
        alpha = self.const_of(n.inputsAt(2))
        if alpha != 1:                              # the operator ignores alpha (sddmm.cu:116-121)
            return False
        out = self.make("my_ops::gsddmm_u_add_v_mul_alpha",
                        [a.inputsAt(0), b.inputsAt(0), n.inputsAt(2), self.dglgraph], n, EDGE)
        n.output().replaceAllUsesWith(out)
        n.destroy()
        return True

    def _fuse_bmm(self, n) -> bool:
        x, w = n.inputsAt(0), n.inputsAt(1)
        wk = w.node().kind()
        one = None
        if wk in ("my_ops::BroadcastSrcNodeType", "my_ops::BroadcastDstNodeType"):
            need = "my_ops::BroadcastSrcNode" if "Src" in wk else "my_ops::BroadcastDstNode"
            if x.node().kind() != need:
                return False
            nd = x.node().inputsAt(0)
            flat = self.make("aten::squeeze", [nd], n, NODE)
            mm = self.make("my_ops::SegmentMMNode", [flat, w.node().inputsAt(0), self.dglgraph], n, NODE)
            wide = self.make(need, [mm, self.dglgraph], n, EDGE)
            one = self.const(1, n)
            out = self.make("aten::unsqueeze", [wide, one], n, EDGE)
        elif wk in ("my_ops::BroadcastEdgeType", "my_ops::BroadcastNodeType"):
            seg = "my_ops::SegmentMMEdge" if wk.endswith("EdgeType") else "my_ops::SegmentMMNode"
            r = EDGE if wk.endswith("EdgeType") else NODE
            if self.where(x) != r:
                return False
            flat = self.make("aten::squeeze", [x], n, r)
            mm = self.make(seg, [flat, w.node().inputsAt(0), self.dglgraph], n, r)
            one = self.const(1, n)
            out = self.make("aten::unsqueeze", [mm, one], n, r)
        else:
            return False
        n.output().replaceAllUsesWith(out)
        n.destroy()
        return True

    def _fuse_gat_chain(self, n) -> bool:
        """gspmm_src_mul_e_sum(z, SegmentSoftmax(leaky_relu(u_add_v(el, er)))) with
        no other reader of the intermediates -> gat_aggregate(el, er, z, slope)."""
        z, att = n.inputsAt(0), n.inputsAt(1)
        sm = att.node()
        if sm.kind() != "my_ops::SegmentSoftmax" or not self.single_use(att):
            return False
        act = sm.inputsAt(0).node()
        if act.kind() not in ("aten::leaky_relu", "aten::leaky_relu_") or \
                not self.single_use(act.output()):
            return False
        add = act.inputsAt(0).node()
        if add.kind() != "my_ops::gsddmm_u_add_v_mul_alpha" or not self.single_use(add.output()):
            return False
        slope = self.const_of(act.inputsAt(1))
        if slope is None:
            return False
        slope_v = self.const(float(slope), n)
        out = self.make("my_ops::gat_aggregate",
                        [add.inputsAt(0), add.inputsAt(1), z, slope_v, self.dglgraph], n, NODE)
        n.output().replaceAllUsesWith(out)
        for dead in (n, sm, act, add):      # the in-place activation would not be swept
            dead.destroy()
        return True


    def _fuse_gat_project(self, n) -> bool:
        """gat_aggregate(mm(z, w_src), mm(z, w_dst), z = mm(h, fc), ...) with node
        data h and shared weights -> (z, el, er) = gat_project(h, fc, w_src, w_dst):
        the projection and both attention products in one operator."""
        el, er, z = n.inputsAt(0).node(), n.inputsAt(1).node(), n.inputsAt(2).node()
        if z.kind() in ("aten::view", "aten::reshape"):
            return self._fuse_gat_project_heads(n)
        if not (el.kind() == er.kind() == z.kind() == "aten::mm"):
            return False
        if el.inputsAt(0).unique() != z.output().unique() or \
                er.inputsAt(0).unique() != z.output().unique():
            return False
        h, fc = z.inputsAt(0), z.inputsAt(1)
        w_s, w_d = el.inputsAt(1), er.inputsAt(1)
        if self.where(h) != NODE or any(self.where(v) != SHARED for v in (fc, w_s, w_d)):
            return False
        # the weights must be defined before the place the product is computed
        def depends_on(v, target, depth=0) -> bool:
            node = v.node()
            if node.kind() == "prim::Param" or depth > 32:
                return False
            return node is target or node == target or \
                any(depends_on(i, target, depth + 1) for i in node.inputs())

        def hoist(v):
            node = v.node()
            if node.kind() == "prim::Param" or node.isBefore(z):
                return
            for i in node.inputs():
                hoist(i)
            node.moveBefore(z)

        if depends_on(w_s, z) or depends_on(w_d, z):
            return False
        hoist(w_s)
        hoist(w_d)
        node = self.G.create("my_ops::gat_project", [h, fc, w_s, w_d], 3)
        node.insertBefore(z)
        for o in node.outputs():
            o.setType(torch._C.TensorType.get())
            self.res[o.unique()] = NODE
        outs = list(node.outputs())
        z.output().replaceAllUsesWith(outs[0])
        el.output().replaceAllUsesWith(outs[1])
        er.output().replaceAllUsesWith(outs[2])
        for dead in (el, er, z):
            dead.destroy()
        return True


    def _fuse_gat_project_heads(self, n) -> bool:
        """Multi-head form: gat_aggregate(sum(zv * a_l, [2], True), sum(zv * a_r, [2],
        True), zv = view(mm(h, fc), [-1, H, D]), ...) with shared (.., H, D) attention
        vectors -> (zv, el, er) = gat_project_heads(h, fc, a_l, a_r): one operator for
        the projection and the per-head attention terms."""
        el, er, zv = n.inputsAt(0).node(), n.inputsAt(1).node(), n.inputsAt(2).node()
        shape = self.const_of(zv.inputsAt(1))
        mm = zv.inputsAt(0).node()
        if mm.kind() != "aten::mm" or not isinstance(shape, list) or len(shape) != 3 \
                or shape[0] != -1 or not self.single_use(mm.output()):
            return False
        h, fc = mm.inputsAt(0), mm.inputsAt(1)
        if self.where(h) != NODE or self.where(fc) != SHARED:
            return False
        vecs = []
        for t in (el, er):
            if t.kind() != "aten::sum" or t.inputsSize() != 4 or \
                    self.const_of(t.inputsAt(1)) != [2] or self.const_of(t.inputsAt(2)) is not True \
                    or not self.single_use(t.output()):
                return False
            mul = t.inputsAt(0).node()
            if mul.kind() != "aten::mul" or not self.single_use(mul.output()):
                return False
            a, b = mul.inputsAt(0), mul.inputsAt(1)
            if a.unique() == zv.output().unique() and self.where(b) == SHARED:
                vecs.append((b, mul))
            elif b.unique() == zv.output().unique() and self.where(a) == SHARED:
                vecs.append((a, mul))
            else:
                return False
        # the attention vectors must already exist where the product is computed
        for v, _ in vecs:
            if v.node().kind() != "prim::Param" and not v.node().isBefore(mm):
                return False
        heads, dim = self.const(int(shape[1]), mm), self.const(int(shape[2]), mm)
        node = self.G.create("my_ops::gat_project_heads",
                             [h, fc, vecs[0][0], vecs[1][0], heads, dim], 3)
        node.insertBefore(mm)
        for o in node.outputs():
            o.setType(torch._C.TensorType.get())
            self.res[o.unique()] = NODE
        outs = list(node.outputs())
        zv.output().replaceAllUsesWith(outs[0])
        el.output().replaceAllUsesWith(outs[1])
        er.output().replaceAllUsesWith(outs[2])
        for dead in (el, er, vecs[0][1], vecs[1][1], zv, mm):
            dead.destroy()
        # with a_l at hand the aggregation can skip a large table of source terms
        agg = self.make("my_ops::gat_aggregate_al",
                        [vecs[0][0], outs[1], outs[2], outs[0], n.inputsAt(3), self.dglgraph],
                        n, NODE)
        n.output().replaceAllUsesWith(agg)
        n.destroy()
        return True

    # ------------------------------------------------- late fusion ----
    def late_fusion(self) -> bool:
        """Rewrites that remove per-edge copies of node rows and per-edge product
        tensors; run once the other passes have settled, because they consume the
        Broadcast nodes those passes match on."""
        changed = False
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::SegmentMMEdge":
                changed |= self._fuse_gather_mm(n)
        for n in list(self.G.nodes()):
            if n.kind() == "aten::sum":
                changed |= self._fuse_mm_dot(n)
        for n in list(self.G.nodes()):
            if n.kind() == "aten::mul":
                changed |= self._fuse_dot_scale(n)
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::SpMMEdge":
                changed |= self._fuse_e_mul_e(n)
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::gspmm_e_mul_e_sum":
                changed |= self._fuse_softmax_sum(n)
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::gspmm_e_mul_e_sum":
                changed |= self._fuse_row_scale(n)
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::SpMMEdge":
                changed |= self._fuse_typed_spmm(n)
        for n in list(self.G.nodes()):
            if n.kind() == "aten::mul":
                changed |= self._fuse_node_scale(n)
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::SegmentMMNodeScaled":
                changed |= self._fuse_type_gate(n)
        for n in list(self.G.nodes()):
            if n.kind() == "my_ops::edge_softmax_sum":
                changed |= self._fuse_pair_attention(n)
        changed |= self._fuse_stacked_mm()
        # last: only the sums no other rewrite has taken
        for n in list(self.G.nodes()):
            if n.kind() in ("aten::relu", "aten::elu"):
                changed |= self._fuse_spmm_tail(n)
        for n in list(self.G.nodes()):
            if n.kind() == "aten::mul":
                changed |= self._fuse_spmm_tail(n)
        return changed

    def _fuse_spmm_tail(self, n) -> bool:
        """relu | elu (SpMMSrc | SpMMEdge (x) [* s]) and SpMMSrc | SpMMEdge (x) * s, s
        a per-node tensor -> SpMMScaled(x, s, activation, edge_rows): what follows the
        sum row by row is applied where the sum is stored (GCN's
        `torch.relu(torch.sum(mailbox, 1))`).  The operator multiplies afterwards when
        s is not one fp32 number per row."""
        act, tail, top = 0, [], n.inputsAt(0)
        if n.kind() == "aten::relu":
            act = 1
        elif n.kind() == "aten::elu":
            if any(self.const_of(n.inputsAt(i)) not in (1, 1.0) for i in (1, 2, 3)):
                return False
            act = 2
        if act:
            if not self.single_use(top) or _mutated(top):
                return False
            mul = top.node() if top.node().kind() == "aten::mul" else None
        else:
            mul = n
        scale, summed = None, top
        if mul is not None:
            for a, b in ((mul.inputsAt(0), mul.inputsAt(1)), (mul.inputsAt(1), mul.inputsAt(0))):
                if a.node().kind() in ("my_ops::SpMMSrc", "my_ops::SpMMEdge") and \
                        isinstance(b.type(), torch._C.TensorType) and self.where(b) == NODE:
                    scale, summed = b, a
                    break
            else:
                return False
            if mul is not n:
                tail.append(mul)
        sp = summed.node()
        if sp.kind() not in ("my_ops::SpMMSrc", "my_ops::SpMMEdge") or \
                not self.single_use(summed) or _mutated(summed):
            return False
        out = self.make("my_ops::SpMMScaled",
                        [sp.inputsAt(0), scale if scale is not None else self.const(None, n),
                         self.const(act, n), self.const(sp.kind().endswith("Edge"), n),
                         self.dglgraph], n, NODE)
        n.output().replaceAllUsesWith(out)
        for dead in [n] + tail + [sp]:
            dead.destroy()
        return True

    def _fuse_gather_mm(self, n) -> bool:
        """SegmentMMEdge(BroadcastSrcNode | BroadcastDstNode (x), w) ->
        SegmentMMEdgeGather(x, w, endpoint): the product reads the node rows
        through the COO column."""
        bc = n.inputsAt(0).node()
        if bc.kind() not in ("my_ops::BroadcastSrcNode", "my_ops::BroadcastDstNode"):
            return False
        which = self.const(0 if bc.kind().endswith("SrcNode") else 1, n)
        out = self.make("my_ops::SegmentMMEdgeGather",
                        [bc.inputsAt(0), n.inputsAt(1), which, self.const(None, n), self.dglgraph],
                        n, EDGE)
        n.output().replaceAllUsesWith(out)
        n.destroy()
        return True

    def _fuse_mm_dot(self, n) -> bool:
        """sum(SegmentMMEdgeGather(x, w, i) * Broadcast{Src,Dst}Node(q), [1], keepdim=True)
        -> SegmentMMEdgeDot(x, w, i, q, j).  The typed products in a plan come
        from bmm (_fuse_bmm), so w is (T, K, M), one head, and the (E, 1) result
        of the sum is the operator's (E, heads) result."""
        if n.inputsSize() != 4 or self.const_of(n.inputsAt(1)) != [1] \
                or self.const_of(n.inputsAt(2)) is not True \
                or n.inputsAt(3).node().kind() != "prim::Constant" \
                or n.inputsAt(3).toIValue() is not None:
            return False
        mul = n.inputsAt(0).node()
        if mul.kind() != "aten::mul" or not self.single_use(mul.output()):
            return False
        for a, b in ((mul.inputsAt(0), mul.inputsAt(1)), (mul.inputsAt(1), mul.inputsAt(0))):
            mm, bc = a.node(), b.node()
            if mm.kind() == "my_ops::SegmentMMEdgeGather" and self.single_use(a) and \
                    bc.kind() in ("my_ops::BroadcastSrcNode", "my_ops::BroadcastDstNode"):
                # only the product this docstring describes: no per-row factor (the
                # dot has no place for one) and one head -- with (T, H, K, M) weights
                # the sum over dim 1 runs over heads * M, not per head
                scale = mm.inputsAt(3)
                if scale.node().kind() != "prim::Constant" or \
                        not isinstance(scale.type(), torch._C.NoneType):
                    continue
                # (typed products in a plan come from bmm, whose operands are 3-D; a
                # weight whose rank is known must say the same)
                w_type = mm.inputsAt(1).type()
                if isinstance(w_type, torch._C.TensorType) and w_type.dim() not in (None, 3):
                    continue
                which = self.const(0 if bc.kind().endswith("SrcNode") else 1, n)
                out = self.make("my_ops::SegmentMMEdgeDot",
                                [mm.inputsAt(0), mm.inputsAt(1), mm.inputsAt(2),
                                 bc.inputsAt(0), which, self.const(None, n), self.dglgraph],
                                n, EDGE)                 # (the product's row factor is None here)
                n.output().replaceAllUsesWith(out)
                n.destroy()
                return True
        return False

    def _fuse_dot_scale(self, n) -> bool:
        """SegmentMMEdgeDot(..., scale=None) * BroadcastEdgeType(p) with p one value
        per type (the dot has one head, see _fuse_mm_dot) -> the factor goes into
        the operator's per-type scale table."""
        for a, b in ((n.inputsAt(0), n.inputsAt(1)), (n.inputsAt(1), n.inputsAt(0))):
            dot, bc = a.node(), b.node()
            if dot.kind() == "my_ops::SegmentMMEdgeDot" and self.single_use(a) and \
                    dot.inputsAt(5).node().kind() == "prim::Constant" and \
                    dot.inputsAt(5).toIValue() is None and \
                    isinstance(dot.inputsAt(5).type(), torch._C.NoneType) and \
                    bc.kind() == "my_ops::BroadcastEdgeType":
                ins = list(dot.inputs())
                ins[5] = bc.inputsAt(0)
                out = self.make("my_ops::SegmentMMEdgeDot", ins, n, EDGE)
                n.output().replaceAllUsesWith(out)
                n.destroy()
                return True
        return False

    def _fuse_row_scale(self, n) -> bool:
        """gspmm_e_mul_e_sum(SegmentMMEdgeGather(x, w, i, None), s) with s read from
        the edge data (a stored per-edge tensor such as RGCN's norm, not something
        computed in the plan) -> SpMMEdge(SegmentMMEdgeGather(x, w, i, s)): the
        factor is applied where the rows are produced, in edge order, instead of
        being gathered through the edge ids by the reduction.  The operator
        multiplies afterwards when s is not one float per edge."""
        for a, b in ((n.inputsAt(0), n.inputsAt(1)), (n.inputsAt(1), n.inputsAt(0))):
            mm, sc = a.node(), b.node()
            if mm.kind() == "my_ops::SegmentMMEdgeGather" and self.single_use(a) and \
                    mm.inputsAt(3).node().kind() == "prim::Constant" and \
                    isinstance(mm.inputsAt(3).type(), torch._C.NoneType) and \
                    sc.kind() == "aten::__getitem__" and self.where(b) == EDGE:
                ins = list(mm.inputs())
                ins[3] = b
                prod = self.make("my_ops::SegmentMMEdgeGather", ins, n, EDGE)
                with self.G.insert_point_guard(n):
                    dims = self.G.insertConstant([1])
                    keep = self.G.insertConstant(False)
                    none = self.G.insertConstant(None)
                out = self.make("my_ops::SpMMEdge", [prod, dims, keep, none, self.dglgraph], n, NODE)
                n.output().replaceAllUsesWith(out)
                n.destroy()
                return True
        return False

    def _fuse_softmax_sum(self, n) -> bool:
        """gspmm_e_mul_e_sum(SegmentSoftmax(x), m) with no other reader of the
        attention -> edge_softmax_sum(x, m): softmax and weighted sum in one pass."""
        for a, b in ((n.inputsAt(0), n.inputsAt(1)), (n.inputsAt(1), n.inputsAt(0))):
            sm = a.node()
            if sm.kind() == "my_ops::SegmentSoftmax" and self.single_use(a):
                out = self.make("my_ops::edge_softmax_sum",
                                [sm.inputsAt(0), b, self.dglgraph], n, NODE)
                n.output().replaceAllUsesWith(out)
                n.destroy()
                sm.destroy()
                return True
        return False

    def _fuse_e_mul_e(self, n) -> bool:
        """SpMMEdge(a * b) with both operands per-edge -> gspmm_e_mul_e_sum(a, b):
        the product tensor is not formed (the operator multiplies first itself
        when neither operand is a per-edge weight)."""
        mul = n.inputsAt(0).node()
        if mul.kind() != "aten::mul" or not self.single_use(mul.output()):
            return False
        a, b = mul.inputsAt(0), mul.inputsAt(1)
        if self.where(a) != EDGE or self.where(b) != EDGE:
            return False
        if not (isinstance(a.type(), torch._C.TensorType) and isinstance(b.type(), torch._C.TensorType)):
            return False
        out = self.make("my_ops::gspmm_e_mul_e_sum", [a, b, self.dglgraph], n, NODE)
        n.output().replaceAllUsesWith(out)
        n.destroy()
        return True


    def _fuse_typed_spmm(self, n) -> bool:
        """SpMMEdge(SegmentMMEdgeGather(x, w, 0, s)) -> TypedSpMMEdge(x, w, s): the
        message and reduce steps of an RGCN layer as one operator, which runs them
        in one pass over destination tiles where that is the faster kernel."""
        mm = n.inputsAt(0).node()
        if mm.kind() != "my_ops::SegmentMMEdgeGather" or not self.single_use(n.inputsAt(0)):
            return False
        if self.const_of(mm.inputsAt(2)) != 0:
            return False
        out = self.make("my_ops::TypedSpMMEdge",
                        [mm.inputsAt(0), mm.inputsAt(1), mm.inputsAt(3), self.dglgraph], n, NODE)
        n.output().replaceAllUsesWith(out)
        n.destroy()
        mm.destroy()
        return True

    def _fuse_pair_attention(self, n) -> bool:
        """edge_softmax_sum(SegmentMMEdgeDot(k, A, src, q, dst, s) [/ c],
        SegmentMMEdgeGather(v, M, src)) -> relation_pair_attention(k, q, v, A, M, s, c):
        HGT's message and reduce stages as one operator, which applies the relation
        matrices per (destination, relation) pair where the graph has such pairs and
        runs these three operators otherwise."""
        score, msg = n.inputsAt(0).node(), n.inputsAt(1).node()
        if msg.kind() != "my_ops::SegmentMMEdgeGather" or not self.single_use(n.inputsAt(1)) \
                or self.const_of(msg.inputsAt(2)) != 0 \
                or msg.inputsAt(3).node().kind() != "prim::Constant" \
                or not isinstance(msg.inputsAt(3).type(), torch._C.NoneType):
            return False
        divisor, div = None, None
        if score.kind() == "aten::div" and self.single_use(n.inputsAt(0)) \
                and score.inputsSize() == 2 \
                and isinstance(score.inputsAt(1).type(), torch._C.FloatType):
            div, divisor = score, score.inputsAt(1)
            score = score.inputsAt(0).node()
            if not self.single_use(div.inputsAt(0)):
                return False
        elif not self.single_use(n.inputsAt(0)):
            return False
        if score.kind() != "my_ops::SegmentMMEdgeDot" or self.const_of(score.inputsAt(2)) != 0 \
                or self.const_of(score.inputsAt(4)) != 1:
            return False
        if divisor is None:
            divisor = self.const(1.0, n)
        out = self.make("my_ops::relation_pair_attention",
                        [score.inputsAt(0), score.inputsAt(3), msg.inputsAt(0), score.inputsAt(1),
                         msg.inputsAt(1), score.inputsAt(5), divisor, self.dglgraph], n, NODE)
        n.output().replaceAllUsesWith(out)
        n.destroy()
        if div is not None:
            div.destroy()
        score.destroy()
        msg.destroy()
        return True

    def _fuse_node_scale(self, n) -> bool:
        """SegmentMMNode(x, w) * BroadcastNodeType(s) -> SegmentMMNodeScaled(x, w,
        BroadcastNodeType(s)): the per-node factor is applied to the product's fp32 sums
        (HGT's gate on the output projection).  The operator itself falls back to the
        two steps when the factor is not (N, 1) or would promote the result."""
        for a, b in ((n.inputsAt(0), n.inputsAt(1)), (n.inputsAt(1), n.inputsAt(0))):
            mm, bc = a.node(), b.node()
            if mm.kind() == "my_ops::SegmentMMNode" and self.single_use(a) and \
                    bc.kind() == "my_ops::BroadcastNodeType":
                out = self.make("my_ops::SegmentMMNodeScaled",
                                [mm.inputsAt(0), mm.inputsAt(1), b, self.dglgraph], n, NODE)
                n.output().replaceAllUsesWith(out)
                n.destroy()
                mm.destroy()
                return True
        return False

    def _fuse_type_gate(self, n) -> bool:
        """SegmentMMNodeScaled(x, w, BroadcastNodeType(unsqueeze([sigmoid](s), 1))) ->
        SegmentMMNodeGated(x, w, s, sigmoid): a factor that is one number per node type
        needs neither the sigmoid nor its copy to the nodes as operators of their own
        (HGT's `trans_out * sigmoid(skip)[ntype]`)."""
        bc = n.inputsAt(2).node()
        if bc.kind() != "my_ops::BroadcastNodeType" or not self.single_use(n.inputsAt(2)):
            return False
        un = bc.inputsAt(0).node()
        if un.kind() != "aten::unsqueeze" or self.const_of(un.inputsAt(1)) not in (1, -1) \
                or not self.single_use(bc.inputsAt(0)):
            return False
        gate, sig = un.inputsAt(0), None
        if gate.node().kind() == "aten::sigmoid" and self.single_use(gate) and not _mutated(gate):
            sig = gate.node()
            gate = sig.inputsAt(0)
        if self.where(gate) != NTYPE or _mutated(gate):
            return False
        out = self.make("my_ops::SegmentMMNodeGated",
                        [n.inputsAt(0), n.inputsAt(1), gate, self.const(sig is not None, n),
                         self.dglgraph], n, NODE)
        n.output().replaceAllUsesWith(out)
        for dead in (n, bc, un) + ((sig,) if sig is not None else ()):
            dead.destroy()
        return True

    def _fuse_stacked_mm(self) -> bool:
        """Two to four SegmentMMNode(x, w_i) of one x -> SegmentMMNodeStacked(x, [w_i]):
        the rows of x are read once (HGT's K, Q, V projections).  The stacked node
        takes the place of the last product of the group (every weight is defined
        by then), so a product joins only while nothing reads an earlier result
        before that place."""
        groups = {}
        for n in self.G.nodes():
            if n.kind() == "my_ops::SegmentMMNode":
                groups.setdefault(n.inputsAt(0).unique(), []).append(n)
        changed = False
        for nodes in groups.values():
            # an input or a result that an in-place operator overwrites somewhere is not
            # one value over the whole group: such products stay where they are
            nodes = [n for n in nodes if not (_mutated(n.inputsAt(0)) or _mutated(n.inputsAt(1))
                                              or _mutated(n.output()))]
            nodes = nodes[:4]
            while len(nodes) >= 2:
                last = nodes[-1]
                if all(u.user.isAfter(last) for n in nodes[:-1] for u in n.output().uses()):
                    break
                nodes = nodes[:-1]
            if len(nodes) < 2:
                continue
            last = nodes[-1]
            tensor = torch._C.TensorType.get()
            lst = self.G.create("prim::ListConstruct", [n.inputsAt(1) for n in nodes], 1)
            lst.insertBefore(last)
            lst.output().setType(torch._C.ListType(tensor))
            st = self.G.create("my_ops::SegmentMMNodeStacked",
                               [last.inputsAt(0), lst.output(), self.dglgraph], 1)
            st.insertBefore(last)
            st.output().setType(torch._C.ListType(tensor))
            un = self.G.create("prim::ListUnpack", [st.output()], len(nodes))
            un.insertBefore(last)
            for n, o in zip(nodes, un.outputs()):
                o.setType(n.output().type())
                self.res[o.unique()] = NODE
                n.output().replaceAllUsesWith(o)
                n.destroy()
            changed = True
        return changed


def split(plan: MPDFG) -> None:
    _Rewriter(plan).split()
    dedup(plan.graph)
    plan.invalidate()


def reorder(plan: MPDFG) -> None:
    rw = _Rewriter(plan)
    for _ in range(16):
        if not rw.reorder():
            break
        dedup(plan.graph)
    dedup(plan.graph)
    plan.invalidate()


def fusion(plan: MPDFG) -> None:
    rw = _Rewriter(plan)
    for _ in range(8):
        if not rw.fusion():
            break
        dedup(plan.graph)
    dedup(plan.graph)
    plan.invalidate()


def optimize(plan: MPDFG, opt_level: int) -> None:
    """python/graphiler/mpdfg_optimizer.py:4-16: level 1 = split + reorder,
    level 2 = + alternating reorder / fusion until nothing changes."""
    if opt_level <= 0:
        return
    split(plan)
    reorder(plan)
    if opt_level > 1:
        for _ in range(3):
            reorder(plan)
            fusion(plan)
        rw = _Rewriter(plan)
        for _ in range(4):
            if not rw.late_fusion():
                break
            dedup(plan.graph)
        plan.invalidate()
