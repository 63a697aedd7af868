"""Message-passing data-flow graph (MP-DFG) builder.

Takes the scripted message / reduce / update functions of a model and stitches
them into ONE TorchScript graph over ``(DGLGraph, ndata, edata, ntypedata,
etypedata, *parameters)`` in which every graph-dependent step is an explicit
``my_ops::*`` operator — the job of src/builder/builder.cpp:44-371 and
python/graphiler/mpdfg_builder.py:35-75, done here through TorchScript's Python
graph API on a freshly created graph (no source template, no temporary file).

Every value carries a *residency* (where its rows live): node, edge, node-type,
edge-type, or shared (parameters and constants).  Rules (builder.cpp:55-291):

* ``edges.src[k]`` / ``edges.dst[k]`` -> ``ndata[k]`` + ``BroadcastSrcNode`` /
  ``BroadcastDstNode``; ``edges.srctype[k]`` / ``edges.dsttype[k]`` ->
  ``ntypedata[k]`` + ``BroadcastSrcNodeType`` / ``BroadcastDstNodeType``;
  ``edges.type[k]`` -> ``etypedata[k]`` + ``BroadcastEdgeType``; ``edges.data[k]``
  -> ``edata[k]``; ``nodes.type[k]`` -> ``ntypedata[k]`` + ``BroadcastNodeType``;
  ``nodes.data[k]`` -> ``ndata[k]``; ``nodes.mailbox[k]`` -> the value the message
  function returned under ``k``.
* in the reduce function ``softmax(x, dim=1)`` of an edge value becomes
  ``SegmentSoftmax`` and ``sum(x, dim=[1])`` becomes ``SpMMEdge``
  (builder.cpp:24-42): the mailbox dimension of DGL's degree-bucketed batches is
  the segment of in-edges here.
* everything else is copied; its result lives where its non-shared inputs live.
* with an update function the reduce function's outputs are stored into
  ``ndata`` (``aten::_set_item``) so the update function reads them back.
"""
from __future__ import annotations

import inspect
from typing import Callable, Dict, List, Optional

import torch

from .. import torch_boundary
from .batch import EdgeBatchDummy, NodeBatchDummy

NODE, EDGE, NTYPE, ETYPE, SHARED = "node", "edge", "ntype", "etype", "shared"

# field of the batch object -> (which plan input holds it, broadcast to apply)
_EDGE_FIELDS = {
    "f_src": ("ndata", "src"), "f_dst": ("ndata", "dst"), "f_edge": ("edata", None),
    "f_srctype": ("ntypedata", "src"), "f_dsttype": ("ntypedata", "dst"),
    "f_edgetype": ("etypedata", "type"),
}
_NODE_FIELDS = {
    "f_mail": ("mail", None), "f_node": ("ndata", None), "f_nodetype": ("ntypedata", "type"),
}


class BuildError(RuntimeError):
    pass


def _plan_input_types():
    """Types of the five fixed plan inputs, taken from a scripted stub."""
    torch_boundary.load()

    def stub(g: torch.classes.my_classes.DGLGraph, d: Dict[str, torch.Tensor]):
        return d

    ins = list(torch.jit.script(stub).graph.inputs())
    return ins[0].type(), ins[1].type()


class MPDFG:
    """A compiled plan: ``forward(DGLGraph, ndata, edata, ntypedata, etypedata,
    *msg_params, *reduce_params, *update_params) -> Dict[str, Tensor]``."""

    def __init__(self, graph: torch._C.Graph, residency: Dict[int, str]):
        self.graph = graph
        self.residency = residency
        self._fn = None

    @property
    def forward(self):
        if self._fn is None:
            self.graph.lint()
            self._fn = torch._C._create_function_from_graph("mpdfg_func", self.graph)
        return self._fn

    def op_kinds(self) -> List[str]:
        return [n.kind() for n in self.graph.nodes()]

    def invalidate(self):
        self._fn = None


class _Stage:
    def __init__(self, name: str, func: Callable, batch_cls):
        self.name = name
        sig = list(inspect.signature(func).parameters.values())
        if not sig or sig[0].annotation is not batch_cls:
            raise BuildError(f"the first parameter of the {name} function must be annotated "
                             f"{batch_cls.__name__}")
        self.graph = torch.jit.script(func).inlined_graph
        torch._C._jit_pass_inline(self.graph)
        # folds the constant branches library wrappers carry (F.leaky_relu's
        # `if inplace:`), leaving straight-line code
        torch._C._jit_pass_constant_propagation(self.graph)
        torch._C._jit_pass_dce(self.graph)
        self.params = list(self.graph.inputs())


def _const_of(value):
    """Python value of a constant (ints, floats, strings, lists of ints), or None."""
    iv = value.toIValue()
    if iv is not None:
        return iv
    node = value.node()
    if node.kind() == "prim::ListConstruct":
        items = [_const_of(i) for i in node.inputs()]
        return None if any(i is None for i in items) else items
    return None


class _Builder:
    def __init__(self, stages: List[_Stage]):
        g_type, dict_type = _plan_input_types()
        self.G = torch._C.Graph()
        self.residency: Dict[int, str] = {}
        self.inputs = {}
        for name, ty, res in (("dglgraph", g_type, SHARED), ("ndata", dict_type, NODE),
                              ("edata", dict_type, EDGE), ("ntypedata", dict_type, NTYPE),
                              ("etypedata", dict_type, ETYPE)):
            v = self.G.addInput()
            v.setType(ty)
            v.setDebugName(name)
            self.inputs[name] = v
            self.residency[v.unique()] = res
        self.mailbox: Dict[str, torch._C.Value] = {}
        self.stages = stages
        # extra parameters of every stage become plan inputs, in stage order
        self.param_maps = []
        for st in stages:
            pm = {}
            for p in st.params[1:]:
                v = self.G.addInput()
                v.setType(p.type())
                v.setDebugName(f"{p.debugName().split('.')[0]}_{st.name}")
                self.residency[v.unique()] = SHARED
                pm[p.unique()] = v
            self.param_maps.append(pm)

    # -- helpers --------------------------------------------------------------
    def _emit(self, kind: str, inputs, like=None, n_out: int = 1):
        node = self.G.create(kind, list(inputs), n_out)
        if like is not None:
            node.copyAttributes(like)
            for o_new, o_old in zip(node.outputs(), like.outputs()):
                o_new.copyMetadata(o_old)
        self.G.insertNode(node)
        return node

    def _graph_op(self, kind: str, inputs, residency: str):
        node = self._emit(kind, list(inputs) + [self.inputs["dglgraph"]])
        node.output().setType(torch._C.TensorType.get())
        self.residency[node.output().unique()] = residency
        return node.output()

    def _res(self, v) -> str:
        return self.residency.get(v.unique(), SHARED)

    # -- one UDF --------------------------------------------------------------
    def run_stage(self, idx: int, last: bool):
        st = self.stages[idx]
        creation = st.name == "msg"
        fields = _EDGE_FIELDS if creation else _NODE_FIELDS
        vmap = dict(self.param_maps[idx])          # UDF value id -> plan value
        dict_bcast = {}                            # UDF dict value id -> broadcast kind
        mail_dicts = set()
        batch_id = st.params[0].unique()
        ret = st.graph.return_node()
        if ret.inputsSize() != 1:
            raise BuildError(f"the {st.name} function must return one dict")
        final = ret.input().node()
        for n in st.graph.nodes():
            kind = n.kind()
            if len(list(n.blocks())):
                raise BuildError(f"control flow ({kind}) in a user function is not supported")
            if kind == "prim::GetAttr" and n.input().unique() == batch_id:
                field = n.s("name")
                if field not in fields:
                    raise BuildError(f"unknown batch field {field}")
                source, bcast = fields[field]
                if source == "mail":
                    mail_dicts.add(n.output().unique())
                else:
                    vmap[n.output().unique()] = self.inputs[source]
                    if bcast:
                        dict_bcast[n.output().unique()] = bcast
                continue
            if kind == "aten::__getitem__" and n.inputsAt(0).unique() in mail_dicts:
                key = _const_of(n.inputsAt(1))
                if key not in self.mailbox:
                    raise BuildError(f"the reduce function reads mailbox[{key!r}] but the message "
                                     f"function returns {sorted(self.mailbox)}")
                vmap[n.output().unique()] = self.mailbox[key]
                continue
            try:
                ins = [vmap[i.unique()] for i in n.inputs()]
            except KeyError:
                raise BuildError(f"{kind} uses a value the builder cannot place "
                                 "(is the batch object passed on?)") from None
            res = [self._res(v) for v in ins]

            if n is final:
                if kind != "prim::DictConstruct":
                    raise BuildError(f"the {st.name} function must return a dict literal")
                keys = [_const_of(k) for k in ins[0::2]]
                if creation:
                    self.mailbox = dict(zip(keys, ins[1::2]))
                    continue
                if not last:          # results become node data for the update function
                    for k, v in zip(ins[0::2], ins[1::2]):
                        self._emit("aten::_set_item", [self.inputs["ndata"], k, v], n_out=0)
                    continue
                out = self._emit(kind, ins, like=n).output()
                self.G.registerOutput(out)
                continue

            # lowering of the two mailbox reductions (builder.cpp:24-42)
            if st.name == "reduce" and res and res[0] == EDGE:
                if kind == "aten::softmax" and _const_of(n.inputsAt(1)) == 1:
                    vmap[n.output().unique()] = self._graph_op("my_ops::SegmentSoftmax", ins, EDGE)
                    continue
                if kind == "aten::sum" and n.inputsSize() == 4 and _const_of(n.inputsAt(1)) == [1]:
                    vmap[n.output().unique()] = self._graph_op("my_ops::SpMMEdge", ins, NODE)
                    continue
                if kind in ("aten::softmax", "aten::sum", "aten::mean", "aten::max", "aten::min"):
                    raise BuildError(f"{kind} over mailbox data is only supported along dim 1")

            new = self._emit(kind, ins, like=n, n_out=n.outputsSize())
            for o_old, o_new in zip(n.outputs(), new.outputs()):
                vmap[o_old.unique()] = o_new

            if kind == "aten::__getitem__" and n.inputsAt(0).unique() in dict_bcast:
                where = dict_bcast[n.inputsAt(0).unique()]
                typed = res[0] in (NTYPE, ETYPE)
                if where == "src":
                    op = "my_ops::BroadcastSrcNodeType" if typed else "my_ops::BroadcastSrcNode"
                elif where == "dst":
                    op = "my_ops::BroadcastDstNodeType" if typed else "my_ops::BroadcastDstNode"
                else:
                    op = "my_ops::BroadcastEdgeType" if creation else "my_ops::BroadcastNodeType"
                self.residency[new.output().unique()] = res[0]
                vmap[n.output().unique()] = self._graph_op(op, [new.output()],
                                                           EDGE if creation else NODE)
                continue
            # residency of a copied operator: that of its non-shared inputs
            live = {r for r in res if r != SHARED}
            if len(live) > 1:
                raise BuildError(f"{kind} mixes {sorted(live)} data; broadcast one side first")
            where = next(iter(live)) if live else SHARED
            for o in new.outputs():
                self.residency[o.unique()] = where


def mpdfg_builder(msg_func: Callable, reduce_func: Callable,
                  update_func: Optional[Callable] = None, opt_level: int = 2) -> MPDFG:
    """Compile a (message, reduce[, update]) triple into a plan
    (python/graphiler/mpdfg_builder.py:35-75).  ``opt_level`` 0: as written;
    1: + split / reorder; 2: + fusion into the graph operators' fused forms."""
    from . import passes
    stages = [_Stage("msg", msg_func, EdgeBatchDummy), _Stage("reduce", reduce_func, NodeBatchDummy)]
    if update_func is not None:
        stages.append(_Stage("update", update_func, NodeBatchDummy))
    b = _Builder(stages)
    for i in range(len(stages)):
        b.run_stage(i, last=i == len(stages) - 1)
    if not list(b.G.outputs()):
        raise BuildError("the plan has no output")
    plan = MPDFG(b.G, b.residency)
    passes.dedup(plan.graph)
    passes.optimize(plan, opt_level)
    return plan
