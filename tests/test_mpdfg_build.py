"""Structure of the plans the MP-DFG builder emits (no GPU needed: the plans are
built and linted, not run)."""
import pytest
import torch

from graphiler_amd.examples import udf as U
from graphiler_amd.mpdfg import BuildError, EdgeBatchDummy, NodeBatchDummy, mpdfg_builder

MODELS = {
    "gcn": (U.gcn_message, U.gcn_reduce),
    "gat": (U.gat_message, U.gat_reduce),
    "rgcn": (U.rgcn_message, U.rgcn_reduce),
    "hgt": (U.hgt_message, U.hgt_reduce, U.hgt_update),
}


def _kinds(name, level):
    plan = mpdfg_builder(*MODELS[name], opt_level=level)
    plan.forward                                    # lints and compiles
    return plan, [k for k in plan.op_kinds() if k.startswith(("my_ops::", "aten::"))]


def test_plan_signature_and_parameters():
    plan, _ = _kinds("gat", 0)
    names = [v.debugName() for v in plan.graph.inputs()]
    assert names[:5] == ["dglgraph", "ndata", "edata", "ntypedata", "etypedata"]
    assert names[5:] == ["fc_weight_msg", "attn_weight_msg"]
    plan, _ = _kinds("hgt", 0)
    assert [v.debugName() for v in plan.graph.inputs()][5:] == ["sqrt_dk_msg"]
    assert str(list(plan.graph.inputs())[5].type()) == "float"


def test_level0_is_broadcast_compute_reduce():
    """Unoptimised: every batch read is a Broadcast operator, the mailbox
    reductions are SegmentSoftmax / SpMMEdge (builder.cpp:24-42, 205-238)."""
    _, k = _kinds("gat", 0)
    assert k.count("my_ops::BroadcastSrcNode") == 1 and k.count("my_ops::BroadcastDstNode") == 1
    assert "aten::cat" in k and "my_ops::SegmentSoftmax" in k and "my_ops::SpMMEdge" in k
    assert k.index("my_ops::SegmentSoftmax") < k.index("my_ops::SpMMEdge")
    _, k = _kinds("hgt", 0)
    assert k.count("my_ops::BroadcastSrcNodeType") == 2 and k.count("my_ops::BroadcastDstNodeType") == 1
    assert k.count("my_ops::BroadcastEdgeType") == 3 and k.count("my_ops::BroadcastNodeType") == 2
    assert "aten::_set_item" in k               # reduce results stored for the update function
    _, k = _kinds("rgcn", 0)
    assert "my_ops::BroadcastEdgeType" in k and "aten::bmm" in k


def test_level1_moves_dense_work_to_the_nodes():
    _, k = _kinds("gat", 1)
    assert "aten::cat" not in k                                 # split
    assert k.index("aten::mm") < k.index("my_ops::BroadcastSrcNode")   # reorder
    assert k.count("aten::mm") == 3             # z once (source and destination share it), el, er
    assert "my_ops::get_feat_dim" not in k and "aten::size" in k   # slice width from the weight
    _, k = _kinds("gcn", 1)
    assert k.index("aten::mul") < k.index("my_ops::BroadcastSrcNode")
    assert k.count("my_ops::BroadcastSrcNode") == 1


def test_level2_fuses_into_graph_operators():
    _, k = _kinds("gcn", 2)
    # the relu of the reduce function rides on the sum's store
    assert [x for x in k if x.startswith("my_ops::")] == ["my_ops::SpMMScaled"]
    assert "aten::relu" not in k
    _, k = _kinds("gat", 2)
    ours = [x for x in k if x.startswith("my_ops::")]
    assert ours == ["my_ops::gat_project", "my_ops::gat_aggregate"]    # two kernels end to end
    assert "aten::mm" not in k
    _, k = _kinds("rgcn", 2)
    ours = [x for x in k if x.startswith("my_ops::")]
    # message and reduce as one operator: the source rows are read through the graph,
    # the norm is applied to the messages, and (where that kernel is the faster one) no
    # per-edge tensor is written at all
    assert ours == ["my_ops::TypedSpMMEdge"]
    assert "aten::bmm" not in k and "aten::mul" not in k
    _, k = _kinds("hgt", 2)
    ours = [x for x in k if x.startswith("my_ops::")]
    # K, V, Q in one pass over h; the output projection takes the gate as its row factor
    assert ours.count("my_ops::SegmentMMNodeStacked") == 1 and ours.count("my_ops::SegmentMMNode") == 0
    # ... and takes the gate per node type: no sigmoid, no copy of it to the nodes, no product
    assert ours == ["my_ops::SegmentMMNodeStacked", "my_ops::relation_pair_attention",
                    "my_ops::SegmentMMNodeGated"]
    assert not any(x in k for x in ("aten::mul", "aten::sigmoid", "aten::unsqueeze"))
    # scores, softmax and weighted sum of transformed values as one operator (it picks the
    # per-pair or the per-edge form from the graph it is given)
    assert ours.count("my_ops::relation_pair_attention") == 1 and "aten::div" not in ours
    assert not any(k in ours for k in ("my_ops::SegmentMMEdgeDot", "my_ops::SegmentMMEdgeGather",
                                       "my_ops::edge_softmax_sum"))
    assert "my_ops::SegmentSoftmax" not in ours and "my_ops::gspmm_e_mul_e_sum" not in ours
    assert not any(x in ("my_ops::BroadcastSrcNode", "my_ops::BroadcastDstNode",
                         "my_ops::SegmentMMEdge", "my_ops::SpMMEdge") for x in ours)
    assert "aten::bmm" not in k and "aten::squeeze" not in k and "aten::sum" not in k


def test_multi_head_attention_reaches_the_fused_kernel():
    """Four-head GAT written with view / per-head sums: the view, the products
    with the attention vectors and the in-row sums hop over the broadcasts to
    node data, and the chain fuses into gat_aggregate."""
    plan = mpdfg_builder(U.gat4_message, U.gat4_reduce, opt_level=2)
    k = plan.op_kinds()
    ours = [x for x in k if x.startswith("my_ops::")]
    assert ours == ["my_ops::gat_project_heads", "my_ops::gat_aggregate_al"]   # two kernels
    assert "aten::mm" not in k and "aten::view" not in k and "aten::sum" not in k
    plan1 = mpdfg_builder(U.gat4_message, U.gat4_reduce, opt_level=1).op_kinds()
    # at level 1 the per-head terms are already computed on node data
    assert plan1.index("aten::sum") < plan1.index("my_ops::BroadcastDstNode")


def gat_reference_style_message(edges: EdgeBatchDummy, fc_weight, attn_weight):
    z_s = torch.mm(edges.src['h'], fc_weight)
    z_d = torch.mm(edges.dst['h'], fc_weight)
    a = torch.mm(torch.cat([z_s, z_d], dim=1), attn_weight)
    return {'z': z_s, 'e': torch.nn.functional.leaky_relu_(a)}      # in place, default slope


def test_inplace_activation_chain_is_fused_and_removed():
    plan = mpdfg_builder(gat_reference_style_message, U.gat_reduce, opt_level=2)
    k = plan.op_kinds()
    assert "my_ops::gat_aggregate" in k and "aten::leaky_relu_" not in k
    assert "my_ops::gsddmm_u_add_v_mul_alpha" not in k


def reads_one_field_twice_message(edges: EdgeBatchDummy):
    x = edges.src['h']
    y = torch.relu_(edges.src['h'] + 0.0)      # a second read, overwritten in place afterwards
    z = torch.relu_(edges.src['h'])            # in place on the broadcast itself
    return {'m': x + y + z}


def test_value_numbering_keeps_reads_that_are_overwritten_apart():
    """Two equal graph operators are one value only while nothing writes to either
    result: the read that relu_ overwrites must not become the read that is used
    unchanged (level 0 runs only the value numbering)."""
    plan = mpdfg_builder(reads_one_field_twice_message, U.gcn_reduce, opt_level=0)
    plan.forward
    nodes = list(plan.graph.nodes())
    reads = [n for n in nodes if n.kind() == "my_ops::BroadcastSrcNode"]
    inplace = [n for n in nodes if n.kind() == "aten::relu_"]
    for r in inplace:
        target = r.inputsAt(0).node()
        if target.kind() == "my_ops::BroadcastSrcNode":
            # the overwritten read feeds the in-place operator only
            assert [u.user.kind() for u in target.output().uses()] == ["aten::relu_"]
    assert len(reads) >= 2 or not any(r.inputsAt(0).node().kind() == "my_ops::BroadcastSrcNode"
                                      for r in inplace)


def gcn_both_norms_reduce(nodes: NodeBatchDummy):
    summed = torch.sum(nodes.mailbox['m'], dim=1)
    return {'h': torch.nn.functional.elu(summed * nodes.data['norm'])}


def gcn_scaled_reduce(nodes: NodeBatchDummy):
    return {'h': nodes.data['norm'] * torch.sum(nodes.mailbox['m'], dim=1)}


def gcn_other_elu_reduce(nodes: NodeBatchDummy):
    return {'h': torch.nn.functional.elu(torch.sum(nodes.mailbox['m'], dim=1), 0.5)}


def gcn_sum_read_twice_reduce(nodes: NodeBatchDummy):
    summed = torch.sum(nodes.mailbox['m'], dim=1)
    return {'h': torch.relu(summed), 'raw': summed}


def gcn_inplace_reduce(nodes: NodeBatchDummy):
    return {'h': torch.relu_(torch.sum(nodes.mailbox['m'], dim=1))}


def _ours(reduce, level=2):
    plan = mpdfg_builder(U.gcn_message, reduce, opt_level=level)
    plan.forward
    return plan, [k for k in plan.op_kinds() if k.startswith(("my_ops::", "aten::"))]


def test_row_wise_tail_of_a_sum_joins_the_sum():
    """A destination-side factor and the activation after a neighbour sum become
    arguments of the sum; anything the operator cannot reproduce stays as it is."""
    plan, k = _ours(gcn_both_norms_reduce)
    assert "my_ops::SpMMScaled" in k and "aten::elu" not in k and "my_ops::SpMMSrc" not in k
    assert k.count("aten::mul") == 1                        # the message's own factor only
    node = [n for n in plan.graph.nodes() if n.kind() == "my_ops::SpMMScaled"][0]
    assert node.inputsAt(1).node().kind() == "aten::__getitem__"       # the stored norm
    assert node.inputsAt(2).toIValue() == 2 and node.inputsAt(3).toIValue() is False
    plan, k = _ours(gcn_scaled_reduce)
    assert "my_ops::SpMMScaled" in k and k.count("aten::mul") == 1
    node = [n for n in plan.graph.nodes() if n.kind() == "my_ops::SpMMScaled"][0]
    assert node.inputsAt(2).toIValue() == 0
    _, k = _ours(gcn_other_elu_reduce)                      # alpha = 0.5: not the operator's elu
    assert "my_ops::SpMMSrc" in k and "aten::elu" in k and "my_ops::SpMMScaled" not in k
    _, k = _ours(gcn_sum_read_twice_reduce)                 # the plain sum is an output too
    assert "my_ops::SpMMSrc" in k and "aten::relu" in k and "my_ops::SpMMScaled" not in k
    _, k = _ours(gcn_inplace_reduce)                        # relu_ is left alone
    assert "my_ops::SpMMSrc" in k and "aten::relu_" in k
    _, k = _ours(gcn_both_norms_reduce, level=1)            # level 1 does not fuse
    assert "my_ops::SpMMScaled" not in k


def bad_reduce(nodes: NodeBatchDummy):
    return {'h': torch.sum(nodes.mailbox['missing'], dim=1)}


def bad_softmax(nodes: NodeBatchDummy):
    return {'h': torch.sum(torch.softmax(nodes.mailbox['m'], dim=0), dim=1)}


def untyped_message(edges, w):
    return {'m': edges.src['h']}


def test_build_errors():
    with pytest.raises(BuildError, match="mailbox"):
        mpdfg_builder(U.gcn_message, bad_reduce)
    with pytest.raises(BuildError, match="dim 1"):
        mpdfg_builder(U.gcn_message, bad_softmax)
    with pytest.raises(BuildError, match="annotated"):
        mpdfg_builder(untyped_message, U.gcn_reduce)


# --- guards of single rewrites, on hand-written plans -------------------------------
_DOT_PLAN = """
graph(%g : __torch__.torch.classes.my_classes.DGLGraph, %x : Tensor, %w : WTYPE,
      %q : Tensor, %s : Tensor):
  %zero : int = prim::Constant[value=0]()
  %one : int = prim::Constant[value=1]()
  %true : bool = prim::Constant[value=1]()
  %none : NoneType = prim::Constant()
  %dims : int[] = prim::ListConstruct(%one)
  %y : Tensor = my_ops::SegmentMMEdgeGather(%x, %w, %zero, SCALE, %g)
  %b : Tensor = my_ops::BroadcastDstNode(%q, %g)
  %m : Tensor = aten::mul(%y, %b)
  %r : Tensor = aten::sum(%m, %dims, %true, %none)
  return (%r)
"""


def _late_fused_kinds(ir):
    from graphiler_amd import torch_boundary
    from graphiler_amd.mpdfg import passes
    from graphiler_amd.mpdfg.builder import MPDFG
    torch_boundary.load()
    plan = MPDFG(torch._C.parse_ir(ir), {})
    rw = passes._Rewriter(plan)
    for _ in range(4):
        if not rw.late_fusion():
            break
    plan.graph.lint()
    # the operator that produces the plan's result, and everything it reads
    live, todo = [], [plan.graph.return_node()]
    while todo:
        for v in todo.pop().inputs():
            if v.node().kind().startswith("my_ops::"):
                live.append(v.node().kind())
            todo.append(v.node())
    return live


def test_typed_product_and_dot_fuse_only_without_row_factor_and_heads():
    """sum(gathered typed product * broadcast rows) becomes SegmentMMEdgeDot only when
    the product has no per-row factor (the dot has no operand for one) and its weights
    are not known to be (T, H, K, M) (the sum over dim 1 would then run across heads)."""
    plain = _DOT_PLAN.replace("WTYPE", "Tensor").replace("SCALE", "%none")
    assert _late_fused_kinds(plain) == ["my_ops::SegmentMMEdgeDot"]
    three_d = _DOT_PLAN.replace("WTYPE", "Float(4, 16, 8)").replace("SCALE", "%none")
    assert _late_fused_kinds(three_d) == ["my_ops::SegmentMMEdgeDot"]

    scaled = _DOT_PLAN.replace("WTYPE", "Tensor").replace("SCALE", "%s")
    assert sorted(_late_fused_kinds(scaled)) == ["my_ops::BroadcastDstNode",
                                                 "my_ops::SegmentMMEdgeGather"]
    heads = _DOT_PLAN.replace("WTYPE", "Float(4, 2, 16, 8)").replace("SCALE", "%none")
    assert sorted(_late_fused_kinds(heads)) == ["my_ops::BroadcastDstNode",
                                                "my_ops::SegmentMMEdgeGather"]


def test_stacked_products_skip_operands_overwritten_in_place():
    """Two SegmentMMNode of one x with an in-place operator on x between them are two
    products of two different values: they must not become one stacked product placed
    after the overwrite.  Without the overwrite the same graph does stack."""
    from types import SimpleNamespace

    from graphiler_amd.mpdfg import passes

    def build(inplace):
        g = torch._C.Graph()
        dgl = g.addInput()
        x, w1, w2 = (g.addInput() for _ in range(3))
        for v in (x, w1, w2):
            v.setType(torch._C.TensorType.get())
        a = g.create("my_ops::SegmentMMNode", [x, w1, dgl], 1)
        g.appendNode(a)
        if inplace:
            m = g.create("aten::relu_", [x], 1)
            g.appendNode(m)
        b = g.create("my_ops::SegmentMMNode", [x, w2, dgl], 1)
        g.appendNode(b)
        s = g.create("aten::add", [a.output(), b.output(), g.insertConstant(1)], 1)
        g.appendNode(s)
        g.registerOutput(s.output())
        rw = passes._Rewriter(SimpleNamespace(graph=g, residency={}))
        changed = rw._fuse_stacked_mm()
        return changed, [n.kind() for n in g.nodes()]

    changed, kinds = build(inplace=False)
    assert changed and kinds.count("my_ops::SegmentMMNodeStacked") == 1
    changed, kinds = build(inplace=True)
    assert not changed and kinds.count("my_ops::SegmentMMNode") == 2


def test_every_operator_the_passes_emit_is_registered():
    """A rewrite that creates a node of an operator the library does not register fails
    only when a plan happens to take it: check the names in the passes' source once."""
    import inspect
    import re
    from graphiler_amd import torch_boundary
    from graphiler_amd.mpdfg import builder, passes
    torch_boundary.load()
    names = set()
    for mod in (builder, passes):
        names |= set(re.findall(r'"(my_ops::\w+)"', inspect.getsource(mod)))
    assert len(names) > 20
    for name in sorted(names):
        assert len(torch._C._jit_get_schemas_for_operator(name)) == 1, name
