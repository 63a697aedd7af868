"""The TorchScript boundary registers the reference's exact schemas (no GPU)."""
import torch

from graphiler_amd import torch_boundary

G = "__torch__.torch.classes.my_classes.DGLGraph"
# schema strings as registered by the reference (spmm.cu:391-406, sddmm.cu:131-134,
# segment_softmax.cu:27-30, segment_mm.cu:35-42, broadcast.cu:102-122)
REFERENCE_SCHEMAS = {
    "SpMMEdge": f"my_ops::SpMMEdge(Tensor x, int[] dim, bool k, int? t, {G} g) -> Tensor y",
    "SpMMSrc": f"my_ops::SpMMSrc(Tensor x, int[] dim, bool k, int? t, {G} g) -> Tensor y",
    "gspmm_src_mul_e_sum": f"my_ops::gspmm_src_mul_e_sum(Tensor x, Tensor y, int[] dim, bool k, int? t, {G} g) -> Tensor z",
    "gspmm_dst_mul_e_sum": f"my_ops::gspmm_dst_mul_e_sum(Tensor x, Tensor y, int[] dim, bool k, int? t, {G} g) -> Tensor z",
    "gsddmm_u_add_v_mul_alpha": f"my_ops::gsddmm_u_add_v_mul_alpha(Tensor x, Tensor y, int alpha, {G} g) -> Tensor z",
    "SegmentSoftmax": f"my_ops::SegmentSoftmax(Tensor x, int dim, int? t, {G} g) -> Tensor y",
    "SegmentMMNode": f"my_ops::SegmentMMNode(Tensor x, Tensor y, {G} g) -> Tensor z",
    "SegmentMMEdge": f"my_ops::SegmentMMEdge(Tensor x, Tensor y, {G} g) -> Tensor z",
    "BroadcastSrcNode": f"my_ops::BroadcastSrcNode(Tensor x, {G} g) -> Tensor y",
    "BroadcastDstNode": f"my_ops::BroadcastDstNode(Tensor x, {G} g) -> Tensor y",
    "BroadcastNodeType": f"my_ops::BroadcastNodeType(Tensor x, {G} g) -> Tensor y",
    "BroadcastSrcNodeType": f"my_ops::BroadcastSrcNodeType(Tensor x, {G} g) -> Tensor y",
    "BroadcastDstNodeType": f"my_ops::BroadcastDstNodeType(Tensor x, {G} g) -> Tensor y",
    "BroadcastEdgeType": f"my_ops::BroadcastEdgeType(Tensor x, {G} g) -> Tensor y",
    "get_feat_dim": "my_ops::get_feat_dim(Tensor _0) -> int _0",
}


def test_schemas_match_the_reference():
    torch_boundary.load()
    for name, want in REFERENCE_SCHEMAS.items():
        schemas = torch._C._jit_get_schemas_for_operator(f"my_ops::{name}")
        assert len(schemas) == 1, name
        assert str(schemas[0]) == want


def test_class_and_host_only_op():
    torch_boundary.load()
    assert torch.ops.my_ops.get_feat_dim(torch.zeros(3, 4, 5)) == 20
    i32 = lambda *a: torch.tensor(a, dtype=torch.int32)
    try:   # CPU tensors are rejected like the reference's CHECK_INPUT would
        torch.classes.my_classes.DGLGraph(i32(0, 1), i32(0), i32(0), i32(0, 1), i32(0),
                                          i32(0), torch.tensor([0]), torch.tensor([0]),
                                          None, None)
    except RuntimeError as e:
        assert "must be a CUDA tensor" in str(e)
    else:
        raise AssertionError("CPU tensors were accepted")


def test_plan_scripts_against_the_boundary():
    """A TorchScript function using the operators compiles to my_ops:: nodes."""
    torch_boundary.load()

    @torch.jit.script
    def gat_plan(g: torch.classes.my_classes.DGLGraph, z: torch.Tensor,
                 el: torch.Tensor, er: torch.Tensor):
        e = torch.ops.my_ops.gsddmm_u_add_v_mul_alpha(el, er, 1, g)
        e = torch.nn.functional.leaky_relu(e, 0.2)
        a = torch.ops.my_ops.SegmentSoftmax(e, 1, None, g)
        return torch.ops.my_ops.gspmm_src_mul_e_sum(z, a, [1], False, None, g)

    text = str(gat_plan.graph)
    for op in ("my_ops::gsddmm_u_add_v_mul_alpha", "my_ops::SegmentSoftmax",
               "my_ops::gspmm_src_mul_e_sum"):
        assert op in text
