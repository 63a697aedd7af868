"""MI355X-native sparse graph primitives behind Graphiler's operator boundary.

``graphiler_amd.ops`` mirrors the reference's ``torch.ops.my_ops.*`` functions,
``graphiler_amd.graph.DGLGraph`` its ``torch.classes.my_classes.DGLGraph``;
both sit on the C ABI of ``include/graphiler_amd.h`` (hand-written gfx950 HIP
kernels in ``graphiler_amd/csrc``).  Importing the package does not load the
library; the first operator call does, and fails if it was not built.
"""
from . import capi, datasets, graph, ops  # noqa: F401
from .graph import DGLGraph, prepare_graph  # noqa: F401

__all__ = ["capi", "datasets", "graph", "ops", "DGLGraph", "prepare_graph"]
