"""Running a compiled plan: ``update_all`` (python/graphiler/update_all.py:1-5)
and the graph-plus-feature-dictionaries holder it expects (the attributes the
reference hangs on a DGL graph in python/graphiler/utils/setup.py:87-100,143-146)."""
from __future__ import annotations

from typing import Dict

import torch

from .. import torch_boundary
from ..graph import DGLGraph


class GraphData:
    """``DGLGraph`` (the scripted class instance) + ``ndata`` / ``edata`` /
    ``ntype_data`` / ``etype_data`` dictionaries."""

    def __init__(self, graph: DGLGraph):
        self.graph = graph
        self.DGLGraph = torch_boundary.script_graph(graph)
        self.ndata: Dict[str, torch.Tensor] = {}
        self.edata: Dict[str, torch.Tensor] = {}
        self.ntype_data: Dict[str, torch.Tensor] = {}
        self.etype_data: Dict[str, torch.Tensor] = {}


def update_all(g: GraphData, mpdfg, msg_params=(), reduce_params=(), update_params=()):
    updated = mpdfg.forward(g.DGLGraph, g.ndata, g.edata, g.ntype_data, g.etype_data,
                            *msg_params, *reduce_params, *update_params)
    for key in updated:
        g.ndata[key] = updated[key]
    return updated
