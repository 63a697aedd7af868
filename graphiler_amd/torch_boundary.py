"""Loader for the TorchScript boundary library (``lib/libgraphiler.so``).

The reference loads its operators with ``torch.classes.load_library`` /
``torch.ops.load_library`` of ``~/.dgl/libgraphiler.so``
(python/graphiler/mpdfg_builder.py:11-14, python/graphiler/utils/setup.py:13-14);
a plan compiled against it only needs this library loaded instead.
"""
from __future__ import annotations

import os

import torch

from .graph import DGLGraph

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib",
                        "libgraphiler.so")
_loaded = False


def load() -> str:
    """Register ``torch.classes.my_classes.DGLGraph`` and ``torch.ops.my_ops.*``."""
    global _loaded
    if not _loaded:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with "
                              "`make -C graphiler_amd/csrc torch`")
        torch.classes.load_library(LIB_PATH)
        torch.ops.load_library(LIB_PATH)
        _loaded = True
    return LIB_PATH


def script_graph(g: DGLGraph):
    """The ``torch.classes.my_classes.DGLGraph`` object for a Python-side graph
    (same tensors, no copies)."""
    load()
    sg = torch.classes.my_classes.DGLGraph(
        g.in_pointer, g.in_node_indices, g.in_edge_indices, g.out_pointer,
        g.out_node_indices, g.out_edge_indices, g.COO_src, g.COO_dst,
        g.ntype_pointer, g.etype_pointer)
    if g.ntype_COO is not None:
        sg.SetNtypeCOO(g.ntype_COO)
    if g.etype_COO is not None:
        sg.SetEtypeCOO(g.etype_COO)
    return sg
