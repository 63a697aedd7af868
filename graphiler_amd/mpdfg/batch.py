"""Stand-ins for DGL's EdgeBatch / NodeBatch that user-defined functions are
written against (the role of python/graphiler/dgl_udf_batch.py:5-57).

A UDF touches only the properties (``edges.src['h']``, ``nodes.mailbox['m']``,
...); scripted, every property read becomes a ``prim::GetAttr`` on one of the
fields below, which is how the builder recognises where a value lives.
"""
from typing import Dict

import torch


@torch.jit.script
class EdgeBatchDummy(object):
    def __init__(self, src: Dict[str, torch.Tensor], edge: Dict[str, torch.Tensor],
                 dst: Dict[str, torch.Tensor], srctype: Dict[str, torch.Tensor],
                 edgetype: Dict[str, torch.Tensor], dsttype: Dict[str, torch.Tensor]):
        self.f_src = src
        self.f_edge = edge
        self.f_dst = dst
        self.f_srctype = srctype
        self.f_edgetype = edgetype
        self.f_dsttype = dsttype

    @property
    def src(self):
        return self.f_src

    @property
    def dst(self):
        return self.f_dst

    @property
    def data(self):
        return self.f_edge

    @property
    def srctype(self):
        return self.f_srctype

    @property
    def dsttype(self):
        return self.f_dsttype

    @property
    def type(self):
        return self.f_edgetype


@torch.jit.script
class NodeBatchDummy(object):
    def __init__(self, mail: Dict[str, torch.Tensor], node: Dict[str, torch.Tensor],
                 nodetype: Dict[str, torch.Tensor]):
        self.f_mail = mail
        self.f_node = node
        self.f_nodetype = nodetype

    @property
    def mailbox(self):
        return self.f_mail

    @property
    def data(self):
        return self.f_node

    @property
    def type(self):
        return self.f_nodetype
