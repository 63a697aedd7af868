"""The GAT layer of the benchmark written as user-defined functions (the form of
examples/GAT/GAT.py:25-36, leaky_relu slope 0.2); `bench.py --path compiled`
compiles them with graphiler_amd.mpdfg.  TorchScript needs them in a file."""
import torch
import torch.nn.functional as F

from graphiler_amd.mpdfg import EdgeBatchDummy, NodeBatchDummy


def gat_message(edges: EdgeBatchDummy, fc_weight, attn_weight):
    z_src = torch.mm(edges.src['h'], fc_weight)
    z_dst = torch.mm(edges.dst['h'], fc_weight)
    score = torch.mm(torch.cat([z_src, z_dst], dim=1), attn_weight)
    return {'z': z_src, 'e': F.leaky_relu(score, 0.2)}


def gat_reduce(nodes: NodeBatchDummy):
    alpha = torch.softmax(nodes.mailbox['e'], dim=1)
    return {'h': torch.sum(alpha * nodes.mailbox['z'], dim=1)}
