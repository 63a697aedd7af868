"""User-defined message / reduce / update functions of the four example models,
written against the batch stand-ins the way a user of the reference writes them
(examples/GCN/GCN.py:21-27, examples/GAT/GAT.py:25-36, examples/RGCN/RGCN.py:25-33,
examples/HGT/HGT.py:28-60).  TorchScript needs them in a source file."""
import torch
import torch.nn.functional as F

from graphiler_amd.mpdfg import EdgeBatchDummy, NodeBatchDummy


# ---- GCN: normalised copy of the source feature, summed, relu -------------------
def gcn_message(edges: EdgeBatchDummy):
    scale = torch.pow(edges.src['degree'], -0.5)
    return {'m': edges.src['h'] * scale}


def gcn_reduce(nodes: NodeBatchDummy):
    return {'h': torch.relu(torch.sum(nodes.mailbox['m'], dim=1))}


# ---- GAT, one head ---------------------------------------------------------------
def gat_message(edges: EdgeBatchDummy, fc_weight, attn_weight):
    z_src = torch.mm(edges.src['h'], fc_weight)
    z_dst = torch.mm(edges.dst['h'], fc_weight)
    both = torch.cat([z_src, z_dst], dim=1)
    score = torch.mm(both, attn_weight)
    return {'z': z_src, 'e': F.leaky_relu(score, 0.2)}


def gat_reduce(nodes: NodeBatchDummy):
    alpha = torch.softmax(nodes.mailbox['e'], dim=1)
    return {'h': torch.sum(alpha * nodes.mailbox['z'], dim=1)}


# ---- GAT, four heads of width 16 (the shape literals must be constants for the
# compiler to see that the view keeps one row per edge) -----------------------------
def gat4_message(edges: EdgeBatchDummy, fc_weight, attn_l, attn_r):
    # fc_weight (K, 64); attn_l / attn_r (1, 4, 16)
    z_src = torch.mm(edges.src['h'], fc_weight).view(-1, 4, 16)
    z_dst = torch.mm(edges.dst['h'], fc_weight).view(-1, 4, 16)
    el = torch.sum(z_src * attn_l, dim=2, keepdim=True)          # (E, 4, 1)
    er = torch.sum(z_dst * attn_r, dim=2, keepdim=True)
    return {'z': z_src, 'e': F.leaky_relu(el + er, 0.2)}


def gat4x64_message(edges: EdgeBatchDummy, fc_weight, attn_l, attn_r):
    """The same layer with four heads of width 64 (the 256-wide layers of the
    products-sized GAT configuration); attn_l / attn_r (1, 4, 64)."""
    z_src = torch.mm(edges.src['h'], fc_weight).view(-1, 4, 64)
    z_dst = torch.mm(edges.dst['h'], fc_weight).view(-1, 4, 64)
    el = torch.sum(z_src * attn_l, dim=2, keepdim=True)
    er = torch.sum(z_dst * attn_r, dim=2, keepdim=True)
    return {'z': z_src, 'e': F.leaky_relu(el + er, 0.2)}


def gat4_reduce(nodes: NodeBatchDummy):
    alpha = torch.softmax(nodes.mailbox['e'], dim=1)             # over the in-edges, per head
    return {'h': torch.sum(alpha * nodes.mailbox['z'], dim=1)}


# ---- RGCN: per-relation weight, per-edge norm --------------------------------------
def rgcn_message(edges: EdgeBatchDummy):
    w = edges.type['weight']
    msg = torch.bmm(edges.src['h'].unsqueeze(1), w).squeeze()
    return {'m': msg * edges.data['norm']}


def rgcn_reduce(nodes: NodeBatchDummy):
    return {'h': torch.sum(nodes.mailbox['m'], dim=1)}


# ---- HGT (single head, as the reference's simplified layer) ----------------------
def hgt_message(edges: EdgeBatchDummy, sqrt_dk: float):
    k = torch.bmm(edges.src['h'].unsqueeze(1), edges.srctype['k_weight']).squeeze()
    v = torch.bmm(edges.src['h'].unsqueeze(1), edges.srctype['v_weight']).squeeze()
    q = torch.bmm(edges.dst['h'].unsqueeze(1), edges.dsttype['q_weight']).squeeze()
    k = torch.bmm(k.unsqueeze(1), edges.type['relation_att']).squeeze()
    v = torch.bmm(v.unsqueeze(1), edges.type['relation_msg']).squeeze()
    score = torch.sum(k * q, dim=1, keepdim=True) * edges.type['relation_pri'] / sqrt_dk
    return {'attn': score, 'v': v}


def hgt_reduce(nodes: NodeBatchDummy):
    t = torch.softmax(nodes.mailbox['attn'], dim=1)
    return {'t': torch.sum(t * nodes.mailbox['v'], dim=1)}


def hgt_update(nodes: NodeBatchDummy):
    alpha = torch.sigmoid(nodes.type['skip'])
    out = torch.bmm(nodes.data['t'].unsqueeze(1), nodes.type['a_weight']).squeeze()
    return {'h': out * alpha.unsqueeze(1)}
