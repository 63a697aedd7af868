"""Graph container and host-side preparation.

``DGLGraph`` mirrors the reference's custom class
(include/dglgraph.h:7-75, registered in src/dglgraph.cpp:5-24): the same ten
constructor arguments, the same four setters and the same public fields, so the
operator wrappers in :mod:`graphiler_amd.ops` read it exactly as the
reference's operators read theirs.  On top of that it caches what the gfx950
kernels need once per graph: the slot->row maps of both adjacencies, whether
the edge-id columns are the identity, and a reusable workspace.

``prepare_graph`` mirrors python/graphiler/utils/setup.py:116-146: in- and
out-adjacency with int32 pointer / neighbour / edge-id columns and int64 COO
columns, built here from a plain (src, dst) edge list instead of a DGL graph.
Inside one node's group the edges keep ascending edge-id order.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from . import capi


@dataclass
class GraphArrays:
    """Host (numpy) form of the arrays ``prepare_graph`` produces."""
    num_nodes: int
    in_pointer: np.ndarray
    in_node_indices: np.ndarray
    in_edge_indices: np.ndarray
    out_pointer: np.ndarray
    out_node_indices: np.ndarray
    out_edge_indices: np.ndarray
    COO_src: np.ndarray
    COO_dst: np.ndarray


def _group(n_nodes: int, key: np.ndarray, other: np.ndarray):
    """Stable grouping of edge ids by ``key`` -> (pointer, neighbour, edge id)."""
    order = np.argsort(key, kind="stable")
    counts = np.bincount(key, minlength=n_nodes)
    pointer = np.zeros(n_nodes + 1, np.int64)
    np.cumsum(counts, out=pointer[1:])
    return (pointer.astype(np.int32), other[order].astype(np.int32),
            order.astype(np.int32))


def build_graph_arrays(src, dst, num_nodes: int) -> GraphArrays:
    """CSR-by-destination and CSR-by-source of an edge list (host, numpy)."""
    src = np.ascontiguousarray(src, dtype=np.int64)
    dst = np.ascontiguousarray(dst, dtype=np.int64)
    if src.shape != dst.shape or src.ndim != 1:
        raise ValueError("src and dst must be 1-D arrays of equal length")
    if src.shape[0] >= 2 ** 31 or num_nodes >= 2 ** 31:
        raise ValueError("graphs are limited to int32 node and edge ids")
    if src.size and (min(src.min(), dst.min()) < 0 or
                     max(src.max(), dst.max()) >= num_nodes):
        raise ValueError("edge endpoint outside [0, num_nodes)")
    ip, inb, ie = _group(num_nodes, dst, src)
    op, onb, oe = _group(num_nodes, src, dst)
    return GraphArrays(num_nodes, ip, inb, ie, op, onb, oe, src, dst)


def type_pointer(type_of, num_types: int) -> np.ndarray:
    """int32 running sum of items per type; ``type_of`` must be sorted
    (ids of one type are contiguous, include/dglgraph.h:68-69)."""
    type_of = np.asarray(type_of, dtype=np.int64)
    if type_of.size and np.any(np.diff(type_of) < 0):
        raise ValueError("items must be sorted by type")
    ptr = np.zeros(num_types + 1, np.int64)
    np.cumsum(np.bincount(type_of, minlength=num_types), out=ptr[1:])
    return ptr.astype(np.int32)


def sort_edges_by_type(src, dst, etype):
    """Stable reorder of an edge list so edge ids of one type are contiguous.
    Returns (src, dst, etype, order) with ``order`` the applied permutation."""
    etype = np.asarray(etype, dtype=np.int64)
    order = np.argsort(etype, kind="stable")
    return (np.asarray(src)[order], np.asarray(dst)[order], etype[order], order)


def _check_index(t: torch.Tensor, dtype: torch.dtype, name: str):
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must be {dtype}")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


class DGLGraph:
    """Drop-in for ``torch.classes.my_classes.DGLGraph``."""

    def __init__(self, in_pointer, in_node_indices, in_edge_indices,
                 out_pointer, out_node_indices, out_edge_indices, COO_src,
                 COO_dst, ntype_pointer: Optional[torch.Tensor] = None,
                 etype_pointer: Optional[torch.Tensor] = None):
        for name, t in (("in_pointer", in_pointer),
                        ("in_node_indices", in_node_indices),
                        ("in_edge_indices", in_edge_indices),
                        ("out_pointer", out_pointer),
                        ("out_node_indices", out_node_indices),
                        ("out_edge_indices", out_edge_indices)):
            _check_index(t, torch.int32, name)
        _check_index(COO_src, torch.int64, "COO_src")
        _check_index(COO_dst, torch.int64, "COO_dst")
        self.in_pointer = in_pointer
        self.in_node_indices = in_node_indices
        self.in_edge_indices = in_edge_indices
        self.out_pointer = out_pointer
        self.out_node_indices = out_node_indices
        self.out_edge_indices = out_edge_indices
        self.COO_src = COO_src
        self.COO_dst = COO_dst
        self.ntype_pointer = None
        self.etype_pointer = None
        self.ntype_COO = None
        self.etype_COO = None
        # include/dglgraph.h:22-27
        self.num_nodes = int(in_pointer.size(0)) - 1
        self.num_edges = int(in_node_indices.size(0))
        self.num_ntypes = 1
        self.num_etypes = 1
        self._cache = {}
        self.SetNtypePointer(ntype_pointer)
        self.SetEtypePointer(etype_pointer)

    # -- setters (include/dglgraph.h:29-46) ---------------------------------
    def SetNtypePointer(self, pointer):
        if pointer is not None:
            _check_index(pointer, torch.int32, "ntype_pointer")
        self.ntype_pointer = pointer
        self.num_ntypes = int(pointer.size(0)) - 1 if pointer is not None else 1

    def SetEtypePointer(self, pointer):
        if pointer is not None:
            _check_index(pointer, torch.int32, "etype_pointer")
        self.etype_pointer = pointer
        self.num_etypes = int(pointer.size(0)) - 1 if pointer is not None else 1
        # the layouts prepared from the edge types belong to the old pointer (a layout
        # already handed to a launch stays alive with that launch's tensors)
        self._cache.pop("typed_tiles", None)
        self._cache.pop("pairs", None)

    def SetNtypeCOO(self, column):
        _check_index(column, torch.int64, "ntype_COO")
        if column.size(0) != self.num_nodes:
            raise RuntimeError("ntype_COO must have one entry per node")
        self.ntype_COO = column

    def SetEtypeCOO(self, column):
        _check_index(column, torch.int64, "etype_COO")
        if column.size(0) != self.num_edges:
            raise RuntimeError("etype_COO must have one entry per edge")
        self.etype_COO = column

    # -- derived data the kernels schedule with -----------------------------
    @property
    def device(self):
        return self.in_pointer.device

    def _row_ids(self, pointer: torch.Tensor) -> torch.Tensor:
        rows = torch.empty(self.num_edges, dtype=torch.int32, device=self.device)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        capi.check(capi.load().ga_csr_row_ids(
            pointer.data_ptr(), self.num_nodes, self.num_edges,
            rows.data_ptr(), stream), "ga_csr_row_ids")
        return rows

    @property
    def in_row_of_slot(self) -> torch.Tensor:
        """Destination node of every slot of the in-adjacency (int32, E)."""
        if "in_rows" not in self._cache:
            self._cache["in_rows"] = self._row_ids(self.in_pointer)
        return self._cache["in_rows"]

    @property
    def out_row_of_slot(self) -> torch.Tensor:
        """Source node of every slot of the out-adjacency (int32, E)."""
        if "out_rows" not in self._cache:
            self._cache["out_rows"] = self._row_ids(self.out_pointer)
        return self._cache["out_rows"]

    def _identity(self, key: str, column: torch.Tensor) -> bool:
        if key not in self._cache:
            n = column.numel()
            ar = torch.arange(n, dtype=torch.int32, device=column.device)
            self._cache[key] = bool(torch.equal(column, ar))
        return self._cache[key]

    @property
    def max_in_degree(self) -> int:
        """Largest number of in-edges of a node (one reduction and host read, then cached)."""
        if "max_in_degree" not in self._cache:
            self._cache["max_in_degree"] = int(torch.diff(self.in_pointer).max().item()) \
                if self.num_nodes > 0 else 0
        return self._cache["max_in_degree"]

    @property
    def in_eid_is_identity(self) -> bool:
        """True when edge ids already are in-adjacency slot numbers."""
        return self._identity("in_ident", self.in_edge_indices)

    @property
    def out_eid_is_identity(self) -> bool:
        return self._identity("out_ident", self.out_edge_indices)

    def relation_pairs(self) -> Optional["RelationPairs"]:
        """The (destination, relation) pairs of the in-adjacency, built once on the
        device: a layer whose per-edge work is linear in a per-relation matrix (HGT's
        ``bmm(k, relation_att)`` and ``bmm(v, relation_msg)``, examples/HGT/HGT.py:35-44)
        can apply that matrix once per pair instead of once per edge.  None when the
        graph has no edge types or the slots of a destination are not grouped by
        relation (they are when edge ids are sorted by type, as
        include/dglgraph.h:24-27 requires for the type pointer)."""
        if "pairs" not in self._cache:
            self._cache["pairs"] = _build_relation_pairs(self)
        return self._cache["pairs"]

    def workspace(self, nbytes: int) -> torch.Tensor:
        """Scratch buffer shared by the operators called on this graph (grows on
        demand).  Calls that use it must be ordered on one stream: two streams
        working on one graph object race on it.  A buffer that was handed out is
        kept alive as long as the graph, because a recorded HIP graph may still
        replay launches that write to it."""
        ws = self._cache.get("ws")
        if ws is None or ws.numel() < nbytes:
            if ws is not None:
                self._cache.setdefault("retired_ws", []).append(ws)
            ws = torch.empty(max(int(nbytes), 256), dtype=torch.uint8,
                             device=self.device)
            self._cache["ws"] = ws
        return ws


@dataclass
class RelationPairs:
    """Slots of the in-adjacency grouped into runs of one (destination, relation).
    Pairs are numbered in slot order (by destination, then relation); ``by_type``
    lists them by relation (stable), which is the row order the typed products need."""
    num_pairs: int
    pair_pointer: torch.Tensor      # (P + 1) int32: first slot of every pair
    pair_of_slot: torch.Tensor      # (E) int32
    pair_dst: torch.Tensor          # (P) int32, ascending
    dst_pointer: torch.Tensor       # (N + 1) int32: first pair of every destination
    type_pointer: torch.Tensor      # (T + 1) int32 over by_type
    by_type: torch.Tensor           # (P) int64: pair ids ordered by relation
    rank: torch.Tensor              # (P) int32: position of a pair in by_type
    rank_of_slot: torch.Tensor      # (E) int32: rank[pair_of_slot]
    dst_by_type: torch.Tensor       # (P) int64: pair_dst[by_type]


def _build_relation_pairs(g: "DGLGraph") -> Optional[RelationPairs]:
    if g.etype_pointer is None or g.num_edges == 0:
        return None
    dev, n_edges, n_types = g.device, g.num_edges, g.num_etypes
    rows = g.in_row_of_slot.long()
    eid = g.in_edge_indices.long()
    etype = torch.bucketize(eid, g.etype_pointer[1:].long(), right=True)
    key = rows * n_types + etype
    if n_edges > 1 and not bool((key[1:] >= key[:-1]).all()):
        return None
    first = torch.ones(n_edges, dtype=torch.bool, device=dev)
    first[1:] = key[1:] != key[:-1]
    pair_of_slot = torch.cumsum(first, 0) - 1
    starts = torch.nonzero(first).reshape(-1)
    n_pairs = int(starts.numel())
    pair_key = key[starts]
    pair_dst = torch.div(pair_key, n_types, rounding_mode="floor")
    pair_type = pair_key - pair_dst * n_types
    by_type = torch.argsort(pair_type, stable=True)
    rank = torch.empty_like(by_type)
    rank[by_type] = torch.arange(n_pairs, device=dev)
    return RelationPairs(
        num_pairs=n_pairs,
        pair_pointer=torch.cat([starts, starts.new_tensor([n_edges])]).int().contiguous(),
        pair_of_slot=pair_of_slot.int().contiguous(),
        pair_dst=pair_dst.int().contiguous(),
        dst_pointer=torch.searchsorted(pair_dst.contiguous(),
                                       torch.arange(g.num_nodes + 1, device=dev)).int().contiguous(),
        type_pointer=torch.searchsorted(pair_type[by_type].contiguous(),
                                        torch.arange(n_types + 1, device=dev)).int().contiguous(),
        by_type=by_type.contiguous(),
        rank=rank.int().contiguous(),
        rank_of_slot=rank[pair_of_slot].int().contiguous(),
        dst_by_type=pair_dst[by_type].contiguous())


def group_on_device(key: torch.Tensor, other: Optional[torch.Tensor], n_keys: int):
    """Stable grouping of item ids by ``key`` on the GPU (setup.py:116-146):
    returns (pointer int32 (n_keys+1), other[order] int32 or None, order int32,
    status int32 (1,)).  ``status`` is left on the device: 1 means a key outside
    [0, n_keys); read it when convenient."""
    from . import capi
    if key.dtype != torch.int64 or not key.is_cuda or not key.is_contiguous():
        raise RuntimeError("key must be a contiguous int64 CUDA tensor")
    if other is not None and (other.dtype != torch.int64 or other.shape != key.shape
                              or not other.is_cuda or not other.is_contiguous()):
        raise RuntimeError("other must match key (contiguous int64 CUDA tensor)")
    n, dev = int(key.numel()), key.device
    if n >= 2 ** 31 or n_keys >= 2 ** 31 - 1:
        raise ValueError("graphs are limited to int32 node and edge ids")
    lib = capi.load()
    pointer = torch.empty(n_keys + 1, dtype=torch.int32, device=dev)
    order = torch.empty(n, dtype=torch.int32, device=dev)
    nbr = torch.empty(n, dtype=torch.int32, device=dev) if other is not None else None
    status = torch.empty(1, dtype=torch.int32, device=dev)
    ws = torch.empty(max(int(lib.ga_group_edges_workspace_bytes(n_keys, n)), 256),
                     dtype=torch.uint8, device=dev)
    capi.check(lib.ga_group_edges(
        key.data_ptr(), None if other is None else other.data_ptr(), n_keys, n,
        pointer.data_ptr(), None if nbr is None else nbr.data_ptr(), order.data_ptr(),
        status.data_ptr(), ws.data_ptr(), ws.numel(),
        torch.cuda.current_stream(dev).cuda_stream), "ga_group_edges")
    return pointer, nbr, order, status


def _type_columns(type_of, num_types: int, dev):
    """Type pointer + type COO column on the device; items must be sorted by
    type (ids of one type contiguous, include/dglgraph.h:68-69)."""
    t = torch.as_tensor(np.ascontiguousarray(type_of, dtype=np.int64)).to(dev)
    pointer, _, _, status = group_on_device(t, None, num_types)
    unsorted = bool((t[1:] < t[:-1]).any().item()) if t.numel() > 1 else False
    if unsorted:
        raise ValueError("items must be sorted by type")
    if int(status.item()):
        raise ValueError("type outside [0, num_types)")
    return pointer, t


def prepare_graph(src, dst, num_nodes: int, device="cuda:0",
                  ntype_of=None, num_ntypes: int = 0, etype_of=None,
                  num_etypes: int = 0) -> DGLGraph:
    """Build the device graph from an edge list (setup.py:116-146); when type
    columns are given also install the type pointers and type COO columns the
    way load_data does for heterogeneous graphs (setup.py:87-100).  The edge
    list is uploaded once and grouped on the GPU (both adjacencies and the type
    pointers); nothing is sorted on the host."""
    dev = torch.device(device)
    src = np.ascontiguousarray(src, dtype=np.int64)
    dst = np.ascontiguousarray(dst, dtype=np.int64)
    if src.shape != dst.shape or src.ndim != 1:
        raise ValueError("src and dst must be 1-D arrays of equal length")
    if src.shape[0] >= 2 ** 31 or num_nodes >= 2 ** 31 - 1:
        raise ValueError("graphs are limited to int32 node and edge ids")
    coo_src, coo_dst = torch.from_numpy(src).to(dev), torch.from_numpy(dst).to(dev)
    ip, inb, ie, st_in = group_on_device(coo_dst, coo_src, num_nodes)
    op, onb, oe, st_out = group_on_device(coo_src, coo_dst, num_nodes)
    if int((st_in | st_out).item()):
        raise ValueError("edge endpoint outside [0, num_nodes)")
    g = DGLGraph(ip, inb, ie, op, onb, oe, coo_src, coo_dst, None, None)
    if ntype_of is not None:
        p, t = _type_columns(ntype_of, num_ntypes, dev)
        g.SetNtypePointer(p)
        g.SetNtypeCOO(t)
    if etype_of is not None:
        p, t = _type_columns(etype_of, num_etypes, dev)
        g.SetEtypePointer(p)
        g.SetEtypeCOO(t)
    return g
