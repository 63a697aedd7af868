"""Feature-shape broadcasting tables of the binary graph operators (host side).

Mirror of ``UseBcast`` / ``CalcBcastOff`` (src/ops/dgl_primitives/bcast.cc:6-71,
struct ``BcastOff`` in bcast.h:17-55): given the operator name and the shapes of
the two operands (dimension 0 is the node / edge dimension and never takes
part), decide whether numpy-style trailing-dimension broadcasting is needed and
produce, for every element of the flattened per-row output, the offset of the
left and of the right operand element that feed it.

Differences from the reference, on purpose:

* the tables are returned as int64 numpy arrays of ``out_len`` entries.  The
  reference wraps its ``std::vector<int64_t>`` with ``from_blob(ptr, {lhs_len})``
  under the default float dtype (bcast.cc:63-67), i.e. a reinterpretation with
  the wrong length; every operator it registers has ``use_bcast == false`` so
  the tensors are never read.  Here the logical content is kept.
* shapes are passed as tuples, no tensors are needed.

For ``op == "dot"`` the last dimension of the left operand is the reduction
length and is skipped; offsets then count vectors of ``reduce_size`` elements,
as the consuming kernel multiplies them by ``reduce_size`` (sddmm.cuh:80-120).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

import numpy as np


@dataclass(frozen=True)
class BcastOff:
    lhs_offset: np.ndarray
    rhs_offset: np.ndarray
    use_bcast: bool
    lhs_len: int
    rhs_len: int
    out_len: int
    reduce_size: int


def _feat_len(shape: Sequence[int]) -> int:
    n = 1
    for d in shape[1:]:
        n *= int(d)
    return n


def use_bcast(op: str, lhs_shape: Sequence[int], rhs_shape: Sequence[int]) -> bool:
    """bcast.cc:6-17: copies never broadcast; otherwise any difference in rank
    or in a feature dimension does."""
    if op in ("copy_lhs", "copy_rhs"):
        return False
    if len(lhs_shape) != len(rhs_shape):
        return True
    return any(int(a) != int(b) for a, b in zip(lhs_shape[1:], rhs_shape[1:]))


def calc_bcast_off(op: str, lhs_shape: Sequence[int], rhs_shape: Sequence[int]) -> BcastOff:
    """bcast.cc:19-71.  Output elements are numbered row-major over the
    broadcast feature shape (last dimension fastest)."""
    lhs_shape = tuple(int(d) for d in lhs_shape)
    rhs_shape = tuple(int(d) for d in rhs_shape)
    l_nd, r_nd = len(lhs_shape), len(rhs_shape)
    lhs_len, rhs_len = _feat_len(lhs_shape), _feat_len(rhs_shape)
    bcast = use_bcast(op, lhs_shape, rhs_shape)
    lhs_off = np.zeros(1, dtype=np.int64)
    rhs_off = np.zeros(1, dtype=np.int64)
    reduce_size, out_len = 1, 1
    if bcast:
        first = 0
        if op == "dot":
            reduce_size = lhs_shape[l_nd - 1]
            first = 1
        stride_l = stride_r = 1
        for j in range(first, max(l_nd, r_nd) - 1):
            dl = 1 if l_nd - 1 - j < 1 else lhs_shape[l_nd - 1 - j]
            dr = 1 if r_nd - 1 - j < 1 else rhs_shape[r_nd - 1 - j]
            steps = np.arange(max(dl, dr), dtype=np.int64)
            # a dimension shorter than its partner contributes offset 0 past
            # its end (size 1 = plain broadcast), bcast.cc:46-47
            add_l = np.where(steps < dl, steps, 0) * stride_l
            add_r = np.where(steps < dr, steps, 0) * stride_r
            lhs_off = (add_l[:, None] + lhs_off[None, :]).reshape(-1)
            rhs_off = (add_r[:, None] + rhs_off[None, :]).reshape(-1)
            out_len *= max(dl, dr)
            stride_l *= dl
            stride_r *= dr
    else:
        out_len = rhs_len if op == "copy_rhs" else lhs_len
        if op == "dot":
            reduce_size = lhs_shape[l_nd - 1]
            out_len //= reduce_size
    return BcastOff(lhs_off, rhs_off, bcast, lhs_len, rhs_len, out_len, reduce_size)
