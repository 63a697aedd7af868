"""CPU oracle for the sparse graph-primitive layer -- TEST INFRASTRUCTURE ONLY.

numpy-in / numpy-out wrappers over ``liboracle.so`` (built from
``graph_ops_oracle.c`` by ``make -C oracle``).  Only the test-suite, the smoke
check and the benchmark's ``cpu_baseline`` leg import this package; the product
package never does and has no CPU fallback.

Each wrapper names the reference operator it restates; the C source carries the
file:line citations.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

OP_COPY_U, OP_COPY_E, OP_U_MUL_E = 0, 1, 2
RED_SUM, RED_MAX, RED_MIN = 0, 1, 2
_OPS = {"copy_u": OP_COPY_U, "copy_e": OP_COPY_E, "u_mul_e": OP_U_MUL_E,
        "u_add_e": 3, "u_sub_e": 4, "u_div_e": 5}
_REDS = {"sum": RED_SUM, "max": RED_MAX, "min": RED_MIN}


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc; returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []),
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in ("orc_group_edges", "orc_type_pointer", "orc_spmm",
                     "orc_spmm_sum_f32", "orc_sddmm_u_add_v",
                     "orc_sddmm_u_dot_v", "orc_segment_softmax",
                     "orc_segment_mm", "orc_segment_mm_f32",
                     "orc_gather_rows", "orc_gat_aggregate"):
            getattr(_lib, name).restype = ctypes.c_int
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return int(lib().orc_num_threads())


def set_num_threads(n: int) -> None:
    lib().orc_set_num_threads(ctypes.c_int(int(n)))


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def _i64(v):
    return ctypes.c_int64(int(v))


def _check(rc, what):
    if rc != 0:
        raise ValueError(f"oracle {what}: invalid arguments (code {rc})")


def group_edges(n_nodes, key, other):
    """(pointer, nbr, eid) grouping edges by ``key`` (prepare_graph)."""
    key = _c(key, np.int64)
    other = _c(other, np.int64)
    e = key.shape[0]
    pointer = np.empty(n_nodes + 1, np.int32)
    nbr = np.empty(e, np.int32)
    eid = np.empty(e, np.int32)
    _check(lib().orc_group_edges(_i64(n_nodes), _i64(e), _p(key), _p(other),
                                 _p(pointer), _p(nbr), _p(eid)), "group_edges")
    return pointer, nbr, eid


def type_pointer(type_of, n_types):
    type_of = _c(type_of, np.int64)
    pointer = np.empty(n_types + 1, np.int32)
    _check(lib().orc_type_pointer(_i64(type_of.shape[0]), _i64(n_types),
                                  _p(type_of), _p(pointer)), "type_pointer")
    return pointer


def spmm(ptr, nbr, eid, u, w=None, *, op="copy_u", reduce="sum", heads=1,
         want_arg=False):
    """Generalised SpMM (SpMMSrc / SpMMEdge / gspmm_*_mul_e_sum, max/min)."""
    ptr = _c(ptr, np.int32)
    nbr = _c(nbr, np.int32)
    eid = _c(eid, np.int32)
    u = _c(u, np.float32)
    w = _c(w, np.float32)
    n = ptr.shape[0] - 1
    feat = int(np.prod(u.shape[1:])) if u.ndim > 1 else 1
    out = np.empty((n, feat), np.float32)
    arg_u = np.empty((n, feat), np.int32) if want_arg else None
    arg_e = np.empty((n, feat), np.int32) if want_arg else None
    _check(lib().orc_spmm(_i64(n), _p(ptr), _p(nbr), _p(eid), _p(u), _p(w),
                          _p(out), _p(arg_u), _p(arg_e), _i64(feat),
                          _i64(heads), ctypes.c_int(_OPS[op]),
                          ctypes.c_int(_REDS[reduce])), "spmm")
    return (out, arg_u, arg_e) if want_arg else out


def spmm_sum_f32(ptr, nbr, eid, u, w=None, *, op="copy_u", heads=1):
    """Sequential fp32 accumulation (reference order); timed CPU baseline."""
    ptr = _c(ptr, np.int32)
    nbr = _c(nbr, np.int32)
    eid = _c(eid, np.int32)
    u = _c(u, np.float32)
    w = _c(w, np.float32)
    n = ptr.shape[0] - 1
    feat = int(np.prod(u.shape[1:])) if u.ndim > 1 else 1
    out = np.empty((n, feat), np.float32)
    _check(lib().orc_spmm_sum_f32(_i64(n), _p(ptr), _p(nbr), _p(eid), _p(u),
                                  _p(w), _p(out), _i64(feat), _i64(heads),
                                  ctypes.c_int(_OPS[op])), "spmm_sum_f32")
    return out


def sddmm_u_add_v(src, dst, u, v):
    """gsddmm_u_add_v_mul_alpha: out[e] = u[src[e]] + v[dst[e]] (fp32)."""
    src = _c(src, np.int64)
    dst = _c(dst, np.int64)
    u = _c(u, np.float32)
    v = _c(v, np.float32)
    feat = int(np.prod(u.shape[1:])) if u.ndim > 1 else 1
    out = np.empty((src.shape[0], feat), np.float32)
    _check(lib().orc_sddmm_u_add_v(_i64(src.shape[0]), _p(src), _p(dst), _p(u),
                                   _p(v), _p(out), _i64(feat)), "u_add_v")
    return out


def sddmm_u_op_v(op, src, dst, u, v):
    """Generic SDDMM: out[e] = u[src[e]] (op) v[dst[e]], op in add/sub/mul/div."""
    src = _c(src, np.int64)
    dst = _c(dst, np.int64)
    u = _c(u, np.float32)
    v = _c(v, np.float32)
    feat = int(np.prod(u.shape[1:])) if u.ndim > 1 else 1
    out = np.empty((src.shape[0], feat), np.float32)
    code = {"add": 0, "sub": 1, "mul": 2, "div": 3}[op]
    _check(lib().orc_sddmm_u_op_v(_i64(src.shape[0]), _p(src), _p(dst), _p(u), _p(v),
                                  _p(out), _i64(feat), ctypes.c_int(code)), "u_op_v")
    return out


def sddmm_u_dot_v(src, dst, u, v):
    """u_dot_v over the last dimension: u, v are (N, H, D) -> (E, H)."""
    src = _c(src, np.int64)
    dst = _c(dst, np.int64)
    u = _c(u, np.float32)
    v = _c(v, np.float32)
    if u.ndim == 2:
        u = u[:, None, :]
        v = v[:, None, :]
    heads, dim = u.shape[1], u.shape[2]
    out = np.empty((src.shape[0], heads), np.float32)
    _check(lib().orc_sddmm_u_dot_v(_i64(src.shape[0]), _p(src), _p(dst), _p(u),
                                   _p(v), _p(out), _i64(heads), _i64(dim)),
           "u_dot_v")
    return out


def segment_softmax(ptr, eid, x, *, zero_floor=False):
    """SegmentSoftmax over each destination's in-edges; x is (E,) or (E, H)."""
    ptr = _c(ptr, np.int32)
    eid = _c(eid, np.int32)
    x = _c(x, np.float32)
    heads = int(np.prod(x.shape[1:])) if x.ndim > 1 else 1
    y = np.empty_like(x)
    _check(lib().orc_segment_softmax(_i64(ptr.shape[0] - 1), _i64(x.shape[0]),
                                     _p(ptr), _p(eid), _p(x), _p(y),
                                     _i64(heads),
                                     ctypes.c_int(1 if zero_floor else 0)),
           "segment_softmax")
    return y


def segment_mm(tp, X, W, *, heads=1, f32_accumulate=False):
    """SegmentMMNode / SegmentMMEdge.  X (rows, heads*K), W (T, heads, K, M)."""
    tp = _c(tp, np.int32)
    X = _c(X, np.float32)
    W = _c(W, np.float32)
    T = tp.shape[0] - 1
    K, M = W.shape[-2], W.shape[-1]
    rows = int(tp[-1]) if T > 0 else 0
    Y = np.empty((rows, heads * M), np.float32)
    fn = lib().orc_segment_mm_f32 if f32_accumulate else lib().orc_segment_mm
    _check(fn(_i64(T), _p(tp), _p(X), _p(W), _p(Y), _i64(heads), _i64(K),
              _i64(M)), "segment_mm")
    return Y


def gather_rows(idx, x):
    """Broadcast*: y = x[idx] (bit-exact copy, any dtype)."""
    idx = _c(idx, np.int64)
    x = np.ascontiguousarray(x)
    row_bytes = int(x.strides[0]) if x.ndim > 0 and x.shape[0] > 0 else (
        int(np.prod(x.shape[1:])) * x.itemsize)
    y = np.empty((idx.shape[0],) + x.shape[1:], x.dtype)
    _check(lib().orc_gather_rows(_i64(idx.shape[0]), _i64(x.shape[0]), _p(idx),
                                 _p(x), _p(y), _i64(row_bytes)), "gather_rows")
    return y


def gat_aggregate(ptr, nbr, el, er, z, *, heads=1, slope=0.2):
    """u_add_v -> leaky_relu -> edge softmax -> u_mul_e sum, in fp64."""
    ptr = _c(ptr, np.int32)
    nbr = _c(nbr, np.int32)
    el = _c(el, np.float32)
    er = _c(er, np.float32)
    z = _c(z, np.float32)
    n = ptr.shape[0] - 1
    feat = int(np.prod(z.shape[1:]))
    out = np.empty((n, feat), np.float32)
    _check(lib().orc_gat_aggregate(_i64(n), _p(ptr), _p(nbr), _p(el), _p(er),
                                   _p(z), _p(out), _i64(heads),
                                   _i64(feat // heads),
                                   ctypes.c_double(slope)), "gat_aggregate")
    return out
