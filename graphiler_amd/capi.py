"""ctypes binding of the C ABI declared in ``include/graphiler_amd.h``.

The shared library is built in-tree (``graphiler_amd/lib/libgraphiler_hip.so``)
by ``make -C graphiler_amd/csrc``.  There is no fallback: importing this module
without the built library raises, so a missing HIP build can never be mistaken
for a working one.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libgraphiler_hip.so")

GA_OK = 0
GA_EINVAL, GA_EUNSUPPORTED, GA_EWORKSPACE, GA_EALIGN, GA_ESCRATCH = -1, -2, -3, -4, -5
GA_STATIC_SCRATCH_BYTES = 32 << 20
GA_ACT_NONE, GA_ACT_RELU, GA_ACT_ELU = 0, 1, 2
GA_F32, GA_BF16 = 0, 1
GA_COPY_U, GA_COPY_E, GA_U_MUL_E, GA_U_ADD_E, GA_U_SUB_E, GA_U_DIV_E = 0, 1, 2, 3, 4, 5
GA_SDDMM_ADD, GA_SDDMM_SUB, GA_SDDMM_MUL, GA_SDDMM_DIV = 0, 1, 2, 3
GA_SUM, GA_MAX, GA_MIN = 0, 1, 2
(GA_BCAST_ADD, GA_BCAST_SUB, GA_BCAST_MUL, GA_BCAST_DIV, GA_BCAST_COPY_LHS, GA_BCAST_COPY_RHS,
 GA_BCAST_DOT) = range(7)

_vp, _i64, _int, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/graphiler_amd.h one to one.
SIGNATURES = {
    "ga_version": (_int, []),
    "ga_error_string": (ctypes.c_char_p, [_int]),
    "ga_csr_row_ids": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "ga_group_edges_workspace_bytes": (_sz, [_i64, _i64]),
    "ga_group_edges": (_int, [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "ga_spmm_workspace_bytes": (_sz, [_i64, _i64]),
    "ga_spmm_csr": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                           _i64, _int, _int, _int, _vp, _sz, _vp]),
    "ga_spmm_scaled_workspace_bytes": (_sz, [_i64, _i64]),
    "ga_spmm_csr_scaled": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64,
                                  _int, _int, _vp, _sz, _vp]),
    "ga_spmm_arg_workspace_bytes": (_sz, [_i64, _i64]),
    "ga_spmm_csr_arg": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                               _i64, _i64, _int, _int, _int, _vp, _sz, _vp]),
    "ga_sddmm_u_add_v": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _i64, _i64, _int,
                                _vp]),
    "ga_sddmm_u_op_v": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _i64, _i64, _int, _int,
                               _vp]),
    "ga_spmm_csr_bcast": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp,
                                 _i64, _i64, _i64, _int, _int, _vp]),
    "ga_sddmm_bcast": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _vp, _vp, _i64, _i64,
                              _i64, _i64, _int, _vp]),
    "ga_sddmm_u_op_v_adj": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "ga_typed_tile_rows": (_i64, [_i64]),
    "ga_typed_tiles_chunk_capacity": (_i64, [_i64, _i64, _i64, _i64]),
    "ga_typed_tiles_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "ga_typed_tiles_build": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp,
                                    _vp, _vp, _vp, _sz, _vp]),
    "ga_typed_spmm": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                             _i64, _i64, _i64, _i64, _int, _vp]),
    "ga_typed_spmm_act": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                                 _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "ga_sddmm_u_dot_v": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _i64, _i64, _i64,
                                _int, _vp]),
    "ga_softmax_workspace_bytes": (_sz, [_i64, _i64]),
    "ga_segment_softmax": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                                  _vp, _sz, _vp]),
    "ga_segment_mm": (_int, [_vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                             _int, _vp]),
    "ga_segment_mm_gated": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _vp]),
    "ga_transpose_scale_blocks": (_int, [_vp, _vp, ctypes.c_float, _vp, _i64, _i64, _int, _vp]),
    "ga_transpose_scale_blocks_as": (_int, [_vp, _vp, _int, ctypes.c_float, _vp, _i64, _i64, _int, _vp]),
    "ga_segment_mm_stacked": (_int, [_vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                     _int, _vp]),
    "ga_segment_mm_gather": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                    _i64, _i64, _i64, _i64, _int, _vp]),
    "ga_gather_rows": (_int, [_vp, _int, _vp, _vp, _i64, _i64, _vp]),
    "ga_linear_attn": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                              _i64, _vp]),
    "ga_linear_rows_scaled": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "ga_project_attn": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                               _i64, _int, _vp]),
    "ga_gat_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "ga_gat_aggregate_from_z": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                                       _i64, _i64, ctypes.c_float, _int, _vp, _sz, _vp]),
    "ga_edge_softmax_sum": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                   _int, _vp, _sz, _vp]),
    "ga_dot_attention_sum": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                                    _i64, _i64, _int, _vp, _sz, _vp]),
    "ga_gat_static_scratch_needed": (_i64, [_i64, _i64, _i64, _int, _int]),
    "ga_gat_aggregate_static": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                                       _i64, _i64, ctypes.c_float, _int, _vp]),
    "ga_gat_aggregate": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                                _i64, _i64, ctypes.c_float, _int, _vp, _sz,
                                _vp]),
    "ga_gat_aggregate_act": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                    ctypes.c_float, _int, _int, _vp, _sz, _vp]),
    "ga_gat_aggregate_from_z_act": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                                           _i64, ctypes.c_float, _int, _int, _vp, _sz, _vp]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with "
                "`make -C graphiler_amd/csrc` (or __graft_entry__.build())")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class GraphilerError(RuntimeError):
    """A C-ABI entry point returned a non-zero code."""

    def __init__(self, code: int, where: str):
        self.code = code
        text = load().ga_error_string(code).decode()
        super().__init__(f"{where}: {text} (code {code})")


def check(code: int, where: str) -> None:
    if code != GA_OK:
        raise GraphilerError(code, where)
