"""ctypes binding of libfeatgraph_hip.so (the C ABI declared in include/featgraph_hip.h).

The library is the only execution path of this package: if it has not been built the
import of any operator fails with an explicit error rather than falling back to another
implementation.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfeatgraph_hip.so")

FG_OK = 0
_lib = None

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int


class FgPlanOpts(ctypes.Structure):
    _fields_ = [("split_threshold", ctypes.c_int32), ("item_edges", ctypes.c_int32),
                ("wide_offsets", ctypes.c_int32), ("tile_major", ctypes.c_int32),
                ("pass_buffers", ctypes.c_int32), ("reserved", ctypes.c_int32 * 3)]


# Options every module passes to fg_spmm_plan_create (None: the library's defaults).
plan_opts = None


def plan_opts_ptr():
    return ctypes.byref(plan_opts) if plan_opts is not None else None


# name -> (restype, argtypes); also the list of symbols the header declares
SIGNATURES = {
    "fg_version": (_int, []),
    "fg_last_error": (ctypes.c_char_p, []),
    "fg_csr_to_dds": (_int, [_i64, _i64, _vp, _vp, _vp, _int, _vp, _vp, _vp]),
    "fg_partition_coo_2d": (_int, [_i64, _i64, _i64, _vp, _vp, _int, _int, _vp, _vp, _vp]),
    "fg_check_csr_host": (_int, [_i64, _i64, _vp, _vp]),
    "fg_spmm_plan_create": (_int, [_vp, _i64, _i64, _int, ctypes.POINTER(FgPlanOpts), ctypes.POINTER(_vp)]),
    "fg_spmm_plan_destroy": (None, [_vp]),
    "fg_spmm_plan_reserve": (_int, [_vp, _int, _int, _int, _int]),
    "fg_spmm_plan_narrow_indices": (_int, [_vp, _vp, _vp]),
    "fg_debug_checks": (_int, [_int]),
    "fg_spmm_plan_bytes": (_i64, [_vp]),
    "fg_spmm_plan_describe": (_int, [_vp, _int, _int, ctypes.c_char_p, ctypes.c_size_t]),
    "fg_spmm_csr_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _vp]),
    "fg_spmm_csr_noalloc_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _vp]),
    "fg_spmm_dds_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _vp]),
    "fg_gspmm_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _vp]),
    "fg_gspmm_arg_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _vp]),
    "fg_edge_values_head_major_f32": (_int, [_vp, _vp, _i64, _int, _vp, _vp]),
    "fg_sddmm_coo_f32": (_int, [_vp, _vp, _i64, _vp, _vp, _vp, _int, _int, _vp]),
    "fg_sddmm_csr_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _vp]),
    "fg_sddmm_dds_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp]),
    "fg_gsddmm_elementwise_f32": (_int, [_vp, _vp, _i64, _vp, _vp, _vp, _int, _int, _vp]),
    "fg_gspmm_bcast_f32": (_int, [_vp, _vp, _vp, _int, _int, _vp, _int, _int, _vp, _vp, _int, _int, _vp, _int, _vp, _vp, _vp, _int, _vp]),
    "fg_gspmm_bcast_dds_f32": (_int, [_vp, _vp, _vp, _vp, _int, _int, _vp, _int, _int, _vp, _vp, _int, _int, _vp, _int, _vp, _vp, _vp, _int, _vp]),
    "fg_gsddmm_bcast_f32": (_int, [_vp, _vp, _i64, _int, _vp, _int, _int, _vp, _vp, _int, _int, _vp, _int, _vp, _int, _int, _vp]),
    "fg_edge_softmax_f32": (_int, [_vp, _vp, _vp, _vp, _int, _vp]),
    "fg_edge_softmax_backward_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp]),
    "fg_edge_softmax_stats_f32": (_int, [_vp, _vp, _vp, _vp, _int, _vp]),
    "fg_edge_softmax_head_major_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _int, _vp, _vp]),
    "fg_graph_attention_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, _vp]),
    "fg_graph_attention_additive_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, _vp]),
    "fg_graph_attention_coef_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _int, _int, _vp]),
    "fg_graph_attention_backward_q_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, _vp]),
    "fg_graph_attention_backward_kv_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, _vp]),
    "fg_graph_attention_additive_coef_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _vp]),
    "fg_graph_attention_additive_backward_er_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, _vp]),
    "fg_graph_attention_additive_backward_elv_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, _vp]),
    "fg_synth_powerlaw_csr": (_int, [_i64, _vp, _vp, _vp, ctypes.c_uint64, _int, _vp, _vp]),
    "fg_synth_community_csr": (_int, [_i64, _vp, _vp, _vp, _int, _vp, _vp, _vp, _vp, ctypes.c_double, ctypes.c_uint64, _int, _vp, _vp]),
}


def lib():
    """Loads the shared library once; raises if it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m featgraph_amd.build` "
                "(there is no other execution path)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error():
    return lib().fg_last_error().decode("utf-8", "replace")


def check(rc):
    """Maps a negative fg_status to the Python exception the module layer documents."""
    if rc >= 0:
        return rc
    msg = last_error()
    if rc in (-1, -2, -3):
        raise ValueError(msg)
    if rc == -5:
        raise MemoryError(msg)
    raise RuntimeError(msg)


def host_ptr(a):
    """Pointer to a C-contiguous numpy array's data (the array must stay alive)."""
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


def dev_ptr(t):
    """Device pointer of a torch tensor (None -> NULL)."""
    return ctypes.c_void_p(0 if t is None else t.data_ptr())
