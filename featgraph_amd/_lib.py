"""ctypes binding of libfeatgraph_hip.so (include/featgraph_hip.h).

There is no fallback: if the library cannot be loaded, every operator of the
package raises.  The CPU checker under oracle/ is never used from here.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libfeatgraph_hip.so")

_i32, _i64, _p = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p

# name -> (restype, argtypes); mirrors include/featgraph_hip.h line by line
SIGNATURES = {
    "fg_version": (ctypes.c_int, []),
    "fg_last_error": (ctypes.c_char_p, []),
    "fg_spmm_plan_create": (ctypes.c_int, [_i64, _i64, _i64, _p, _p, ctypes.POINTER(_p)]),
    "fg_spmm_plan_create_partitioned": (ctypes.c_int, [_i64, _i64, _i64, _p, _p, _i32, ctypes.POINTER(_p)]),
    "fg_spmm_plan_destroy": (None, [_p]),
    "fg_spmm_plan_row_order": (ctypes.c_int, [_p, _p, ctypes.POINTER(_i32)]),
    "fg_spmm_csr_f32": (ctypes.c_int, [_p, _p, _p, _p, _i32, _i32, _p]),
    "fg_spmm_csr_noalloc_f32": (ctypes.c_int, [_i64, _i64, _i64, _p, _p, _p, _p, _p, _i32, _p]),
    "fg_spmm_csr_general_f32": (ctypes.c_int, [_p, _p, _p, _p, _i32, _i32, _i32, _p]),
    "fg_spmm_csr_mh_general_f32": (ctypes.c_int, [_p, _p, _p, _p, _i32, _i32, _i32, _i32, _p]),
    "fg_edge_softmax_backward_csr_f32": (ctypes.c_int, [_i64, _p, _p, _p, _p, _i32, _p]),
    "fg_permute_rows_f32": (ctypes.c_int, [_i64, _i32, _p, _p, _p, _p]),
    "fg_spmm_csr_pitched_f32": (ctypes.c_int, [_p, _p, _i32, _p, _p, _i32, _p]),
    "fg_pad_rows_f32": (ctypes.c_int, [_i64, _i32, _i32, _p, _p, _p]),
    "fg_sddmm_coo_plan_pitched_f32": (ctypes.c_int, [_p, _p, _p, _i32, _p, _i32, _p]),
    "fg_add_f32": (ctypes.c_int, [_i64, _p, _p, _p, _p]),
    "fg_sddmm_coo_general_f32": (ctypes.c_int, [_i64, _p, _p, _p, _p, _p, _i32, _i32, _p]),
    "fg_spmm_csr_mh_f32": (ctypes.c_int, [_p, _p, _p, _p, _i32, _i32, _i32, _p]),
    "fg_sddmm_coo_f32": (ctypes.c_int, [_i64, _p, _p, _p, _p, _p, _i32, _p]),
    "fg_sddmm_coo_mh_f32": (ctypes.c_int, [_i64, _p, _p, _p, _p, _p, _i32, _i32, _p]),
    "fg_sddmm_plan_create": (ctypes.c_int, [_i64, _i64, _i64, _p, _p, ctypes.POINTER(_p)]),
    "fg_sddmm_plan_create_partitioned": (ctypes.c_int, [_i64, _i64, _i64, _p, _p, _i32, ctypes.POINTER(_p)]),
    "fg_sddmm_plan_destroy": (None, [_p]),
    "fg_sddmm_coo_plan_f32": (ctypes.c_int, [_p, _p, _p, _p, _i32, _i32, _p]),
    "fg_sddmm_coo_general_plan_f32": (ctypes.c_int, [_p, _p, _p, _p, _i32, _i32, _p]),
    "fg_edge_softmax_csr_f32": (ctypes.c_int, [_i64, _p, _p, _p, _i32, _p]),
    "fg_sddmm_softmax_plan_f32": (ctypes.c_int, [_p, _p, _p, _p, _i32, _i32, _p]),
    "fg_attention_csr_mh_f32": (ctypes.c_int, [_p, _p, _p, _p, _p, _i32, _i32, _p]),
    "fg_sddmm_plan_describe": (ctypes.c_int, [_p, _i32, _i32, ctypes.c_char_p, _i64]),
    "fg_check_indices": (ctypes.c_int, [_i64, _p, _i64, ctypes.POINTER(_i64), _p]),
    "fg_probe_gather_f32": (ctypes.c_int, [_p, _i64, _i32, _i32, _i32, _i64, _p, _p]),
    "fg_probe_gather_count": (_i64, [_i64, _i32, _i32, _i64]),
    "fg_probe_gather_rows_f32": (ctypes.c_int, [_p, _i64, _i32, _i64, _p, _p]),
    "fg_probe_gather_rows_count": (_i64, [_i32, _i64]),
    "fg_probe_gather_write_rows_f32": (ctypes.c_int, [_p, _i64, _i32, _i64, _i32, _p, _i64, _p, _p]),
    "fg_probe_gather_write_rows_count": (ctypes.c_int, [_i32, _i64, _i32, _p, _p]),
    "fg_probe_store_rows_f32": (_i64, [_p, _i64, _i32, _i64, _p]),
    "fg_probe_gather_stream_f32": (_i64, [_p, _i32, _i64, _p, _i64, _i64, _i32, _p, _p]),
    "fg_config_set": (ctypes.c_int, [ctypes.c_char_p, _i32]),
    "fg_config_get": (ctypes.c_int, [ctypes.c_char_p, ctypes.POINTER(_i32)]),
    "fg_spmm_describe": (ctypes.c_int, [_p, _i32, _i32, _i32, ctypes.c_char_p, _i64]),
    "fg_sddmm_describe": (ctypes.c_int, [_i64, _i32, _i32, ctypes.c_char_p, _i64]),
}

FG_EUNSUPPORTED = -4   # include/featgraph_hip.h

_lib = None


class FeatGraphError(RuntimeError):
    """A libfeatgraph_hip.so entry point returned an error code."""

    def __init__(self, code, message):
        super().__init__("libfeatgraph_hip error %d: %s" % (code, message))
        self.code = code


def lib():
    """The loaded library.  Raises (never falls back) when it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m featgraph_amd.build` "
                "(there is no CPU or PyTorch fallback)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(code):
    if code != 0:
        raise FeatGraphError(code, lib().fg_last_error().decode("utf-8", "replace"))


def config_set(key, value):
    check(lib().fg_config_set(key.encode(), int(value)))


def config_get(key):
    out = _i32(0)
    check(lib().fg_config_get(key.encode(), ctypes.byref(out)))
    return out.value
