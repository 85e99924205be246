"""ctypes binding of libpsa_hip.so (declared in include/psa_hip.h).

There is no fallback: if the shared library is missing, importing this module raises
ImportError with the command that builds it.
"""
import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpsa_hip.so")

PSA_OK = 0
PSA_ERR_ARG = -1
PSA_ERR_UNSUPPORTED = -2
PSA_ERR_LAUNCH = -3
PSA_MODE_TOPK = 0
PSA_MODE_THRESHOLDBOUND = 1
PSA_MAX_LEVEL_ITEMS = 8


PSA_DTYPE_BF16, PSA_DTYPE_F16, PSA_DTYPE_F32 = 0, 1, 2


class Tensor4(Structure):
    _fields_ = [("ptr", c_void_p), ("stride_b", c_int64), ("stride_h", c_int64), ("stride_l", c_int64), ("dtype", c_int32),
                ("reserved", c_int32)]


# name -> (restype, argtypes); one entry per symbol declared in include/psa_hip.h
SIGNATURES = {
    "psa_version": (c_int, []),
    "psa_last_error": (c_char_p, []),
    "psa_pool_elems": (c_int64, [c_int, c_int, c_int, c_int, c_int]),
    "psa_pool_level_offset": (c_int64, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "psa_pool_kv": (c_int, [Tensor4, Tensor4, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "psa_estimate_workspace_bytes": (c_int64, [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "psa_estimate_sampled": (
        c_int,
        [Tensor4, Tensor4, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_float, c_int, c_int, c_void_p],
    ),
    "psa_estimate_sampled_map": (
        c_int,
        [Tensor4, Tensor4, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_float, c_int, c_int, c_void_p, c_int, c_int, c_int, POINTER(c_int32), POINTER(c_double), c_int, c_int, c_double,
         c_void_p],
    ),
    "psa_draw_sample_offsets": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_uint64, c_void_p]),
    "psa_level_map": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_int, POINTER(c_int32), POINTER(c_double), c_int,
         c_int, c_double, c_void_p],
    ),
    "psa_level_map_qwen": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, POINTER(c_int32), POINTER(c_double), POINTER(c_double), c_int, c_int,
         c_void_p],
    ),
    "psa_estimate_xattn_workspace_bytes": (c_int64, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "psa_estimate_xattn": (
        c_int,
        [Tensor4, Tensor4, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "psa_map_from_list": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_void_p]),
    "psa_list_from_map": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "psa_ksim": (c_int, [Tensor4, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_float, c_void_p]),
    "psa_map_min_cap": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "psa_density": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_int, c_void_p, c_void_p]),
    "psa_gather_rows": (c_int, [POINTER(Tensor4), POINTER(Tensor4), POINTER(c_int), c_int, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                c_void_p]),
    "psa_pool_kv_indexed": (c_int, [Tensor4, Tensor4, c_void_p, Tensor4, Tensor4, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                    c_void_p]),
    "psa_estimate_sampled_indexed": (
        c_int,
        [Tensor4, c_void_p, Tensor4, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_int, c_float, c_int, c_int, c_void_p],
    ),
    "psa_estimate_sampled_map_indexed": (
        c_int,
        [Tensor4, c_void_p, Tensor4, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_int, c_float, c_int, c_int, c_void_p, c_int, c_int, c_int, POINTER(c_int32), POINTER(c_double), c_int, c_int,
         c_double, c_void_p],
    ),
    "psa_fwd_indexed": (
        c_int,
        [Tensor4, c_void_p, Tensor4, Tensor4, c_void_p, c_void_p, c_void_p, c_int, Tensor4, c_void_p, c_int, c_int, c_int, c_int,
         c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p],
    ),
    "psa_fwd": (
        c_int,
        [Tensor4, Tensor4, Tensor4, c_void_p, c_void_p, c_void_p, c_int, Tensor4, c_void_p, c_int, c_int, c_int, c_int,
         c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p],
    ),
    "psa_fwd_workspace_bytes": (c_int64, [c_int, c_int, c_int, c_int]),
    "psa_schedule_bytes": (c_int64, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "psa_build_schedule": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "psa_fwd_scheduled": (
        c_int,
        [Tensor4, c_void_p, Tensor4, Tensor4, c_void_p, c_void_p, c_void_p, c_int, c_void_p, Tensor4, c_void_p, c_int, c_int, c_int,
         c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    ),
    "psa_fwd_noalloc": (
        c_int,
        [Tensor4, Tensor4, Tensor4, c_void_p, c_void_p, c_void_p, c_int, Tensor4, c_void_p, c_int, c_int, c_int, c_int,
         c_int, c_int, c_int, c_float, c_int, c_void_p],
    ),
    "psa_fwd_noalloc_max_rows": (c_int64, []),
    "psa_bwd_workspace_bytes": (c_int64, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "psa_bwd": (
        c_int,
        [Tensor4, Tensor4, Tensor4, c_void_p, c_void_p, c_void_p, c_int, Tensor4, Tensor4, c_void_p, Tensor4, Tensor4, Tensor4,
         c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    ),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libpsa_hip.so is not built (%s). Build it with: python pyramid-sparse-attention_amd/build_ext.py" % LIB_PATH
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


class PSAError(RuntimeError):
    pass


def check(rc, what=""):
    """Raise for a non-zero return code: ValueError for argument errors (the reference raises
    ValueError / AssertionError for bad configurations), PSAError otherwise."""
    if rc == PSA_OK:
        return
    msg = lib.psa_last_error().decode() or ("%s failed with code %d" % (what, rc))
    if rc in (PSA_ERR_ARG, PSA_ERR_UNSUPPORTED):
        raise ValueError(msg)
    raise PSAError(msg)
