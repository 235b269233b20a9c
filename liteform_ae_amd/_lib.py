"""ctypes binding of liblfhip.so (declared in include/liteform_hip.h).

The library is loaded from the package directory.  There is no fallback: when the
shared object is missing, loading raises and every operation of the package fails with
that error.  torch is imported first so that the HIP runtime already in the process is
the one the library binds to.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

LF_OK = 0
LF_ERR_INVALID = -1
LF_ERR_TOO_SMALL = -2
LF_ERR_HIP = -3
LF_ERR_CONFIG = -4
LF_ERR_UNSUPPORTED = -5
LF_ERR_WORKSPACE = -6

LF_MAX_CLASSES = 11
LF_STATS_FIELDS = 4
LF_SPMM_INFO_FIELDS = 9
LF_DTYPE_F32 = 0
LF_DTYPE_BF16 = 1
LF_COST_REFERENCE = 0
LF_COST_GFX950 = 1
LF_CSR_CANONICAL = 1
LF_CSR_UNIT_VALUES = 2

# LITEFORM_HIP_LIB points at another build of the same library (kernel tuning experiments)
LIB_PATH = os.environ.get("LITEFORM_HIP_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                                              "liblfhip.so")

i32p = C.POINTER(C.c_int32)
i64p = C.POINTER(C.c_int64)
f32p = C.POINTER(C.c_float)
f64p = C.POINTER(C.c_double)
vp = C.c_void_p


class BucketDesc(C.Structure):
    """struct lf_bucket_desc"""
    _fields_ = [("width", C.c_int32), ("part", C.c_int32), ("num_ell_rows", C.c_int64),
                ("d_rows", vp), ("d_cols", vp), ("d_vals", vp), ("d_meta", vp)]


# name -> (restype, argtypes); one entry per function declared in the header
SIGNATURES = {
    "lf_version": (C.c_int, []),
    "lf_last_error": (C.c_char_p, []),
    "lf_status_string": (C.c_char_p, [C.c_int]),
    "lf_stats_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int64, C.c_int32]),
    "lf_bucket_stats": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, C.c_int32, C.c_int32, vp, C.c_size_t,
                                  i64p, i64p, vp]),
    "lf_coo_degrees": (C.c_int, [vp, vp, C.c_int64, C.c_int64, C.c_int64, C.c_int32, vp, vp]),
    "lf_row_features": (C.c_int, [vp, C.c_int64, vp, vp, vp]),
    "lf_row_features_static": (C.c_int, [vp, C.c_int64, vp, vp]),
    "lf_search_bucket_config": (C.c_int, [i64p, i64p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                          i32p, i32p, f64p, i32p]),
    "lf_model_spmm_ms": (C.c_int, [i64p, C.c_int32, C.c_int32, C.c_int64, C.c_int64, C.c_int32, C.c_int32, f64p]),
    "lf_row_overlap": (C.c_int, [vp, vp, C.c_int64, C.c_int64, vp, vp, vp]),
    "lf_hyb_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int32, C.c_int32]),
    "lf_hyb_layout": (C.c_int, [i64p, i32p, C.c_int32, i64p, i64p, i64p, i64p]),
    "lf_stats_seg_bounds": (vp, [vp, C.c_int64, C.c_int32]),
    "lf_hyb_plan": (C.c_int, [vp, vp, vp, vp, C.c_int64, C.c_int64, C.c_int32, i32p, i32p, vp, C.c_size_t,
                              i64p, vp]),
    "lf_hyb_build": (C.c_int, [vp, vp, vp, vp, C.c_int64, C.c_int64, C.c_int32, i32p, i32p, i64p, vp,
                               C.c_size_t, vp, vp, vp, vp, vp, vp]),
    "lf_spmm_create": (C.c_int, [C.POINTER(vp), C.POINTER(BucketDesc), C.c_int32, C.c_int32, C.c_int64,
                                 C.c_int64, C.c_int32, C.c_int32, vp]),
    "lf_spmm_run": (C.c_int, [vp, vp, vp, vp]),
    "lf_spmm_destroy": (C.c_int, [vp]),
    "lf_spmm_set_windows": (C.c_int, [vp, C.c_int32]),
    "lf_spmm_info": (C.c_int, [vp, i64p]),
    "lf_spmm_time_ms": (C.c_int, [vp, vp, vp, C.c_int32, C.c_int32, vp, C.c_size_t, f32p, vp]),
    "lf_csr_check": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, C.c_int64, vp, i32p, vp]),
    "lf_csr_spmm": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32, vp, vp, vp, vp]),
    "lf_csr_spmm_trusted": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, C.c_int32, C.c_int32, vp, vp, vp]),
    "lf_coo_to_csr_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int64, C.c_int64]),
    "lf_coo_to_csr": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, C.c_int64, vp, C.c_size_t, vp, vp, vp, i64p, vp]),
    "lf_bsr_spmm": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32, vp, vp, vp, vp]),
    "lf_bsr_spmm_trusted": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, C.c_int32, C.c_int32, vp, vp, vp]),
}

_lock = threading.Lock()
_lib = None


def load():
    """Returns the loaded library; raises RuntimeError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m liteform_ae_amd.build` "
                "(needs hipcc); there is no CPU fallback")
        import torch  # noqa: F401  (brings the process's HIP runtime in first)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error() -> str:
    return load().lf_last_error().decode("utf-8", "replace")


def check(status: int):
    """Maps a status code to the exception type the reference raises in that situation."""
    if status == LF_OK:
        return
    msg = last_error()
    if status == LF_ERR_TOO_SMALL:
        raise ValueError(msg)                       # format_algos.py:921
    if status == LF_ERR_CONFIG:
        raise IndexError(msg)                       # format_algos.py:279
    if status == LF_ERR_INVALID and msg.startswith("invalid padding"):
        raise AssertionError(msg)                   # format_algos.py:303
    if status == LF_ERR_INVALID:
        raise ValueError(msg)
    if status == LF_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(f"liblfhip: {msg} (status {status})")


def ptr(t):
    """Device (or host) address of a torch tensor / numpy array, or None."""
    if t is None:
        return None
    if hasattr(t, "data_ptr"):
        return t.data_ptr()
    return t.ctypes.data


def np_ptr(a, ctype):
    return a.ctypes.data_as(C.POINTER(ctype))
