"""The C-ABI library loads without a GPU and exports every function the header declares."""
import ctypes
import os
import re

import pytest

from liteform_ae_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "liteform_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lf_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_something():
    names = declared_functions()
    assert "lf_spmm_run" in names and "lf_hyb_build" in names and len(names) >= 15


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} is not built (python -m liteform_ae_amd.build)")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"not exported: {missing}"


def test_binding_covers_header():
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_version_and_error_strings():
    lib = _lib.load()
    assert lib.lf_version() == 110
    assert lib.lf_status_string(0) == b"ok"
    assert b"single nonzero" in lib.lf_status_string(_lib.LF_ERR_TOO_SMALL)
    # an argument error is reported, not raised as a crash, and leaves a message
    rc = lib.lf_search_bucket_config(None, None, 1, 1024, 32, 1, 0, None, None, None, None)
    assert rc == _lib.LF_ERR_INVALID and "null" in _lib.last_error()


def test_layout_is_aligned():
    import numpy as np
    lib = _lib.load()
    ell = np.array([3, 0, 1000, 5], dtype=np.int64)
    w = np.array([1, 2, 4, 1024], dtype=np.int32)
    ro = np.zeros(4, np.int64)
    so = np.zeros(4, np.int64)
    tr, ts = ctypes.c_int64(), ctypes.c_int64()
    _lib.check(lib.lf_hyb_layout(_lib.np_ptr(ell, ctypes.c_int64), _lib.np_ptr(w, ctypes.c_int32), 4,
                                 _lib.np_ptr(ro, ctypes.c_int64), _lib.np_ptr(so, ctypes.c_int64),
                                 ctypes.byref(tr), ctypes.byref(ts)))
    assert (ro % 64 == 0).all() and (so % 1024 == 0).all()
    assert ro.tolist() == [0, 64, 64, 1088] and so.tolist() == [0, 1024, 1024, 5120]
    assert tr.value == 1152 and ts.value == 5120 + 5120
