"""There is no CPU path: without the library or without a GPU the product raises."""
import numpy as np
import pytest

from liteform_ae_amd import _lib
from liteform_ae_amd.format_matrix_market import MTX


def _has_gpu():
    import torch
    return torch.cuda.is_available()


def test_missing_library_raises(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/liblfhip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()


@pytest.mark.skipif(_has_gpu(), reason="only meaningful where no GPU is visible")
def test_operations_raise_without_gpu():
    from liteform_ae_amd import format_algos as fa
    g = MTX.from_coo(np.array([0, 1, 1]), np.array([0, 0, 1]), (2, 2))
    for call in (lambda: fa.search_bucket_config(g, 1, fa.CostModelSettings(32, 1)),
                 lambda: fa.build_hyb_format(g, [[1, 2]]),
                 lambda: fa.build_hyb_format_device(g, [[1, 2]]),
                 lambda: fa.bench_naive(g, np.ones((2, 32), np.float32), None, feat_size=32),
                 lambda: fa.choose_num_partitions(g, 32),
                 lambda: fa.choose_launch_shape(g, 128),
                 lambda: fa.matrix_features_device(g)):
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            call()


def test_package_does_not_import_the_oracle():
    """The oracle is test infrastructure; nothing shipped may reach for it."""
    import os
    import re
    root = os.path.dirname(os.path.abspath(_lib.__file__))
    for dirpath, _, files in os.walk(root):
        for name in files:
            if name.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(dirpath, name)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), name
