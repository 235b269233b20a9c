"""MI355X-native implementation of LiteForm's CELL/hyb SpMM path.

Public names follow the reference's ``format_algos`` / ``format_matrix_market``
modules so that its driver flow runs unchanged:

    from liteform_ae_amd import (MTX, CostModelSettings, search_bucket_config,
                                 build_hyb_format, bench_hyb_with_config)
"""
from .format_matrix_market import MTX, Bucket  # noqa: F401

__version__ = "0.1.0"


def __getattr__(name):
    # format_algos needs torch and the HIP library; load it on first use so that
    # the container classes stay importable on their own.
    if name in ("CostModelSettings", "search_bucket_config", "build_hyb_format",
                "bench_hyb_with_config", "bench_naive", "bench_bsrmm", "HybFormat", "build_hyb_format_device"):
        from . import format_algos
        return getattr(format_algos, name)
    raise AttributeError(name)
