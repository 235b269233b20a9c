"""Seeded random cases across the SpMM paths: skewed, wide, dense-row, stencil and banded
matrices with random feature counts, operand types, column partitions, feature windows and cost
models, each against scipy CSR(f64) @ dense(f64) under the bound 1e-5 * sum|a||b| (and
bit-reproducible run to run).  The case table is a function of the seed alone."""
import numpy as np
import pytest

from helpers import skewed_matrix
from test_gpu_spmm import banded_matrix, check, grid_stencil

pytestmark = pytest.mark.gpu


def random_case(seed):
    rng = np.random.default_rng(seed)
    kind = str(rng.choice(["skew", "grid3", "grid2", "band", "dense", "skew_wide"]))
    if kind == "skew":
        g = skewed_matrix(rng, int(rng.integers(50, 6000)), int(rng.integers(50, 9000)), mean_deg=float(rng.uniform(1, 20)),
                          heavy_rows=int(rng.integers(0, 4)), heavy_len=int(rng.integers(10, 5000)))
    elif kind == "skew_wide":
        g = skewed_matrix(rng, int(rng.integers(50, 2000)), int(rng.integers(20000, 400000)), mean_deg=float(rng.uniform(1, 8)),
                          heavy_rows=int(rng.integers(1, 4)), heavy_len=int(rng.integers(5000, 150000)))
    elif kind == "grid3":
        g = grid_stencil(rng, tuple(int(x) for x in rng.integers(5, 40, size=3)))
    elif kind == "grid2":
        g = grid_stencil(rng, tuple(int(x) for x in rng.integers(20, 220, size=2)), reach=int(rng.integers(1, 3)))
    elif kind == "band":
        g = banded_matrix(rng, int(rng.integers(4100, 12000)), int(rng.integers(2, 30)), block=int(rng.choice([1, 1, 4])))
    else:
        g = skewed_matrix(rng, int(rng.integers(100, 800)), int(rng.integers(150000, 700000)), mean_deg=4,
                          heavy_rows=int(rng.integers(1, 4)), heavy_len=int(rng.integers(20000, 120000)))
    dt = str(rng.choice(["f32", "f32", "bf16"]))
    feat = int(rng.choice([32, 64, 96, 128, 160, 256, 512] if dt == "f32" else [64, 128, 256, 512]))
    parts = int(rng.choice([1, 1, 2, 3]))
    windows = int(rng.choice([w for w in (1, 2, 4) if feat % w == 0 and (feat // w) % (64 if dt == "bf16" else 32) == 0]))
    if kind in ("grid3", "grid2", "band") and rng.random() < 0.7:           # the shapes the cells take
        dt, per, windows = "f32", int(rng.choice([128, 256])), int(rng.choice([1, 2, 4]))
        feat = per * windows
        if feat > 1024:
            feat, windows = per, 1
    model = str(rng.choice(["gfx950", "reference"]))
    if g.num_dst_nodes() * feat * 4 > 600e6:                                 # keep B and its float64 copy small
        feat, windows = (64 if dt == "bf16" else 32), 1
    return g, dt, feat, parts, windows, model


@pytest.mark.parametrize("seed", range(3000, 3060))
def test_random_case(seed):
    import torch
    from liteform_ae_amd import format_algos as fa
    g, dt, feat, parts, windows, model = random_case(seed)
    try:
        widths = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts, cost_model=model))
    except ValueError:
        pytest.skip("a column partition holds a single nonzero (the reference raises too)")
    check(fa, torch, g, widths, feat, dt, seed=seed, windows=windows)


def random_structured_case(seed):
    """Stencils and bands in the shapes the 16-row cells take: fp32, 128 or 256 features per pass."""
    rng = np.random.default_rng(seed)
    kind = str(rng.choice(["grid3", "grid3", "grid2", "band"]))
    if kind == "grid3":
        g = grid_stencil(rng, tuple(int(x) for x in rng.integers(5, 40, size=3)))
    elif kind == "grid2":
        g = grid_stencil(rng, tuple(int(x) for x in rng.integers(20, 220, size=2)), reach=int(rng.integers(1, 3)))
    else:
        g = banded_matrix(rng, int(rng.integers(4100, 12000)), int(rng.integers(2, 30)), block=int(rng.choice([1, 1, 4])))
    per, windows = int(rng.choice([128, 256])), int(rng.choice([1, 1, 2]))
    parts = int(rng.choice([1, 1, 2, 3]))
    model = str(rng.choice(["gfx950", "reference"]))
    return g, per * windows, parts, windows, model


@pytest.mark.parametrize("seed", range(5000, 5024))
def test_random_structured_case(seed):
    # quarters of a cell that lack a column are skipped, cells at the edge of a grid hold fewer than
    # 16 rows, partitions after the first add to C: all of it varies with the grid's shape
    import torch
    from liteform_ae_amd import format_algos as fa
    g, feat, parts, windows, model = random_structured_case(seed)
    try:
        widths = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts, cost_model=model))
    except ValueError:
        pytest.skip("a column partition holds a single nonzero (the reference raises too)")
    check(fa, torch, g, widths, feat, "f32", seed=seed, windows=windows)
