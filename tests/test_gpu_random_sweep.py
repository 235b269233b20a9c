"""Seeded sweep over shapes, width configurations, partition counts, feature sizes and
operand types: format slabs bit-exact against the oracle's sequential builder, product
within 1e-5 * sum |a||b| of scipy CSR(f64) @ dense(f64)."""
import numpy as np
import pytest

from liteform_ae_amd.format_matrix_market import MTX
from oracle import liteform_oracle as O

from helpers import assert_hyb_equal

pytestmark = pytest.mark.gpu

WIDTHS = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024]


def random_case(seed):
    rng = np.random.default_rng(seed)
    nr = int(rng.integers(1, 900))
    nc = int(rng.integers(1, 1500))
    parts = int(rng.choice([1, 1, 2, 3, 5]))
    style = rng.integers(0, 4)
    if style == 0:                                   # short rows
        deg = rng.integers(0, min(nc, 6) + 1, size=nr)
    elif style == 1:                                 # log-normal with a few long rows
        deg = np.clip(np.rint(rng.lognormal(2.0, 1.2, size=nr)), 0, nc).astype(np.int64)
        deg[rng.integers(nr, size=2)] = min(nc, int(rng.integers(200, 1400)))
    elif style == 2:                                 # banded
        deg = np.full(nr, min(nc, int(rng.integers(3, 40))))
    else:                                            # every row long
        deg = rng.integers(min(nc, 100), min(nc, 700) + 1, size=nr)
    rows, cols = [], []
    for r, d in enumerate(deg):
        if d == 0:
            continue
        if style == 2:
            start = int(rng.integers(0, max(1, nc - d + 1)))
            c = np.arange(start, start + d)
        else:
            c = rng.choice(nc, size=int(d), replace=False)
        rows.append(np.full(len(c), r))
        cols.append(c)
    if rows:
        rows, cols = np.concatenate(rows), np.concatenate(cols)
    else:
        rows, cols = np.zeros(0, np.int64), np.zeros(0, np.int64)
    data = rng.uniform(-1, 1, size=len(rows)).astype(np.float32)
    g = MTX.from_coo(rows, cols, (nr, nc), data=data)
    widths = []
    for _ in range(parts):
        k = int(rng.integers(1, 6))
        widths.append(sorted(int(w) for w in rng.choice(WIDTHS, size=k, replace=False)))
    feat = int(rng.choice([32, 64, 128, 256, 512, 96, 1024]))
    b_dtype = "bf16" if (feat % 64 == 0 and rng.random() < 0.3) else "f32"
    return g, widths, feat, b_dtype


@pytest.mark.parametrize("block", range(12))
def test_random_sweep(block):
    import torch
    from liteform_ae_amd import format_algos as fa
    for seed in range(block * 20, block * 20 + 20):
        g, widths, feat, b_dtype = random_case(9000 + seed)
        tag = f"seed {9000 + seed}: shape {g.coo_mtx.shape}, nnz {g.num_edges()}, widths {widths}, N {feat}, {b_dtype}"
        if g.num_edges() < 60000:                    # the sequential oracle is a Python loop
            ones = MTX.from_coo(g.coo_mtx.row, g.coo_mtx.col, g.coo_mtx.shape)
            assert_hyb_equal(fa.build_hyb_format(ones, widths), O.build_hyb_format_sequential(ones, widths))
        nr, nc = g.coo_mtx.shape
        rng = np.random.default_rng(seed)
        B = rng.uniform(-1, 1, size=(nc, feat)).astype(np.float32)
        if b_dtype == "bf16":
            Bt = torch.from_numpy(B).to(torch.bfloat16)
            B, Bd = Bt.to(torch.float32).numpy(), Bt.cuda()
        else:
            Bd = torch.from_numpy(B).cuda()
        plan = fa.HybSpMM(fa.build_hyb_format_device(g, widths), feat, b_dtype)
        C = plan.run(Bd).cpu().numpy()
        plan.close()
        indptr, indices, data = g.adj_tensors("csr")
        data = np.asarray(data, dtype=np.float32)
        ref = O.spmm_csr_f64(indptr, indices, data, (nr, nc), B)
        bound = O.spmm_abs_bound(indptr, indices, data, (nr, nc), B)
        err = np.abs(C.astype(np.float64) - ref)
        assert C.shape == ref.shape, tag
        assert (err <= 1e-5 * bound).all(), f"{tag}: max excess {(err - 1e-5 * bound).max()}"
