"""Block-sparse fp16 SpMM (32 x 32 blocks, MFMA) against scipy BSR in float64.

Tolerance: inputs are exact fp16, products are accumulated in fp32 and the result is rounded
to fp16 once: |Y - ref| <= 2^-10 |ref| + 1e-5 * sum|a||x| + 1e-7."""
import numpy as np
import pytest
import scipy.sparse as sp

from oracle import liteform_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa():
    from liteform_ae_amd import format_algos
    return format_algos


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def random_bsr(rng, mb, nb, blocks_per_row, empty_rows=0, fill=1.0):
    indptr = [0]
    indices = []
    for i in range(mb):
        k = 0 if i < empty_rows else int(rng.integers(1, blocks_per_row + 1))
        cols = np.sort(rng.choice(nb, size=min(k, nb), replace=False))
        indices.extend(cols.tolist())
        indptr.append(len(indices))
    # fp16-representable values held as float32 (scipy's sparse containers refuse float16)
    data = rng.uniform(-1, 1, size=(len(indices), 32, 32)).astype(np.float16).astype(np.float32)
    if fill < 1.0:
        data[rng.random(data.shape) > fill] = 0
    return sp.bsr_matrix((data, np.array(indices, dtype=np.int32), np.array(indptr, dtype=np.int32)),
                         shape=(mb * 32, nb * 32))


def check(fa, torch, a, feat, seed=0):
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, size=(a.shape[1], feat)).astype(np.float16)
    y = fa.spmm_bsr(a, torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    ref = O.spmm_bsr_f64(a, x)
    bound = O.spmm_bsr_abs_bound(a, x)
    tol = 2.0 ** -10 * np.abs(ref) + 1e-5 * bound + 1e-7
    assert y.shape == ref.shape
    worst = float((np.abs(y - ref) - tol).max())
    assert worst <= 0, f"excess {worst}, max err {np.abs(y - ref).max()}"


@pytest.mark.parametrize("feat", [8, 32, 64, 128, 200, 256, 512])
def test_feature_sizes(fa, torch, feat):
    rng = np.random.default_rng(feat)
    check(fa, torch, random_bsr(rng, 40, 50, 6, empty_rows=3), feat, seed=feat)


def test_shapes_and_fill(fa, torch):
    rng = np.random.default_rng(2)
    check(fa, torch, random_bsr(rng, 1, 1, 1), 128)
    check(fa, torch, random_bsr(rng, 300, 7, 7), 128)                 # dense block rows
    check(fa, torch, random_bsr(rng, 7, 300, 40), 64)                 # long block rows
    check(fa, torch, random_bsr(rng, 100, 100, 5, fill=0.05), 128)    # sparse inside the blocks


def test_identity_and_empty(fa, torch):
    n = 64 * 32
    eye = sp.identity(n, dtype=np.float32, format="csr").tobsr(blocksize=(32, 32))
    x = torch.rand((n, 96), device="cuda").to(torch.float16)
    assert torch.equal(fa.spmm_bsr(eye, x), x)
    empty = sp.bsr_matrix((np.zeros((0, 32, 32), np.float32), np.zeros(0, np.int32), np.zeros(5, np.int32)),
                          shape=(4 * 32, 64 * 32))
    y = fa.spmm_bsr(empty, x)
    assert y.shape == (128, 96) and float(y.abs().max()) == 0.0


def test_reference_driver_branch(fa, torch, monkeypatch):
    """proc05.spmm.end-to-end.py:196-223: pad to a multiple of 32, fp16 BSR, half features."""
    from liteform_ae_amd.format_matrix_market import MTX
    rng = np.random.default_rng(4)
    n = 1000
    r = rng.integers(0, n, size=8000)
    c = rng.integers(0, n, size=8000)
    key = np.unique(r * n + c)
    g = MTX.from_coo(key // n, key % n, (n, n))
    padded = -(-n // 32) * 32
    bsr_weight = g.tobsr_with_padding(shape=(padded, padded), blocksize=(32, 32))
    x = torch.rand(bsr_weight.shape[1], 64).half()
    monkeypatch.setenv("LF_REPEAT", "3")
    monkeypatch.setenv("LF_WARMUP", "1")
    ms = fa.bench_bsrmm(bsr_weight, x, block_size=32)
    assert ms > 0 and np.isfinite(ms)
    y = fa.bench_bsrmm.last_output.cpu().numpy().astype(np.float64)
    ref = O.spmm_bsr_f64(bsr_weight, x.numpy())
    assert (np.abs(y - ref) <= 2.0 ** -10 * np.abs(ref) + 1e-5 * O.spmm_bsr_abs_bound(bsr_weight, x.numpy()) + 1e-7).all()
    with pytest.raises(NotImplementedError):
        fa.bench_bsrmm(g.tobsr_with_padding(shape=(1008, 1008), blocksize=(16, 16)), torch.rand(1008, 64).half(), 16)


def test_driver_block_and_csr_branches(fa, torch, monkeypatch):
    """proc05.spmm.end-to-end.py:191-261 through the driver: BSR, CSR, and the table's columns."""
    from liteform_ae_amd import driver
    from liteform_ae_amd.format_matrix_market import MTX
    rng = np.random.default_rng(6)
    n = 700
    key = np.unique(rng.integers(0, n, size=5000) * n + rng.integers(0, n, size=5000))
    g = MTX.from_coo(key // n, key % n, (n, n), name="toy")
    monkeypatch.setenv("LF_REPEAT", "2")
    monkeypatch.setenv("LF_WARMUP", "1")
    df = driver.run_end_to_end([g], feat_sizes=(32, 64), select_format=lambda m: "BSR")
    assert (df["format"] == "BSR").all() and (df["time_exe_our(ms)"] > 0).all() and (df["num_parts"] == 0).all()
    df = driver.run_end_to_end([g], feat_sizes=(64,), select_format=lambda m: "CSR")
    assert (df["format"] == "CSR").all() and (df["time_exe_our(ms)"] > 0).all()
