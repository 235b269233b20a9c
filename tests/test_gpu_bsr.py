"""Block-sparse fp16 SpMM (blocks of 16, 32 or 64, MFMA) against scipy BSR in float64.

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


def random_bsr(rng, mb, nb, blocks_per_row, empty_rows=0, fill=1.0, bs=32):
    indptr = [0]
    indices = []
    for i in range(mb):
        k = 0 if i < empty_rows else int(rng.integers(1, blocks_per_row + 1))
        cols = np.sort(rng.choice(nb, size=min(k, nb), replace=False))
        indices.extend(cols.tolist())
        indptr.append(len(indices))
    # fp16-representable values held as float32 (scipy's sparse containers refuse float16)
    data = rng.uniform(-1, 1, size=(len(indices), bs, bs)).astype(np.float16).astype(np.float32)
    if fill < 1.0:
        data[rng.random(data.shape) > fill] = 0
    return sp.bsr_matrix((data, np.array(indices, dtype=np.int32), np.array(indptr, dtype=np.int32)),
                         shape=(mb * bs, nb * bs))


def check(fa, torch, a, feat, seed=0):
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, size=(a.shape[1], feat)).astype(np.float16)
    y = fa.spmm_bsr(a, torch.from_numpy(x).cuda(), block_size=a.blocksize[0]).cpu().numpy().astype(np.float64)
    ref = O.spmm_bsr_f64(a, x)
    bound = O.spmm_bsr_abs_bound(a, x)
    tol = 2.0 ** -10 * np.abs(ref) + 1e-5 * bound + 1e-7
    assert y.shape == ref.shape
    worst = float((np.abs(y - ref) - tol).max())
    assert worst <= 0, f"excess {worst}, max err {np.abs(y - ref).max()}"


@pytest.mark.parametrize("bs", [16, 32, 64])
@pytest.mark.parametrize("feat", [8, 32, 64, 128, 200, 256, 512])
def test_feature_sizes(fa, torch, feat, bs):
    rng = np.random.default_rng(feat + bs)
    check(fa, torch, random_bsr(rng, 40, 50, 6, empty_rows=3, bs=bs), feat, seed=feat)


@pytest.mark.parametrize("bs", [16, 32, 64])
def test_shapes_and_fill(fa, torch, bs):
    rng = np.random.default_rng(2 + bs)
    check(fa, torch, random_bsr(rng, 1, 1, 1, bs=bs), 128)
    check(fa, torch, random_bsr(rng, 300, 7, 7, bs=bs), 128)                 # dense block rows
    check(fa, torch, random_bsr(rng, 7, 300, 40, bs=bs), 64)                 # long block rows
    check(fa, torch, random_bsr(rng, 100, 100, 5, fill=0.05, bs=bs), 128)    # sparse inside the blocks


@pytest.mark.parametrize("bs", [16, 32, 64])
def test_identity_and_empty(fa, torch, bs):
    n = 64 * 32
    eye = sp.identity(n, dtype=np.float32, format="csr").tobsr(blocksize=(bs, bs))
    x = torch.rand((n, 96), device="cuda").to(torch.float16)
    assert torch.equal(fa.spmm_bsr(eye, x, block_size=bs), x)
    empty = sp.bsr_matrix((np.zeros((0, bs, bs), np.float32), np.zeros(0, np.int32), np.zeros(5, np.int32)),
                          shape=(4 * bs, n))
    y = fa.spmm_bsr(empty, x, block_size=bs)
    assert y.shape == (4 * bs, 96) and float(y.abs().max()) == 0.0
    # a permutation of block columns with one entry per row: every output row is one row of x
    perm = np.random.default_rng(bs).permutation(n)
    pm = sp.csr_matrix((np.ones(n, np.float32), (np.arange(n), perm)), shape=(n, n)).tobsr(blocksize=(bs, bs))
    assert torch.equal(fa.spmm_bsr(pm, x, block_size=bs), x[torch.from_numpy(perm).cuda()])


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
    # the other block sizes the reference's schedule can take (any multiple of 16,
    # format_algos.py:1581-1582): 16 and 64 are served, the rest is refused
    for bs, side in ((16, 1008), (64, 1024)):
        w = g.tobsr_with_padding(shape=(side, side), blocksize=(bs, bs))
        xb = torch.rand(side, 64).half()
        assert fa.bench_bsrmm(w, xb, block_size=bs) > 0
        y = fa.bench_bsrmm.last_output.cpu().numpy().astype(np.float64)
        ref = O.spmm_bsr_f64(w, xb.numpy())
        assert (np.abs(y - ref) <= 2.0 ** -10 * np.abs(ref) + 1e-5 * O.spmm_bsr_abs_bound(w, xb.numpy()) + 1e-7).all()
    with pytest.raises(NotImplementedError):
        fa.bench_bsrmm(g.tobsr_with_padding(shape=(1008, 1008), blocksize=(48, 48)), torch.rand(1008, 64).half(), 48)


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
