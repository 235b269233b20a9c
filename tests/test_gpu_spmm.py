"""GPU parity of the fused hyb SpMM with scipy CSR(f64) @ dense(f64).

Tolerance (stated by the task): |C - C_ref| <= 1e-5 * sum_k |a_ik| |b_kj| per element."""
import numpy as np
import pytest
import scipy.sparse as sp

from oracle import liteform_oracle as O

from liteform_ae_amd.format_matrix_market import MTX

from helpers import skewed_matrix

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def fa():
    from liteform_ae_amd import format_algos
    return format_algos


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def to_bf16_exact(torch, B):
    return torch.from_numpy(B).to(torch.bfloat16)


def check(fa, torch, g, widths, feat, b_dtype="f32", seed=0, windows=1):
    rng = np.random.default_rng(seed)
    nr, nc = g.coo_mtx.shape
    B = rng.uniform(-1, 1, size=(nc, feat)).astype(np.float32)
    if b_dtype == "bf16":
        Bt = to_bf16_exact(torch, B)
        B = Bt.to(torch.float32).numpy()
        Bd = Bt.cuda()
    else:
        Bd = torch.from_numpy(B).cuda()
    fmt = fa.build_hyb_format_device(g, widths)
    plan = fa.HybSpMM(fmt, feat, b_dtype, windows=windows)
    C1 = plan.run(Bd).cpu().numpy()
    C2 = plan.run(Bd).cpu().numpy()
    plan.close()
    np.testing.assert_array_equal(C1, C2)              # run-to-run bit reproducible
    indptr, indices, data = g.adj_tensors("csr")
    data = np.asarray(data, dtype=np.float32)
    ref = O.spmm_csr_f64(indptr, indices, data, (nr, nc), B)
    bound = O.spmm_abs_bound(indptr, indices, data, (nr, nc), B)
    err = np.abs(C1.astype(np.float64) - ref)
    worst = float((err - TOL * bound).max()) if err.size else 0.0
    assert worst <= 0, f"max excess over 1e-5*bound: {worst}; max err {err.max()}"
    return C1, plan.info


@pytest.mark.parametrize("feat", [32, 64, 128, 256, 512, 96])
def test_feature_sizes(fa, torch, feat):
    rng = np.random.default_rng(feat)
    g = skewed_matrix(rng, 3000, 2500, mean_deg=7, heavy_rows=3, heavy_len=1800)
    cfg = fa.search_bucket_config(g, 1, fa.CostModelSettings(feat, 1))
    check(fa, torch, g, cfg, feat, seed=feat)


@pytest.mark.parametrize("parts", [1, 2, 3, 8])
def test_column_partitions(fa, torch, parts):
    rng = np.random.default_rng(parts)
    g = skewed_matrix(rng, 4000, 5000, mean_deg=10, heavy_rows=4, heavy_len=3000)
    cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(128, parts))
    check(fa, torch, g, cfg, 128, seed=parts)


@pytest.mark.parametrize("widths", [[[1]], [[2]], [[4]], [[8]], [[16]], [[64]], [[256]], [[1024]],
                                    [[1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024]], [[4, 32]]])
def test_every_width_path(fa, torch, widths):
    """Each width as the only (hence widest, row-splitting) bucket, then all widths at once."""
    rng = np.random.default_rng(len(widths[0]) * 1000 + widths[0][0])
    g = skewed_matrix(rng, 1500, 2000, mean_deg=9, heavy_rows=3, heavy_len=4000)
    check(fa, torch, g, widths, 128)


@pytest.mark.parametrize("feat,b_dtype", [(32, "f32"), (64, "f32"), (128, "f32"), (256, "f32"), (512, "f32"),
                                          (64, "bf16"), (256, "bf16"), (1024, "bf16")])
def test_folded_configurations_split_rows_over_ell_rows(fa, torch, feat, b_dtype):
    """Widest bucket narrower than most rows: segments of 2..8 ELL rows (many cross a tile
    boundary), summed row by row through LDS where the tile's partial sums fit."""
    rng = np.random.default_rng(500 + feat)
    g = skewed_matrix(rng, 2500, 3000, mean_deg=40, heavy_rows=3, heavy_len=2000)
    plain = fa.HybSpMM(fa.build_hyb_format_device(g, [[1024]]), feat, b_dtype)
    static_lds = plain.info["lds_bytes"]
    plain.close()
    for widths in ([[8]], [[16]], [[32]], [[1, 2, 4, 8, 16, 32]], [[64]], [[4, 16], [2, 32]]):
        _, info = check(fa, torch, g, widths, feat, b_dtype, seed=feat)
        lpr = min(64, feat // (8 if b_dtype == "bf16" else 4))
        rows_per_tile = max(512, 64 * 256 // lpr) // widths[0][-1]
        if rows_per_tile * feat * 4 <= 16384 and len(widths) == 1:
            assert info["lds_bytes"] > static_lds, (widths, info)


@pytest.mark.parametrize("feat,b_dtype", [(32, "f32"), (64, "f32"), (128, "f32"), (256, "f32"), (128, "bf16")])
def test_small_matrix_with_narrow_row_splitting_bucket(fa, torch, feat, b_dtype):
    """Few rows, widest bucket of 1, 2 or 4 slots: short tiles, so the per-ELL-row sums of a
    split row go through LDS with fewer slots per row than gathers in flight."""
    rng = np.random.default_rng(700 + feat)
    g = skewed_matrix(rng, 300, 400, mean_deg=5, heavy_rows=2, heavy_len=90)
    for widths in ([[1]], [[2]], [[4]], [[1, 2]], [[2, 4]], [[1], [2]], [[4], [1, 2]]):
        check(fa, torch, g, widths, feat, b_dtype, seed=feat)


@pytest.mark.parametrize("feat,b_dtype", [(32, "f32"), (128, "f32"), (512, "bf16")])
def test_very_long_rows_are_split_into_chunks(fa, torch, feat, b_dtype):
    rng = np.random.default_rng(77)
    g = skewed_matrix(rng, 600, 40000, mean_deg=5, heavy_rows=2, heavy_len=30000)
    for widths in ([[1, 2, 4, 8, 16]], [[8, 1024]]):
        _, info = check(fa, torch, g, widths, feat, b_dtype)
        assert info["heavy_rows"] >= 2 and info["partial_rows"] >= 2 * 8


def test_every_row_takes_the_cooperative_path(fa, torch):
    """A matrix of long rows only: every lane of the table-building pass owns a heavy row,
    single-chunk rows (<= 2048 slots) and multi-chunk rows mixed."""
    rng = np.random.default_rng(91)
    nr, nc = 700, 6000
    deg = rng.integers(300, 5000, size=nr)
    rows = np.repeat(np.arange(nr), deg)
    cols = np.concatenate([rng.choice(nc, size=d, replace=False) for d in deg])
    g = MTX.from_coo(rows, cols, (nr, nc), data=rng.uniform(-1, 1, size=len(rows)).astype(np.float32))
    for widths in ([[16]], [[256, 1024]], [[8, 64], [1024]]):
        _, info = check(fa, torch, g, widths, 64, seed=5)
        assert info["heavy_rows"] > 0 and info["partial_rows"] > 0


@pytest.mark.parametrize("feat,b_dtype", [(768, "f32"), (1024, "f32"), (1024, "bf16"), (32, "bf16"), (160, "f32")])
def test_wide_and_odd_feature_sizes(fa, torch, feat, b_dtype):
    """Several 16-byte chunks per lane (N > 256 fp32, N > 512 bf16) and lanes past the end."""
    rng = np.random.default_rng(feat)
    g = skewed_matrix(rng, 700, 900, mean_deg=6, heavy_rows=2, heavy_len=2500)
    for widths in ([[1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024]], [[2, 16]]):
        check(fa, torch, g, widths, feat, b_dtype, seed=feat)


def test_bf16_dense_operand(fa, torch):
    rng = np.random.default_rng(5)
    g = skewed_matrix(rng, 2000, 3000, mean_deg=8, heavy_rows=3, heavy_len=2500)
    for feat in (64, 128, 512):
        for parts in (1, 2):
            cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts))
            check(fa, torch, g, cfg, feat, "bf16", seed=feat + parts)


def test_library_special_cases(fa, torch):
    n, feat = 777, 64
    rng = np.random.default_rng(1)
    B = rng.uniform(-1, 1, size=(n, feat)).astype(np.float32)
    Bd = torch.from_numpy(B).cuda()
    from liteform_ae_amd.format_matrix_market import MTX
    # identity -> C == B exactly
    g = MTX.from_coo(np.arange(n), np.arange(n), (n, n))
    C = fa.spmm_hyb(fa.build_hyb_format_device(g, [[1]]), Bd).cpu().numpy()
    np.testing.assert_array_equal(C, B)
    # diagonal -> row scaling, exact in fp32 (one product per element)
    d = rng.uniform(-2, 2, size=n).astype(np.float32)
    g = MTX.from_coo(np.arange(n), np.arange(n), (n, n), data=d)
    C = fa.spmm_hyb(fa.build_hyb_format_device(g, [[1]]), Bd).cpu().numpy()
    np.testing.assert_array_equal(C, d[:, None] * B)
    # permutation -> gather
    perm = rng.permutation(n)
    g = MTX.from_coo(np.arange(n), perm, (n, n))
    C = fa.spmm_hyb(fa.build_hyb_format_device(g, [[1]]), Bd).cpu().numpy()
    np.testing.assert_array_equal(C, B[perm])
    # one dense row of ones -> column sums
    g = MTX.from_coo(np.zeros(n, dtype=np.int64), np.arange(n), (3, n))
    C = fa.spmm_hyb(fa.build_hyb_format_device(g, [[64]]), Bd).cpu().numpy()
    np.testing.assert_allclose(C[0], B.astype(np.float64).sum(0), rtol=0, atol=1e-5 * np.abs(B).sum(0).max())
    assert (C[1:] == 0).all()                      # rows without nonzeros are cleared
    # all-ones A with small-integer B is exact whatever the summation order
    a = sp.random(500, n, 0.05, random_state=3, format="csr")
    a.data[:] = 1
    g = MTX(None)
    g.coo_mtx = a.tocoo()
    Bi = rng.integers(-4, 5, size=(n, feat)).astype(np.float32)
    for parts in (1, 3):
        cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts))
        C = fa.spmm_hyb(fa.build_hyb_format_device(g, cfg), torch.from_numpy(Bi).cuda()).cpu().numpy()
        np.testing.assert_array_equal(C, (a @ Bi.astype(np.float64)).astype(np.float32))


def test_stale_output_is_overwritten(fa, torch):
    """C needs no clearing: every row is written by the first partition's launch."""
    rng = np.random.default_rng(9)
    g = skewed_matrix(rng, 1000, 1000, mean_deg=3, heavy_rows=0)
    cfg = fa.search_bucket_config(g, 2, fa.CostModelSettings(64, 2))
    fmt = fa.build_hyb_format_device(g, cfg)
    B = torch.rand((1000, 64), device="cuda") - 0.5
    plan = fa.HybSpMM(fmt, 64)
    c0 = plan.run(B).clone()
    junk = torch.full((1000, 64), float("nan"), device="cuda")
    plan.run(B, junk)
    plan.close()
    assert torch.equal(c0, junk)


def test_reference_style_driver_flow(fa, torch, monkeypatch):
    """proc05.spmm.end-to-end.py:153-176 with ones as features and the mask as values."""
    rng = np.random.default_rng(21)
    g = skewed_matrix(rng, 1200, 1200, mean_deg=6, heavy_rows=2, values=False)
    feat, parts = 64, 2
    cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat_size=feat, num_parts=parts))
    x = torch.ones((g.num_dst_nodes(), feat))
    y = g.dot(x.numpy())
    hyb = fa.build_hyb_format(g, cfg)
    monkeypatch.setenv("LF_REPEAT", "3")
    monkeypatch.setenv("LF_WARMUP", "1")
    ms = fa.bench_hyb_with_config(g, x, y, feat_size=feat, bucket_widths=cfg, bucketing_format=hyb,
                                  coarsening_factor=2, num_col_parts=parts, use_implicit_unroll=True,
                                  check_correctness=True)
    assert ms > 0 and np.isfinite(ms)
    np.testing.assert_array_equal(fa.bench_hyb_with_config.last_output.cpu().numpy(), y.astype(np.float32))
    ms = fa.bench_naive(g, x, y, feat_size=feat, check_correctness=True)
    assert ms > 0


def test_csr_kernel(fa, torch):
    rng = np.random.default_rng(31)
    g = skewed_matrix(rng, 2500, 1800, mean_deg=9, heavy_rows=2, heavy_len=1500)
    B = rng.uniform(-1, 1, size=(1800, 128)).astype(np.float32)
    C = fa.spmm_csr(g, torch.from_numpy(B).cuda()).cpu().numpy()
    indptr, indices, data = g.adj_tensors("csr")
    ref = O.spmm_csr_f64(indptr, indices, data, g.coo_mtx.shape, B)
    bound = O.spmm_abs_bound(indptr, indices, data, g.coo_mtx.shape, B)
    assert (np.abs(C - ref) <= TOL * bound).all()


def test_workloads_scaled(fa, torch):
    from liteform_ae_amd.synthetic import make_workload
    for name, scale, parts in (("cfg1", 1.0, 1), ("cfg2", 0.05, 2), ("cfg3", 0.005, 1), ("cfg4", 0.004, 1),
                               ("cfg5", 0.01, 2)):
        wl = make_workload(name, scale)
        cfg = fa.search_bucket_config(wl.matrix, parts, fa.CostModelSettings(wl.feat_size, parts))
        check(fa, torch, wl.matrix, cfg, wl.feat_size, wl.b_dtype, seed=wl.seed)


def test_partition_chooser_and_driver_table(fa, torch, monkeypatch):
    from liteform_ae_amd import driver
    rng = np.random.default_rng(41)
    g = skewed_matrix(rng, 3000, 3000, mean_deg=8, heavy_rows=2, values=False)
    g.name = "toy"
    best, timings = fa.choose_num_partitions(g, 64, candidates=(1, 2), return_timings=True)
    assert best in timings and set(timings) == {1, 2}
    assert fa.guess_num_partitions(g, 64) == 1            # B is far smaller than the memory-side cache
    monkeypatch.setenv("LF_REPEAT", "2")
    monkeypatch.setenv("LF_WARMUP", "1")
    df = driver.run_end_to_end([g], feat_sizes=(32, 64), num_parts=2, check_correctness=True)
    assert list(df.columns[:8]) == ["name", "format", "feat_size", "num_parts", "time_select(s)",
                                    "time_num_parts(s)", "time_bucket(s)", "time_exe_our(ms)"]
    assert len(df) == 2 and (df["format"] == "CELL").all() and np.isfinite(df["time_exe_our(ms)"]).all()
    # a matrix with values: the check compares with the values the format is composed with
    # (ones by default, like the reference's matrices; the matrix's own with keep_values)
    gw = skewed_matrix(rng, 2000, 2500, mean_deg=6, heavy_rows=1)
    gw.name = "weighted"
    for keep in (False, True):
        df = driver.run_end_to_end([gw], feat_sizes=(64,), cost_model="gfx950", check_correctness=True, keep_values=keep)
        assert np.isfinite(df["time_exe_our(ms)"]).all(), keep
    # the reference's driver sets the partition count of two graphs by name, whatever its
    # predictor says (proc05.spmm.end-to-end.py:145-148): the override table does the same
    g.name = "ppi"
    df = driver.run_end_to_end([g, gw], feat_sizes=(64,), check_correctness=True,
                               num_parts_override=driver.REFERENCE_NUM_PARTS_OVERRIDE)
    assert df["num_parts"].tolist() == [16, 1] and np.isfinite(df["time_exe_our(ms)"]).all()


@pytest.mark.parametrize("feat,b_dtype,windows", [(128, "f32", 2), (256, "f32", 4), (512, "f32", 2), (256, "bf16", 2),
                                                  (1024, "bf16", 4), (96, "f32", 3)])
def test_feature_windows_match_single_pass(fa, torch, feat, b_dtype, windows):
    """The product in several passes over feature windows: within tolerance of the oracle and
    equal to the single-pass result on rows that are summed slot by slot in one ELL row (split
    and cooperatively reduced rows are summed in pieces whose size follows the lane count)."""
    rng = np.random.default_rng(800 + feat)
    g = skewed_matrix(rng, 2000, 2600, mean_deg=12, heavy_rows=3, heavy_len=2400)
    nr, nc = g.coo_mtx.shape
    B = rng.uniform(-1, 1, size=(nc, feat)).astype(np.float32)
    Bd = torch.from_numpy(B).cuda()
    if b_dtype == "bf16":
        Bd = Bd.to(torch.bfloat16)
        B = Bd.to(torch.float32).cpu().numpy()
    indptr, indices, data = g.adj_tensors("csr")
    data = np.asarray(data, dtype=np.float32)
    ref = O.spmm_csr_f64(indptr, indices, data, (nr, nc), B)
    bound = O.spmm_abs_bound(indptr, indices, data, (nr, nc), B)
    for widths in ([[1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024]], [[4, 32]], [[2, 16], [8, 64]]):
        fmt = fa.build_hyb_format_device(g, widths)
        one = fa.HybSpMM(fmt, feat, b_dtype)
        many = fa.HybSpMM(fmt, feat, b_dtype, windows=windows)
        assert many.info["windows"] == windows and many.info["launches"] == windows * one.info["launches"]
        C1 = one.run(Bd).cpu().numpy()
        Cw = many.run(Bd).cpu().numpy()
        Cw2 = torch.full((nr, feat), 7.0, device="cuda")          # stale output is overwritten
        many.run(Bd, Cw2)
        one.close()
        many.close()
        np.testing.assert_array_equal(Cw, Cw2.cpu().numpy())
        assert (np.abs(Cw.astype(np.float64) - ref) <= TOL * bound).all()
        if len(widths[0]) == 11:          # every width present: a row up to 128 entries is one ELL row,
            light = np.diff(indptr) <= 128        # summed slot by slot whatever the lane count
            np.testing.assert_array_equal(Cw[light], C1[light])
    with pytest.raises(ValueError):
        fa.HybSpMM(fmt, feat, b_dtype, windows=7)


def banded_matrix(rng, n, half_width, block=1):
    """Rows hold the columns within half_width of the diagonal (clipped), in blocks of
    `block` identical rows: consecutive rows share most (block > 1: all) of their columns."""
    rows, cols = [], []
    for r in range(n):
        c0 = (r // block) * block
        lo, hi = max(0, c0 - half_width), min(n, c0 + half_width + 1)
        rows.append(np.full(hi - lo, r))
        cols.append(np.arange(lo, hi))
    rows, cols = np.concatenate(rows), np.concatenate(cols)
    return MTX.from_coo(rows, cols, (n, n), data=rng.uniform(-1, 1, size=len(rows)).astype(np.float32))


def mixed_band_matrix(rng, n):
    """Bands of 7, 13, 25 and 49 columns in turn, 2000 rows each: four buckets, all shared."""
    rows, cols = [], []
    for r in range(n):
        half = (3, 6, 12, 24)[(r // 2000) % 4]
        lo, hi = max(0, r - half), min(n, r + half + 1)
        rows.append(np.full(hi - lo, r))
        cols.append(np.arange(lo, hi))
    rows, cols = np.concatenate(rows), np.concatenate(cols)
    return MTX.from_coo(rows, cols, (n, n), data=rng.uniform(-1, 1, size=len(rows)).astype(np.float32))


@pytest.mark.parametrize("feat,b_dtype,parts,nc", [(64, "f32", 1, 640_000), (128, "bf16", 1, 640_000),
                                                   (256, "f32", 2, 320_000), (512, "bf16", 1, 160_000)])
def test_dense_rows_are_walked_in_column_order(fa, torch, feat, b_dtype, parts, nc, monkeypatch):
    """Rows holding a large share of the columns are cut into short chunks that are walked in
    column order and added up by a whole workgroup; the product is the same (to rounding) as
    with the chunks of ordinary long rows, and bit-reproducible.  (Only where a partition's
    part of B is larger than the memory-side cache: 160 MB here.)"""
    rng = np.random.default_rng(500 + feat)
    nr = 3000
    g = skewed_matrix(rng, nr, nc, mean_deg=6, heavy_rows=3, heavy_len=90_000)      # 88 chunks of 1024 per dense row
    widths = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts, cost_model="gfx950"))
    C1, info = check(fa, torch, g, widths, feat, b_dtype, seed=feat)
    assert info["partial_rows"] >= 3 * 64                            # more than 64 a row: added up by a whole workgroup (one partition)
    monkeypatch.setenv("LF_DENSE_ROWS", "0")
    C0, info0 = check(fa, torch, g, widths, feat, b_dtype, seed=feat)
    monkeypatch.delenv("LF_DENSE_ROWS")
    assert info0["partial_rows"] < info["partial_rows"]
    indptr, _, data = g.adj_tensors("csr")
    row_abs = np.add.reduceat(np.abs(np.asarray(data, dtype=np.float64)), np.minimum(indptr[:-1], len(data) - 1))
    row_abs[np.diff(indptr) == 0] = 0
    assert (np.abs(C1 - C0) <= 2e-5 * row_abs[:, None] + 1e-30).all()


def test_very_long_row_is_added_up_by_a_workgroup(fa, torch):
    """A row of ~170,000 entries in a small matrix (B fits the memory-side cache, so nothing is
    reordered): over 80 chunks of 2048 slots, more partial rows than a sub-wave adds up alone."""
    rng = np.random.default_rng(77)
    g = skewed_matrix(rng, 500, 300_000, mean_deg=5, heavy_rows=1, heavy_len=260_000)
    widths = fa.search_bucket_config(g, 1, fa.CostModelSettings(32, 1, cost_model="gfx950"))
    _, info = check(fa, torch, g, widths, 32, "f32", seed=3)
    assert info["partial_rows"] > 64
    _, info = check(fa, torch, g, widths, 96, "f32", seed=4)          # three 16-byte chunks per lane, one unused
    assert info["partial_rows"] > 64


def grid_stencil(rng, dims, reach=1):
    """Every point of a grid (first dimension fastest) coupled to its neighbours within `reach`
    in every direction: 9 columns per interior row in two dimensions, 27 in three."""
    shape = tuple(reversed(dims))
    idx = np.arange(int(np.prod(dims))).reshape(shape)
    rows, cols = [], []
    offsets = np.stack(np.meshgrid(*[np.arange(-reach, reach + 1)] * len(dims), indexing="ij"), -1).reshape(-1, len(dims))
    for off in offsets:
        src = tuple(slice(max(0, -o), s - max(0, o)) for o, s in zip(off, shape))
        dst = tuple(slice(max(0, o), s - max(0, -o)) for o, s in zip(off, shape))
        rows.append(idx[src].ravel())
        cols.append(idx[dst].ravel())
    rows, cols = np.concatenate(rows), np.concatenate(cols)
    n = idx.size
    return MTX.from_coo(rows, cols, (n, n), data=rng.uniform(-1, 1, size=len(rows)).astype(np.float32))


@pytest.mark.parametrize("feat,windows,b_dtype", [(256, 1, "f32"), (512, 2, "f32"), (128, 1, "f32"), (256, 2, "f32"),
                                                  (512, 4, "f32")])
def test_grid_stencils_are_served_as_cells(fa, torch, feat, windows, b_dtype, monkeypatch):
    """fp32 B, 128 or 256 features per pass: buckets of a stencil become 16-row cells
    (neighbours in every direction of the grid, found from the column differences) on the
    matrix cores; the product is the plain path's to rounding and within the bound of the
    float64 oracle."""
    rng = np.random.default_rng(77 + feat)
    for g, widths in ((grid_stencil(rng, (37, 29, 23)), [[8, 16, 32]]),        # 27 points, ragged cell edges
                      (grid_stencil(rng, (150, 131)), [[4, 8, 16]]),           # 9 points, two strides
                      (grid_stencil(rng, (64, 40, 16)), [[32]]),               # one bucket for faces and interior
                      (banded_matrix(rng, 9001, 10), [[8, 16, 32]])):          # one stride
        C1, info = check(fa, torch, g, widths, feat, b_dtype, seed=feat, windows=windows)
        assert info["cell_buckets"] >= 1, (widths, info)
        monkeypatch.setenv("LF_ROW_GROUPS", "4")
        C4, info4 = check(fa, torch, g, widths, feat, b_dtype, seed=feat, windows=windows)
        monkeypatch.setenv("LF_ROW_GROUPS", "0")
        C0, info0 = check(fa, torch, g, widths, feat, b_dtype, seed=feat, windows=windows)
        monkeypatch.delenv("LF_ROW_GROUPS")
        assert info4["cell_buckets"] == 0 and info4["row_group_buckets"] >= 1
        assert info0["row_group_buckets"] == 0
        # same terms per row on all three paths (the cells add them as one or two interleaved
        # partial sums): they differ only in rounding (|a|, |b| < 1, at most 27 terms)
        assert np.abs(C1 - C0).max() <= 2e-5 and np.abs(C4 - C0).max() <= 2e-5
    g = skewed_matrix(rng, 20000, 30000, mean_deg=20, heavy_rows=0)
    _, info = check(fa, torch, g, [[8, 16, 32, 64]], feat, b_dtype, seed=feat, windows=windows)
    assert info["cell_buckets"] == 0


@pytest.mark.parametrize("feat,windows", [(256, 1), (128, 1), (512, 2)])
def test_cells_in_two_column_partitions(fa, torch, feat, windows, monkeypatch):
    """Cells in both column partitions: the first partition's cell launch stores C with ordinary
    stores (the second one reads it again), the second one adds to C and streams its stores.
    Rows on the grid plane where the partitions meet take terms from both."""
    rng = np.random.default_rng(300 + feat)
    for g, widths in ((grid_stencil(rng, (64, 40, 16)), [[32], [32]]),
                      (grid_stencil(rng, (37, 29, 23)), None),
                      (grid_stencil(rng, (150, 131)), [[4, 8, 16], [4, 8, 16]])):
        if widths is None:
            widths = fa.search_bucket_config(g, 2, fa.CostModelSettings(feat, 2, cost_model="gfx950"))
        C1, info = check(fa, torch, g, widths, feat, "f32", seed=feat, windows=windows)
        assert info["cell_buckets"] >= 2, (widths, info)              # at least one bucket of either partition
        monkeypatch.setenv("LF_ROW_GROUPS", "0")
        C0, info0 = check(fa, torch, g, widths, feat, "f32", seed=feat, windows=windows)
        monkeypatch.delenv("LF_ROW_GROUPS")
        assert info0["row_group_buckets"] == 0
        assert np.abs(C1 - C0).max() <= 2e-5


@pytest.mark.parametrize("feat", [96, 160, 224])
def test_feature_counts_that_leave_lanes_unused_stay_with_row_groups(fa, torch, feat):
    """160 features take 40 of 64 lanes: the lane layout of the 256-feature kernels, but not the
    cells' (they want every lane of the row to hold features)."""
    rng = np.random.default_rng(feat)
    _, info = check(fa, torch, grid_stencil(rng, (30, 22, 17)), [[8, 16, 32]], feat, "f32", seed=feat)
    assert info["cell_buckets"] == 0 and info["row_group_buckets"] >= 1


@pytest.mark.parametrize("feat,b_dtype", [(32, "f32"), (64, "f32"), (128, "f32"), (256, "f32"), (256, "bf16"),
                                          (512, "bf16")])
def test_rows_sharing_columns_are_served_in_groups(fa, torch, feat, b_dtype, monkeypatch):
    """Banded and block-structured matrices: buckets whose consecutive rows share columns are
    processed four rows at a time with shared gathers; a random matrix never is."""
    rng = np.random.default_rng(900 + feat)
    for g, widths in ((banded_matrix(rng, 9001, 10), [[8, 16, 32]]),          # 21 per row, last group partial
                      (banded_matrix(rng, 6000, 7, block=4), [[16]]),          # 4 x 1 blocks: all columns shared
                      (banded_matrix(rng, 10000, 12), [[16, 32], [8, 16]]),    # two partitions (second one adds)
                      (mixed_band_matrix(rng, 24000), [[8, 16, 32, 64]])):     # several buckets of one partition
        _, info = check(fa, torch, g, widths, feat, b_dtype, seed=feat)
        assert info["row_group_buckets"] >= (4 if len(widths[0]) == 4 else 1), (widths, info)
        monkeypatch.setenv("LF_ROW_GROUPS", "0")
        _, info_off = check(fa, torch, g, widths, feat, b_dtype, seed=feat)
        monkeypatch.delenv("LF_ROW_GROUPS")
        assert info_off["row_group_buckets"] == 0
    g = skewed_matrix(rng, 20000, 30000, mean_deg=20, heavy_rows=0)
    _, info = check(fa, torch, g, [[8, 16, 32, 64]], feat, b_dtype, seed=feat)
    assert info["row_group_buckets"] == 0
