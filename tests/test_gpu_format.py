"""GPU parity of the format pass (statistics, search, hyb composition) with the oracle.

Everything goes through the C ABI (ctypes) behind the reference-shaped Python functions.
Format structures must match bit for bit."""
import numpy as np
import pytest

from oracle import liteform_oracle as O

from helpers import assert_hyb_equal, mtx_from_rows, skewed_matrix, stats_from_oracle

pytestmark = pytest.mark.gpu

HAND = [[0, 1, 2, 5], [1], [], [0, 1, 2, 3, 4, 6], [2, 7], [0, 3, 4, 5, 6]]


@pytest.fixture(scope="module")
def fa():
    from liteform_ae_amd import format_algos
    return format_algos


def test_hand_example_end_to_end(fa):
    g = mtx_from_rows(HAND, (6, 8))
    cfg = fa.search_bucket_config(g, 2, fa.CostModelSettings(32, 2))
    assert cfg == [[1, 4], [1, 2]]
    rows, cols, mask = fa.build_hyb_format(g, cfg)
    assert rows[0][1].tolist() == [0, 3, 5]
    assert cols[0][1].tolist() == [[0, 1, 2, 0], [0, 1, 2, 3], [0, 3, 0, 0]]
    assert mask[0][1].tolist() == [[1, 1, 1, 0], [1, 1, 1, 1], [1, 1, 0, 0]]
    assert rows[1][1].tolist() == [3, 5, 5]
    assert cols[1][1].tolist() == [[4, 6], [4, 5], [6, 0]]
    assert mask[1][1].tolist() == [[1, 1], [1, 1], [1, 0]]
    assert rows[0][0].dtype == np.int64 and cols[0][1].shape == (3, 4)
    assert_hyb_equal((rows, cols, mask), O.build_hyb_format_sequential(g, cfg))


@pytest.mark.parametrize("seed", range(8))
def test_bucket_stats_match_oracle(fa, seed):
    rng = np.random.default_rng(40 + seed)
    nr, nc = int(rng.integers(100, 3000)), int(rng.integers(100, 3000))
    parts = int(rng.choice([1, 2, 3, 7, 16]))
    g = skewed_matrix(rng, nr, nc, mean_deg=float(rng.choice([3, 8, 20])), heavy_rows=3, values=False)
    stats, hist = fa.bucket_statistics(g, parts)
    wstats, whist = stats_from_oracle(g, parts)
    np.testing.assert_array_equal(stats, wstats)
    np.testing.assert_array_equal(hist, whist)


@pytest.mark.parametrize("seed", range(8))
def test_search_matches_oracle(fa, seed):
    rng = np.random.default_rng(60 + seed)
    nr, nc = int(rng.integers(200, 2500)), int(rng.integers(200, 2500))
    parts = int(rng.choice([1, 2, 4, 8]))
    feat = int(rng.choice([32, 128, 512]))
    g = skewed_matrix(rng, nr, nc, mean_deg=8, heavy_rows=2, values=False)
    try:
        want = O.search_bucket_config(g, parts, O.OracleCostModelSettings(feat, parts))
    except ValueError:
        with pytest.raises(ValueError):
            fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts))
        return
    assert fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts)) == want


def test_single_nonzero_partition_raises_value_error(fa):
    g = mtx_from_rows([[3]], (1, 8))
    with pytest.raises(ValueError, match="only having 1 non-zero element"):
        fa.search_bucket_config(g, 1, fa.CostModelSettings(32, 1))


@pytest.mark.parametrize("seed", range(10))
def test_builder_matches_sequential_oracle(fa, seed):
    rng = np.random.default_rng(80 + seed)
    nr, nc = int(rng.integers(30, 700)), int(rng.integers(30, 700))
    parts = int(rng.choice([1, 2, 3, 5]))
    g = skewed_matrix(rng, nr, nc, mean_deg=6, heavy_rows=2, values=False)
    all_w = [1 << i for i in range(8)]
    widths = [sorted(rng.choice(all_w, size=int(rng.integers(1, 6)), replace=False).tolist())
              for _ in range(parts)]
    got = fa.build_hyb_format(g, widths)
    assert_hyb_equal(got, O.build_hyb_format_sequential(g, widths))


def test_builder_with_searched_config_mid_size(fa):
    rng = np.random.default_rng(7)
    g = skewed_matrix(rng, 20000, 20000, mean_deg=12, heavy_rows=5, heavy_len=6000, values=False)
    for parts in (1, 4):
        cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(128, parts))
        assert cfg == O.search_bucket_config(g, parts, O.OracleCostModelSettings(128, parts))
        assert_hyb_equal(fa.build_hyb_format(g, cfg), O.build_hyb_format_closed_form(g, cfg))


def test_builder_edge_cases(fa):
    # empty matrix rows, an empty partition, a single bucket of width 1 holding a long row
    g = mtx_from_rows([[], [0, 1, 2, 3, 4], [], [1]], (4, 16))
    for widths in ([[1], []], [[8], []], [[1, 2, 4, 8], []]):
        assert_hyb_equal(fa.build_hyb_format(g, widths), O.build_hyb_format_sequential(g, widths))
    with pytest.raises(IndexError):
        fa.build_hyb_format(g, [[], [4]])                 # nonzeros in a partition without widths
    with pytest.raises(AssertionError):
        fa.build_hyb_format(g, [[3], []])                 # not a power of two
    # empty buckets are kept with shapes (0,), (0, W)   (format_algos.py:365-368)
    rows, cols, mask = fa.build_hyb_format(g, [[1, 2, 4, 8], []])
    assert rows[0][1].shape == (0,) and cols[0][1].shape == (0, 2) and mask[0][2].shape == (0, 4)


def test_duplicate_coo_entries(fa):
    """COO duplicates raise the degree but not the fill (format_algos.py:250-254)."""
    from liteform_ae_amd.format_matrix_market import MTX
    rng = np.random.default_rng(11)
    r = rng.integers(0, 50, size=600)
    c = rng.integers(0, 64, size=600)
    g = MTX.from_coo(r, c, (50, 64))
    assert g.num_edges() != g.adj_tensors("csr")[1].shape[0]      # there are duplicates
    for parts in (1, 2):
        widths = [[2, 8, 16]] * parts
        assert_hyb_equal(fa.build_hyb_format(g, widths), O.build_hyb_format_sequential(g, widths))
        stats, hist = fa.bucket_statistics(g, parts)
        wstats, whist = stats_from_oracle(g, parts)
        np.testing.assert_array_equal(stats, wstats)
        np.testing.assert_array_equal(hist, whist)


def test_workload_shapes_scaled(fa):
    from liteform_ae_amd.synthetic import make_workload
    for name, scale, parts in (("cfg1", 1.0, 1), ("cfg2", 0.05, 2), ("cfg3", 0.005, 1), ("cfg3", 0.005, 4),
                               ("cfg4", 0.004, 1), ("cfg5", 0.01, 2)):
        wl = make_workload(name, scale)
        g = wl.matrix
        cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(wl.feat_size, parts))
        assert cfg == O.search_bucket_config(g, parts, O.OracleCostModelSettings(wl.feat_size, parts)), name
        assert_hyb_equal(fa.build_hyb_format(g, cfg), O.build_hyb_format_closed_form(g, cfg))


def test_device_ingest_matches_scipy_tocsr(fa):
    """lf_coo_to_csr against coo.tocsr() (format_matrix_market.py:74-76): unsorted triplets,
    duplicates, empty rows, rectangular shapes."""
    import scipy.sparse as sp
    from liteform_ae_amd.format_matrix_market import MTX
    rng = np.random.default_rng(17)
    for (nr, nc, n, weighted) in ((1, 1, 1, False), (300, 500, 4000, False), (2000, 70, 30000, True),
                                  (5, 100000, 2000, True), (100000, 3, 50000, False)):
        r = rng.integers(0, nr, size=n)
        c = rng.integers(0, nc, size=n)
        d = rng.uniform(-1, 1, size=n) if weighted else None
        g = MTX.from_coo(r, c, (nr, nc), data=d)
        dev = fa._DeviceCSR(g)
        want = g.coo_mtx.tocsr()
        want.sum_duplicates()
        assert dev.nnz == want.nnz and dev.coo_nnz == n
        np.testing.assert_array_equal(dev.indptr.cpu().numpy(), want.indptr)
        np.testing.assert_array_equal(dev.indices.cpu().numpy(), want.indices)
        np.testing.assert_allclose(dev.values.cpu().numpy(), want.data, rtol=1e-5, atol=1e-6)
        assert dev.all_ones == (not weighted and want.nnz == n)
    g = MTX.from_coo(np.zeros(0, np.int64), np.zeros(0, np.int64), (7, 9))
    dev = fa._DeviceCSR(g)
    assert dev.nnz == 0 and dev.indptr.cpu().numpy().tolist() == [0] * 8


def test_canonical_csr_input_goes_in_as_it_is(fa):
    """A container made from canonical CSR arrays is uploaded and checked (lf_csr_check), not
    converted to COO and sorted: same device arrays, statistics and slabs as the COO route."""
    import scipy.sparse as sp
    from liteform_ae_amd.format_matrix_market import MTX
    rng = np.random.default_rng(19)
    for (nr, nc, deg, weighted) in ((1, 1, 1, False), (700, 900, 9, True), (3000, 40, 5, False), (40, 30000, 200, True)):
        src = skewed_matrix(rng, nr, nc, mean_deg=deg, heavy_rows=1, values=weighted)
        indptr, indices, data = src.adj_tensors("csr")
        g = MTX.from_csr(indptr, indices, (nr, nc), data=data if weighted else None)
        assert g._coo is None                                   # no COO view was built
        dev = fa._DeviceCSR(g)
        assert dev.path == "csr" and g._coo is None
        ref = fa._DeviceCSR(MTX.from_coo(src.coo_mtx.row, src.coo_mtx.col, (nr, nc), data=data if weighted else None))
        assert ref.path == "coo"
        assert dev.nnz == ref.nnz == dev.coo_nnz and dev.all_ones == ref.all_ones == (not weighted)
        np.testing.assert_array_equal(dev.indptr.cpu().numpy(), ref.indptr.cpu().numpy())
        np.testing.assert_array_equal(dev.indices.cpu().numpy(), ref.indices.cpu().numpy())
        np.testing.assert_array_equal(dev.values.cpu().numpy(), ref.values.cpu().numpy())
        if nr > 1:
            widths = [[1, 4, 16]] * 2
            assert_hyb_equal(fa.build_hyb_format(g, widths), O.build_hyb_format_sequential(src, widths))
            np.testing.assert_array_equal(fa.bucket_statistics(g, 2)[0], stats_from_oracle(src, 2)[0])
    # float32 ones given as data are recognised on the GPU
    g = MTX.from_csr(indptr, indices, (nr, nc), data=np.ones(len(indices), dtype=np.float32))
    assert fa._DeviceCSR(g).all_ones
    # an empty matrix
    dev = fa._DeviceCSR(MTX.from_csr(np.zeros(8, np.int32), np.zeros(0, np.int32), (7, 9)))
    assert dev.path == "csr" and dev.nnz == 0


def test_csr_input_that_is_not_canonical_takes_the_sort(fa):
    """Unsorted columns or duplicates inside a row: the check says so and the arrays go the
    COO route, ending as scipy's tocsr() has them (format_matrix_market.py:74-76).  Arrays that
    are no CSR structure at all are refused."""
    import scipy.sparse as sp
    from liteform_ae_amd.format_matrix_market import MTX
    rng = np.random.default_rng(23)
    nr, nc = 400, 300
    deg = rng.integers(0, 12, size=nr)
    indptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int32)
    for kind in ("unsorted", "duplicates"):
        if kind == "unsorted":
            indices = np.concatenate([rng.permutation(nc)[:d] for d in deg]).astype(np.int32)
        else:
            indices = np.concatenate([np.sort(rng.integers(0, 6, size=d)) for d in deg]).astype(np.int32)
        data = rng.uniform(-1, 1, size=len(indices)).astype(np.float32)
        g = MTX.from_csr(indptr, indices, (nr, nc), data=data)
        dev = fa._DeviceCSR(g)
        assert dev.path == "coo"
        want = sp.csr_matrix((data, indices, indptr), shape=(nr, nc)).tocoo().tocsr()
        want.sum_duplicates()
        assert dev.nnz == want.nnz and dev.coo_nnz == len(indices)
        np.testing.assert_array_equal(dev.indptr.cpu().numpy(), want.indptr)
        np.testing.assert_array_equal(dev.indices.cpu().numpy(), want.indices)
        np.testing.assert_allclose(dev.values.cpu().numpy(), want.data, rtol=1e-5, atol=1e-6)
        widths = [[2, 8]]
        assert_hyb_equal(fa.build_hyb_format(g, widths), O.build_hyb_format_sequential(g, widths))
    bad = np.sort(rng.integers(0, nc, size=int(indptr[-1]))).astype(np.int32)
    bad[5] = nc                                                    # a column outside the matrix
    m = MTX(None)
    m._csr_source = sp.csr_matrix((nr, nc), dtype=np.float32)      # placeholder, arrays replaced below
    m._csr_source.indptr, m._csr_source.indices = indptr, bad
    m._csr_source.data = np.ones(len(bad), dtype=np.float32)
    with pytest.raises(ValueError, match="outside"):
        fa._DeviceCSR(m)
