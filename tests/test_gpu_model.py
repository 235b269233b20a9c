"""The launch-shape model and the fold model against the GPU: the matrix features they read
(lf_row_overlap) against numpy and the decisions on small and structured matrices.  (Timing
comparisons of the models' choices live in test_zy_timing.py.)"""
import numpy as np
import pytest

from liteform_ae_amd.format_matrix_market import MTX

from helpers import skewed_matrix

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa():
    from liteform_ae_amd import format_algos
    return format_algos


def overlap_numpy(g, stride):
    indptr, indices, _ = g.adj_tensors("csr")
    both = seen = 0
    for r in range(1, g.num_src_nodes(), stride):
        a = indices[indptr[r - 1]:indptr[r]][:64]         # the first 64 entries of either row
        b = indices[indptr[r]:indptr[r + 1]][:64]
        both += len(np.intersect1d(a, b))
        seen += len(b)
    return both, seen


def test_row_overlap_matches_numpy(fa):
    import ctypes as C
    import torch
    from liteform_ae_amd import _lib
    from liteform_ae_amd.synthetic import make_workload
    lib = _lib.load()
    rng = np.random.default_rng(61)
    for g, stride in ((make_workload("cfg4", 0.01).matrix, 1), (make_workload("cfg4", 0.01).matrix, 7),
                      (skewed_matrix(rng, 3000, 500, mean_deg=12, heavy_rows=2), 1),
                      (skewed_matrix(rng, 2000, 4000, mean_deg=40, heavy_rows=6, heavy_len=3000), 1),
                      (MTX.from_coo(np.array([0]), np.array([0]), (1, 4)), 1)):
        dev = fa._device_csr(g)
        out = np.zeros(2, dtype=np.int64)
        scratch = torch.empty(2, dtype=torch.int64, device="cuda")
        _lib.check(lib.lf_row_overlap(dev.indptr.data_ptr(), dev.indices.data_ptr(), dev.num_rows, stride,
                                      scratch.data_ptr(), _lib.np_ptr(out, C.c_int64), None))
        assert tuple(out) == overlap_numpy(g, stride)
    assert fa.row_overlap_device(MTX.from_coo(np.array([], dtype=np.int32), np.array([], dtype=np.int32), (10, 10))) == 0.0
    assert fa.predict_launch_shape(MTX.from_coo(np.array([], dtype=np.int32), np.array([], dtype=np.int32), (10, 10)), 64) == (1, 1)
    assert fa.predict_launch_shape(MTX.from_coo(np.array([0]), np.array([0]), (1, 5)), 128)[0] == 1
    assert fa.row_overlap_device(make_workload("cfg4", 0.05).matrix) > 0.6      # 18 of 27 columns, less at the faces
    assert fa.row_overlap_device(skewed_matrix(rng, 20000, 200000, mean_deg=10)) < 0.01


def test_structured_and_small_matrices_get_one_launch(fa):
    from liteform_ae_amd.synthetic import make_workload
    best, table = fa.predict_launch_shape(make_workload("cfg4", 0.05).matrix, 256, return_predictions=True)
    assert best == (1, 1) and table == {}                 # decided by the overlap of neighbouring rows
    rng = np.random.default_rng(62)
    g = skewed_matrix(rng, 30000, 30000, mean_deg=8, heavy_rows=2)
    best, table = fa.predict_launch_shape(g, 128, return_predictions=True)
    many = g.num_edges() > fa.DENSE_USES_PER_B_ROW * g.num_dst_nodes()      # then up to 32 partitions are priced
    assert best == (1, 1) and set(table) == {(p, w) for p in fa.PARTITION_CANDIDATES if p <= 4 or many for w in (1, 2)}
    sparse = skewed_matrix(rng, 30000, 30000, mean_deg=2, heavy_rows=0)
    assert set(fa.predict_launch_shape(sparse, 128, return_predictions=True)[1]) == {(p, w) for p in (1, 2, 3, 4) for w in (1, 2)}
    assert fa.guess_num_partitions(g, 128) == 1
