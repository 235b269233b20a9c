"""MTX(path): the MatrixMarket ingest of the reference's container
(playground_pipline/format_matrix_market.py:58-65): the file is read with scipy.io.mmread,
every stored value is replaced by 1, the name is the file's stem.  The CPU part checks the
container; the GPU part takes the same files through the device ingest, the search, the
builder and the product."""
import numpy as np
import pytest
import scipy.sparse as sp

from liteform_ae_amd.format_matrix_market import MTX
from oracle import liteform_oracle as O

# 5 x 6, coordinate entries unsorted; (2,3) and (4,1) appear twice (MatrixMarket allows repeated
# coordinates in a general matrix; scipy keeps them as separate COO triplets)
REAL_GENERAL = """%%MatrixMarket matrix coordinate real general
% unsorted, with repeated coordinates
5 6 9
4 1 2.5
1 1 -1.0
2 3 0.25
5 6 7.0
2 3 4.0
3 2 1e-3
1 5 3.0
4 1 -2.5
2 1 9.0
"""

PATTERN_GENERAL = """%%MatrixMarket matrix coordinate pattern general
4 7 6
3 7
1 2
1 1
4 4
2 6
3 1
"""

INTEGER_SYMMETRIC = """%%MatrixMarket matrix coordinate integer symmetric
4 4 4
1 1 5
3 1 2
4 2 -3
4 4 8
"""

FILES = {"real_general": REAL_GENERAL, "pattern_general": PATTERN_GENERAL, "integer_symmetric": INTEGER_SYMMETRIC}
# stored triplets after reading (row, col), 0-based, in file order; symmetric files are expanded by mmread
TRIPLETS = {
    "real_general": ((5, 6), [(3, 0), (0, 0), (1, 2), (4, 5), (1, 2), (2, 1), (0, 4), (3, 0), (1, 0)]),
    "pattern_general": ((4, 7), [(2, 6), (0, 1), (0, 0), (3, 3), (1, 5), (2, 0)]),
    "integer_symmetric": ((4, 4), [(0, 0), (2, 0), (3, 1), (3, 3), (0, 2), (1, 3)]),
}


@pytest.fixture(params=sorted(FILES))
def mtx_file(request, tmp_path):
    path = tmp_path / f"{request.param}.mtx"
    path.write_text(FILES[request.param])
    return request.param, str(path)


def test_mtx_path_reads_pattern_and_forces_ones(mtx_file):
    name, path = mtx_file
    g = MTX(path)
    shape, trip = TRIPLETS[name]
    assert g.name == name
    assert g.coo_mtx.shape == shape
    assert g.num_src_nodes() == shape[0] and g.num_dst_nodes() == shape[1]
    assert g.num_edges() == len(trip)
    assert sorted(zip(g.coo_mtx.row.tolist(), g.coo_mtx.col.tolist())) == sorted(trip)
    assert (g.coo_mtx.data == 1).all() and g.coo_mtx.data.dtype == np.float64     # format_matrix_market.py:63-64
    indptr, indices, data = g.adj_tensors("csr")
    want = sp.coo_matrix((np.ones(len(trip)), tuple(zip(*trip))), shape=shape).tocsr()
    np.testing.assert_array_equal(indptr, want.indptr)
    np.testing.assert_array_equal(indices, want.indices)
    np.testing.assert_array_equal(data, want.data)        # repeated coordinates add up to 2
    # the container's product is the scipy one
    B = np.arange(shape[1] * 3, dtype=np.float64).reshape(shape[1], 3)
    np.testing.assert_array_equal(g.dot(B), want @ B)


@pytest.mark.gpu
def test_mtx_path_through_the_gpu_pipeline(mtx_file):
    import torch
    from liteform_ae_amd import format_algos as fa
    name, path = mtx_file
    g = MTX(path)
    shape, trip = TRIPLETS[name]
    dev = fa._DeviceCSR(g)
    want = g.coo_mtx.tocsr()
    want.sum_duplicates()
    assert dev.coo_nnz == len(trip) and dev.nnz == want.nnz
    np.testing.assert_array_equal(dev.indptr.cpu().numpy(), want.indptr)
    np.testing.assert_array_equal(dev.indices.cpu().numpy(), want.indices)
    np.testing.assert_array_equal(dev.values.cpu().numpy(), want.data.astype(np.float32))
    assert dev.all_ones == (want.nnz == len(trip))
    # search and builder against the oracle (degrees come from the raw triplets, fills from the CSR)
    cfg = fa.search_bucket_config(g, 1, fa.CostModelSettings(32, 1))
    assert cfg == O.search_bucket_config(g, 1, O.OracleCostModelSettings(32, 1))
    got = fa.build_hyb_format(g, cfg)
    ref = O.build_hyb_format_closed_form(g, cfg)
    for a_parts, b_parts in zip(got, ref):
        for ab, bb in zip(a_parts, b_parts):
            for x, y in zip(ab, bb):
                assert x.shape == y.shape and np.array_equal(x, y)
    # product with the summed values against the container's own scipy product
    B = np.arange(shape[1] * 32, dtype=np.float32).reshape(shape[1], 32) % 7
    out = fa.spmm_hyb(fa.build_hyb_format_device(g, cfg), torch.from_numpy(B).cuda()).cpu().numpy()
    np.testing.assert_array_equal(out, g.dot(B.astype(np.float64)).astype(np.float32))
