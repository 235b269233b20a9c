"""lf_row_features_static - the entry point that allocates nothing - against lf_row_features
through the raw C ABI: same four integers, on two calls in a row (the second on a smaller
matrix, so stale accumulators would show), then on an empty matrix and a refused size."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _features_both_ways(lib, torch, indptr_host):
    from liteform_ae_amd import _lib
    stream = torch.cuda.current_stream().cuda_stream
    num_rows = len(indptr_host) - 1
    d_indptr = torch.from_numpy(np.ascontiguousarray(indptr_host, dtype=np.int32)).cuda()
    # existing entry point: caller-supplied scratch, host output
    want = np.zeros(4, dtype=np.int64)
    scratch = torch.empty(4, dtype=torch.int64, device="cuda")
    _lib.check(lib.lf_row_features(d_indptr.data_ptr(), num_rows, scratch.data_ptr(),
                                   want.ctypes.data, stream))
    # the variant: output in device memory, stream ordered
    d_out = torch.full((4,), -7, dtype=torch.int64, device="cuda")
    _lib.check(lib.lf_row_features_static(d_indptr.data_ptr(), num_rows, d_out.data_ptr(), stream))
    torch.cuda.current_stream().synchronize()
    return d_out.cpu().numpy(), want


def test_static_scratch_matches_workspace_variant():
    import torch
    from liteform_ae_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(11)
    big = np.zeros(300_001, dtype=np.int64)
    big[1:] = np.cumsum(rng.integers(0, 700, size=300_000))
    small = np.zeros(1_001, dtype=np.int64)
    small[1:] = np.cumsum(rng.integers(3, 9, size=1_000))
    for indptr in (big, small):                      # the second call sees the first call's leftovers
        got, want = _features_both_ways(lib, torch, indptr)
        deg = np.diff(indptr)
        np.testing.assert_array_equal(want, [deg.min(), deg.max(), deg.sum(), (deg * deg).sum()])
        np.testing.assert_array_equal(got, want)
    got, want = _features_both_ways(lib, torch, np.zeros(1, dtype=np.int64))      # no rows
    np.testing.assert_array_equal(got, [0, 0, 0, 0])
    np.testing.assert_array_equal(got, want)


def test_static_scratch_rejects_oversize_and_null():
    import torch
    from liteform_ae_amd import _lib
    lib = _lib.load()
    d_out = torch.zeros(4, dtype=torch.int64, device="cuda")
    d_indptr = torch.zeros(2, dtype=torch.int32, device="cuda")
    rc = lib.lf_row_features_static(d_indptr.data_ptr(), 2**31 - 1, d_out.data_ptr(), None)
    assert rc == _lib.LF_ERR_UNSUPPORTED and "at most" in _lib.last_error()
    rc = lib.lf_row_features_static(d_indptr.data_ptr(), 1, None, None)
    assert rc == _lib.LF_ERR_INVALID


def test_static_scratch_inside_a_hip_graph():
    """The use the entry point is there for: recorded into a HIP graph (after one eager call on
    the device, which looks up the array's address) and replayed on changing data, with eager
    work and synchronisations between the replays; every replay against lf_row_features."""
    import torch
    from liteform_ae_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(12)
    num_rows = 50_000
    d_indptr = torch.zeros(num_rows + 1, dtype=torch.int32, device="cuda")
    d_out = torch.zeros(4, dtype=torch.int64, device="cuda")
    _lib.check(lib.lf_row_features_static(d_indptr.data_ptr(), num_rows, d_out.data_ptr(),
                                          torch.cuda.current_stream().cuda_stream))         # eager warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check(lib.lf_row_features_static(d_indptr.data_ptr(), num_rows, d_out.data_ptr(),
                                              torch.cuda.current_stream().cuda_stream))
    scratch = torch.empty(4, dtype=torch.int64, device="cuda")
    for hi in (900, 7, 60):
        deg = rng.integers(0, hi, size=num_rows)
        indptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int32)
        d_indptr.copy_(torch.from_numpy(indptr).cuda())
        d_out.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = np.zeros(4, dtype=np.int64)
        _lib.check(lib.lf_row_features(d_indptr.data_ptr(), num_rows, scratch.data_ptr(), want.ctypes.data,
                                       torch.cuda.current_stream().cuda_stream))
        np.testing.assert_array_equal(d_out.cpu().numpy(), want)
        np.testing.assert_array_equal(want, [deg.min(), deg.max(), deg.sum(), (deg.astype(np.int64) ** 2).sum()])
