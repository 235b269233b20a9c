"""The C ABI driven directly through ctypes, the way a non-Python host would: explicit
workspaces, plan -> layout -> build, plan handle life cycle, and the error paths."""
import ctypes as C

import numpy as np
import pytest

from oracle import liteform_oracle as O

from helpers import assert_hyb_equal, skewed_matrix

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    from liteform_ae_amd import _lib
    return _lib.load(), _lib, torch


def dev(torch, a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=dtype)).cuda()


def test_raw_abi_end_to_end(env):
    lib, L, torch = env
    rng = np.random.default_rng(5)
    g = skewed_matrix(rng, 1500, 1200, mean_deg=7, heavy_rows=2, heavy_len=3000)
    rows, cols = g.coo_mtx.shape
    indptr, indices, data = g.adj_tensors("csr")
    d_ptr, d_idx, d_val = dev(torch, indptr, np.int32), dev(torch, indices, np.int32), dev(torch, data, np.float32)
    P, feat = 2, 64

    # statistics + search
    nbytes = lib.lf_stats_workspace_bytes(rows, cols, P)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    stats = np.zeros((P, 11, 4), np.int64)
    hist = np.zeros((P, 2048), np.int64)
    assert lib.lf_bucket_stats(d_ptr.data_ptr(), d_idx.data_ptr(), None, rows, cols, P, 1024, ws.data_ptr(), nbytes,
                               L.np_ptr(stats, C.c_int64), L.np_ptr(hist, C.c_int64), None) == 0
    widths = np.zeros((P, 11), np.int32)
    nw = np.zeros(P, np.int32)
    assert lib.lf_search_bucket_config(L.np_ptr(stats, C.c_int64), L.np_ptr(hist, C.c_int64), P, 1024, feat, P, 0,
                                       L.np_ptr(widths, C.c_int32), L.np_ptr(nw, C.c_int32), None, None) == 0
    cfg = [widths[p, :nw[p]].tolist() for p in range(P)]
    assert cfg == O.search_bucket_config(g, P, O.OracleCostModelSettings(feat, P))

    # plan -> layout -> build
    flat = np.concatenate([widths[p, :nw[p]] for p in range(P)]).astype(np.int32)
    off = np.concatenate(([0], np.cumsum(nw))).astype(np.int32)
    nb = int(off[-1])
    hb = lib.lf_hyb_workspace_bytes(rows, P, nb)
    hws = torch.empty(hb, dtype=torch.uint8, device="cuda")
    ell = np.zeros(nb, np.int64)
    # the statistics pass left the per-partition row bounds in its workspace; the plan takes them
    bounds = lib.lf_stats_seg_bounds(ws.data_ptr(), rows, P)
    assert (bounds is not None) == (P > 1)
    ell_own = np.zeros(nb, np.int64)
    args = (rows, cols, P, L.np_ptr(flat, C.c_int32), L.np_ptr(off, C.c_int32))
    assert lib.lf_hyb_plan(d_ptr.data_ptr(), d_idx.data_ptr(), None, None, *args, hws.data_ptr(), hb,
                           L.np_ptr(ell_own, C.c_int64), None) == 0
    assert lib.lf_hyb_plan(d_ptr.data_ptr(), d_idx.data_ptr(), None, bounds, *args, hws.data_ptr(), hb,
                           L.np_ptr(ell, C.c_int64), None) == 0
    np.testing.assert_array_equal(ell, ell_own)     # same counts with its own pass over the indices
    ro, so = np.zeros(nb, np.int64), np.zeros(nb, np.int64)
    tr, ts = C.c_int64(), C.c_int64()
    assert lib.lf_hyb_layout(L.np_ptr(ell, C.c_int64), L.np_ptr(flat, C.c_int32), nb, L.np_ptr(ro, C.c_int64),
                             L.np_ptr(so, C.c_int64), C.byref(tr), C.byref(ts)) == 0
    d_rows = torch.empty(tr.value, dtype=torch.int32, device="cuda")
    d_meta = torch.empty(tr.value, dtype=torch.int32, device="cuda")
    d_cols = torch.empty(ts.value, dtype=torch.int32, device="cuda")
    d_vals = torch.empty(ts.value, dtype=torch.float32, device="cuda")
    d_mask = torch.empty(ts.value, dtype=torch.float32, device="cuda")
    assert lib.lf_hyb_build(d_ptr.data_ptr(), d_idx.data_ptr(), d_val.data_ptr(), None, rows, cols, P,
                            L.np_ptr(flat, C.c_int32), L.np_ptr(off, C.c_int32), L.np_ptr(ell, C.c_int64),
                            hws.data_ptr(), hb, d_rows.data_ptr(), d_meta.data_ptr(), d_cols.data_ptr(),
                            d_vals.data_ptr(), d_mask.data_ptr(), None) == 0
    torch.cuda.synchronize()
    want = O.build_hyb_format_closed_form(g, cfg, with_values=True)
    got = ([], [], [])
    k = 0
    for p in range(P):
        gp = ([], [], [])
        for b, w in enumerate(cfg[p]):
            R = int(ell[k])
            gp[0].append(d_rows[ro[k]:ro[k] + R].cpu().numpy().astype(np.int64))
            gp[1].append(d_cols[so[k]:so[k] + R * w].cpu().numpy().astype(np.int64).reshape(R, w))
            gp[2].append(d_mask[so[k]:so[k] + R * w].cpu().numpy().astype(np.int64).reshape(R, w))
            np.testing.assert_array_equal(d_vals[so[k]:so[k] + R * w].cpu().numpy().reshape(R, w),
                                          want[3][p][b].astype(np.float32))
            k += 1
        for i in range(3):
            got[i].append(gp[i])
    assert_hyb_equal(got, want[:3])

    # SpMM plan: create / info / run / time / destroy
    descs = (L.BucketDesc * nb)()
    k = 0
    for p in range(P):
        for w in cfg[p]:
            R = int(ell[k])
            descs[k] = L.BucketDesc(w, p, R, d_rows[ro[k]:].data_ptr(), d_cols[so[k]:].data_ptr(),
                                    d_vals[so[k]:].data_ptr(), d_meta[ro[k]:].data_ptr())
            k += 1
    plan = C.c_void_p()
    assert lib.lf_spmm_create(C.byref(plan), descs, nb, P, rows, cols, feat, 0, None) == 0
    info = np.zeros(8, np.int64)
    assert lib.lf_spmm_info(plan, L.np_ptr(info, C.c_int64)) == 0 and info[2] == P and info[0] > 0
    B = rng.uniform(-1, 1, size=(cols, feat)).astype(np.float32)
    dB = dev(torch, B, np.float32)
    dC = torch.empty((rows, feat), dtype=torch.float32, device="cuda")
    assert lib.lf_spmm_run(plan, dB.data_ptr(), dC.data_ptr(), None) == 0
    torch.cuda.synchronize()
    ref = O.spmm_csr_f64(indptr, indices, data, (rows, cols), B)
    bound = O.spmm_abs_bound(indptr, indices, data, (rows, cols), B)
    assert (np.abs(dC.cpu().numpy() - ref) <= 1e-5 * bound).all()
    ms = np.zeros(4, np.float32)
    assert lib.lf_spmm_time_ms(plan, dB.data_ptr(), dC.data_ptr(), 1, 4, None, 0, L.np_ptr(ms, C.c_float), None) == 0
    assert (ms > 0).all()
    # a second stream is honoured
    s2 = torch.cuda.Stream()
    dC2 = torch.empty_like(dC)
    assert lib.lf_spmm_run(plan, dB.data_ptr(), dC2.data_ptr(), s2.cuda_stream) == 0
    s2.synchronize()
    assert torch.equal(dC, dC2)
    assert lib.lf_spmm_destroy(plan) == 0
    assert lib.lf_spmm_destroy(None) == 0


def test_error_paths_report_and_do_not_crash(env):
    lib, L, torch = env
    rows, cols = 100, 100
    indptr = dev(torch, np.arange(rows + 1), np.int32)
    indices = dev(torch, np.arange(rows), np.int32)
    stats = np.zeros((1, 11, 4), np.int64)
    hist = np.zeros((1, 2048), np.int64)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    sp, hp = L.np_ptr(stats, C.c_int64), L.np_ptr(hist, C.c_int64)
    # workspace too small
    assert lib.lf_bucket_stats(indptr.data_ptr(), indices.data_ptr(), None, rows, cols, 1, 1024, ws.data_ptr(), 16,
                               sp, hp, None) == L.LF_ERR_WORKSPACE
    assert "workspace" in L.last_error()
    # width limit that is not a power of two, null row pointer, zero partitions
    assert lib.lf_bucket_stats(indptr.data_ptr(), indices.data_ptr(), None, rows, cols, 1, 1000, ws.data_ptr(),
                               1 << 20, sp, hp, None) == L.LF_ERR_INVALID
    assert lib.lf_bucket_stats(None, indices.data_ptr(), None, rows, cols, 1, 1024, ws.data_ptr(), 1 << 20,
                               sp, hp, None) == L.LF_ERR_INVALID
    assert lib.lf_bucket_stats(indptr.data_ptr(), indices.data_ptr(), None, rows, cols, 0, 1024, ws.data_ptr(),
                               1 << 20, sp, hp, None) == L.LF_ERR_INVALID
    # statistics without the column pass, then the reference model refuses the missing histogram
    assert lib.lf_bucket_stats(indptr.data_ptr(), indices.data_ptr(), None, rows, cols, 1, 1024, ws.data_ptr(),
                               1 << 20, sp, None, None) == 0
    assert stats[0, 0, 2] == rows and stats[0, 0, 1] == rows
    w = np.zeros((1, 11), np.int32)
    n = np.zeros(1, np.int32)
    assert lib.lf_search_bucket_config(sp, None, 1, 1024, 32, 1, 0, L.np_ptr(w, C.c_int32), L.np_ptr(n, C.c_int32),
                                       None, None) == L.LF_ERR_INVALID
    assert lib.lf_search_bucket_config(sp, None, 1, 1024, 32, 1, 1, L.np_ptr(w, C.c_int32), L.np_ptr(n, C.c_int32),
                                       None, None) == 0
    assert w[0, :n[0]].tolist() == [1]
    # widths: not a power of two / not ascending
    flat = np.array([3], np.int32)
    off = np.array([0, 1], np.int32)
    ell = np.zeros(1, np.int64)
    assert lib.lf_hyb_plan(indptr.data_ptr(), indices.data_ptr(), None, None, rows, cols, 1, L.np_ptr(flat, C.c_int32),
                           L.np_ptr(off, C.c_int32), ws.data_ptr(), 1 << 20, L.np_ptr(ell, C.c_int64),
                           None) == L.LF_ERR_INVALID
    flat = np.array([4, 2], np.int32)
    off = np.array([0, 2], np.int32)
    ell = np.zeros(2, np.int64)
    assert lib.lf_hyb_plan(indptr.data_ptr(), indices.data_ptr(), None, None, rows, cols, 1, L.np_ptr(flat, C.c_int32),
                           L.np_ptr(off, C.c_int32), ws.data_ptr(), 1 << 20, L.np_ptr(ell, C.c_int64),
                           None) == L.LF_ERR_INVALID
    # SpMM: unsupported feature size, bad dtype, null output handle
    plan = C.c_void_p()
    assert lib.lf_spmm_create(C.byref(plan), None, 0, 1, rows, cols, 48, 0, None) == L.LF_ERR_UNSUPPORTED
    assert lib.lf_spmm_create(C.byref(plan), None, 0, 1, rows, cols, 64, 7, None) == L.LF_ERR_INVALID
    assert lib.lf_spmm_create(None, None, 0, 1, rows, cols, 64, 0, None) == L.LF_ERR_INVALID
    assert not plan.value
    # an empty format is a valid plan: the product is all zeros
    assert lib.lf_spmm_create(C.byref(plan), None, 0, 1, rows, cols, 64, 0, None) == 0
    B = torch.ones((cols, 64), device="cuda")
    Cd = torch.full((rows, 64), 5.0, device="cuda")
    assert lib.lf_spmm_run(plan, B.data_ptr(), Cd.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert float(Cd.abs().max()) == 0.0
    assert lib.lf_spmm_run(plan, None, Cd.data_ptr(), None) == L.LF_ERR_INVALID
    assert lib.lf_spmm_run(plan, B.data_ptr() + 4, Cd.data_ptr(), None) == L.LF_ERR_INVALID      # misaligned
    assert lib.lf_spmm_destroy(plan) == 0


def test_gfx950_search_ignores_column_sets(env):
    lib, L, torch = env
    from liteform_ae_amd import format_algos as fa
    rng = np.random.default_rng(13)
    g = skewed_matrix(rng, 4000, 4000, mean_deg=10, heavy_rows=3, values=False)
    for parts in (1, 3):
        cfgm = fa.CostModelSettings(128, parts, cost_model="gfx950")
        s1, h1 = fa.bucket_statistics(g, parts, with_columns=True)
        s2, h2 = fa.bucket_statistics(g, parts, with_columns=False)
        np.testing.assert_array_equal(s1, s2)
        assert h2 is None
        assert fa.search_from_statistics(s1, h1, cfgm) == fa.search_from_statistics(s2, None, cfgm) \
            == fa.search_bucket_config(g, parts, cfgm)
