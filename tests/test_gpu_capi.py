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
    info = np.zeros(L.LF_SPMM_INFO_FIELDS, np.int64)
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


def _tuple_descs(L, torch, rows_nd, cols_nd, vals_nd, widths, metas=None):
    """lf_bucket_desc array for reference-style slabs (one partition), with the tensors that
    keep them alive."""
    keep = []
    descs = (L.BucketDesc * len(widths))()
    for b, w in enumerate(widths):
        r = dev(torch, rows_nd[b], np.int32)
        c = dev(torch, np.asarray(cols_nd[b]).reshape(-1), np.int32)
        v = dev(torch, np.asarray(vals_nd[b]).reshape(-1), np.float32)
        m = dev(torch, metas[b], np.int32) if metas is not None else None
        keep += [r, c, v, m]
        descs[b] = L.BucketDesc(int(w), 0, int(r.numel()), r.data_ptr(), c.data_ptr(), v.data_ptr(),
                                m.data_ptr() if m is not None else None)
    return descs, keep


def test_bad_slabs_are_refused_at_plan_creation(env):
    """Caller-supplied slabs (the reference hands rows, cols and values to its kernel unchecked,
    format_algos.py:552-578) are validated before any kernel gathers or stores through them:
    only the status code is read, no product runs on the bad data."""
    lib, L, torch = env
    rng = np.random.default_rng(77)
    g = skewed_matrix(rng, 600, 500, mean_deg=5, heavy_rows=1, heavy_len=300, values=False)
    rows, cols = g.coo_mtx.shape
    cfg = [[1, 2, 4, 8]]
    rows_nd, cols_nd, mask_nd = O.build_hyb_format_closed_form(g, cfg)
    rows_nd, cols_nd, mask_nd = rows_nd[0], cols_nd[0], mask_nd[0]

    def create(r, c, v, metas=None):
        descs, keep = _tuple_descs(L, torch, r, c, v, cfg[0], metas)
        plan = C.c_void_p()
        rc = lib.lf_spmm_create(C.byref(plan), descs, len(cfg[0]), 1, rows, cols, 64, 0, None)
        msg = L.last_error()
        if rc == 0:
            assert lib.lf_spmm_destroy(plan) == 0
        else:
            assert not plan.value
        return rc, msg

    assert create(rows_nd, cols_nd, mask_nd)[0] == 0                       # the good slabs pass
    for bad_col in (cols, -1, 2**31 - 1):
        c = [a.copy() for a in cols_nd]
        c[2][len(c[2]) // 2, 1] = bad_col
        rc, msg = create(rows_nd, c, mask_nd)
        assert rc == L.LF_ERR_INVALID and "column index" in msg
    for bad_row in (rows, -5):
        r = [a.copy() for a in rows_nd]
        r[1][0] = bad_row
        rc, msg = create(r, cols_nd, mask_nd)
        assert rc == L.LF_ERR_INVALID and "row index" in msg
    # caller-supplied meta: a length above W, a segment that leaves the bucket, an orphan continuation row
    def good_meta():
        out = []
        for b, w in enumerate(cfg[0]):
            ln = np.maximum(1, (np.asarray(mask_nd[b]) != 0).sum(1)).astype(np.int64)
            r = np.asarray(rows_nd[b])
            m = np.zeros(len(r), dtype=np.int64)
            i = 0
            while i < len(r):
                j = i
                while j + 1 < len(r) and r[j + 1] == r[i]:
                    j += 1
                m[i] = ln[i] | ((j - i + 1) << 11)
                for t in range(i + 1, j + 1):
                    m[t] = ln[t] | ((t - i) << 11) | (1 << 31)
                i = j + 1
            out.append(m.astype(np.uint32).view(np.int32))
        return out
    assert create(rows_nd, cols_nd, mask_nd, good_meta())[0] == 0
    m = good_meta(); m[0][3] = 2 | (1 << 11)                               # 2 valid slots in a 1-wide row
    assert create(rows_nd, cols_nd, mask_nd, m)[0] == L.LF_ERR_INVALID
    m = good_meta(); m[3][-1] = int(m[3][-1] & 0x7FF) | (5 << 11)          # head announcing rows past the end
    rc, msg = create(rows_nd, cols_nd, mask_nd, m)
    assert rc == L.LF_ERR_INVALID and "meta" in msg
    m = good_meta(); m[1][0] = np.int32(-(2**31) + (1 << 11) + 1)          # continuation row with no head
    assert create(rows_nd, cols_nd, mask_nd, m)[0] == L.LF_ERR_INVALID


def test_a_head_announcing_a_huge_segment_is_refused(env):
    """A head word that announces 100,000 ELL rows in a 64-wide bucket of a few rows: the
    announced segment is long enough for the cooperative (chunked) path, whose counting pass
    is enqueued together with the slab checks; it must not read the meta word of the
    announced last ELL row, ~400 KB past the array.  Status only."""
    lib, L, torch = env
    rng = np.random.default_rng(79)
    g = skewed_matrix(rng, 300, 5000, mean_deg=4, heavy_rows=2, heavy_len=200, values=False)
    rows, cols = g.coo_mtx.shape
    cfg = [[64]]
    rows_nd, cols_nd, mask_nd = O.build_hyb_format_closed_form(g, cfg)
    r, c, v = rows_nd[0][0], cols_nd[0][0], mask_nd[0][0]
    ln = np.maximum(1, (np.asarray(v) != 0).sum(1)).astype(np.int64)
    meta = np.zeros(len(r), dtype=np.int64)
    i = 0
    while i < len(r):
        j = i
        while j + 1 < len(r) and r[j + 1] == r[i]:
            j += 1
        meta[i] = ln[i] | ((j - i + 1) << 11)
        for t in range(i + 1, j + 1):
            meta[t] = ln[t] | ((t - i) << 11) | (1 << 31)
        i = j + 1
    for at, announced in ((0, 100_000), (len(r) - 1, (1 << 20) - 1), (len(r) // 2, 70)):
        m = meta.copy()
        m[at] = int(m[at] & 0x7FF) | (announced << 11)
        descs, keep = _tuple_descs(L, torch, [r], [c], [v], cfg[0], [m.astype(np.uint32).view(np.int32)])
        plan = C.c_void_p()
        rc = lib.lf_spmm_create(C.byref(plan), descs, 1, 1, rows, cols, 64, 0, None)
        assert rc == L.LF_ERR_INVALID and "meta" in L.last_error() and not plan.value
    descs, keep = _tuple_descs(L, torch, [r], [c], [v], cfg[0], [meta.astype(np.uint32).view(np.int32)])
    plan = C.c_void_p()
    assert lib.lf_spmm_create(C.byref(plan), descs, 1, 1, rows, cols, 64, 0, None) == 0
    assert lib.lf_spmm_destroy(plan) == 0


def test_derived_meta_of_long_segments(env):
    """Slabs without meta whose widest bucket holds rows split over hundreds of ELL rows (runs
    of equal row ids crossing several 256-row blocks of the derivation pass)."""
    lib, L, torch = env
    from liteform_ae_amd import format_algos as fa
    rng = np.random.default_rng(78)
    g = skewed_matrix(rng, 900, 4000, mean_deg=3, heavy_rows=3, heavy_len=2500, values=False)
    rows, cols = g.coo_mtx.shape
    cfg = [[1, 2]]
    hyb = O.build_hyb_format_closed_form(g, cfg)
    assert max(np.bincount(hyb[0][0][1])) > 600                             # one row id on > 600 ELL rows
    B = rng.uniform(-1, 1, size=(cols, 32)).astype(np.float32)
    plan = fa.HybSpMM(hyb, 32, num_rows=rows, num_cols=cols, bucket_widths=cfg)
    out = plan.run(torch.from_numpy(B).cuda()).cpu().numpy()
    plan.close()
    indptr, indices, data = g.adj_tensors("csr")
    ref = O.spmm_csr_f64(indptr, indices, data, (rows, cols), B)
    bound = O.spmm_abs_bound(indptr, indices, data, (rows, cols), B)
    assert (np.abs(out - ref) <= 1e-5 * bound).all()


def test_csr_and_bsr_index_arrays_are_checked_before_any_gather(env):
    """lf_csr_spmm and lf_bsr_spmm take index arrays straight from the caller: an index outside
    the dense operand, or a row pointer that is not one, must come back as LF_ERR_INVALID with
    the output untouched - no product kernel may run on such arrays.  Status and output only."""
    lib, L, torch = env
    rng = np.random.default_rng(81)
    rows, cols, feat = 300, 200, 64
    deg = rng.integers(0, 9, size=rows)
    indptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int32)
    nnz = int(indptr[-1])
    indices = np.concatenate([np.sort(rng.choice(cols, size=d, replace=False)) for d in deg]).astype(np.int32)
    vals = rng.uniform(-1, 1, size=nnz).astype(np.float32)
    B = rng.uniform(-1, 1, size=(cols, feat)).astype(np.float32)
    dB, dV = dev(torch, B, np.float32), dev(torch, vals, np.float32)
    scratch = torch.zeros(4, dtype=torch.int32, device="cuda")
    flags = C.c_int32(-1)

    def check(ptr_, idx_, n=nnz, v=None):
        p, i = dev(torch, ptr_, np.int32), dev(torch, idx_, np.int32)
        return lib.lf_csr_check(p.data_ptr(), i.data_ptr(), v, rows, cols, n, scratch.data_ptr(), C.byref(flags), None)

    def product(ptr_, idx_, n=nnz):
        p, i = dev(torch, ptr_, np.int32), dev(torch, idx_, np.int32)
        out = torch.full((rows, feat), 7.0, device="cuda")
        rc = lib.lf_csr_spmm(p.data_ptr(), i.data_ptr(), dV.data_ptr(), rows, cols, n, feat, 0, dB.data_ptr(),
                             out.data_ptr(), scratch.data_ptr(), None)
        torch.cuda.synchronize()
        return rc, out

    assert check(indptr, indices, v=dV.data_ptr()) == 0 and flags.value == L.LF_CSR_CANONICAL
    ones = torch.ones(nnz, device="cuda")
    assert check(indptr, indices, v=ones.data_ptr()) == 0 and flags.value == L.LF_CSR_CANONICAL | L.LF_CSR_UNIT_VALUES
    rc, out = product(indptr, indices)
    assert rc == 0
    ref = O.spmm_csr_f64(indptr, indices, vals, (rows, cols), B)
    bound = O.spmm_abs_bound(indptr, indices, vals, (rows, cols), B)
    assert (np.abs(out.cpu().numpy() - ref) <= 1e-5 * bound).all()
    # the trusted entry gives the same bits
    p, i = dev(torch, indptr, np.int32), dev(torch, indices, np.int32)
    out2 = torch.empty_like(out)
    assert lib.lf_csr_spmm_trusted(p.data_ptr(), i.data_ptr(), dV.data_ptr(), rows, cols, feat, 0, dB.data_ptr(),
                                   out2.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, out2)

    # valid but not canonical: a swapped pair inside a row, a repeated column
    r = int(np.argmax(deg >= 3))
    swapped = indices.copy()
    swapped[indptr[r]], swapped[indptr[r] + 1] = indices[indptr[r] + 1], indices[indptr[r]]
    assert check(indptr, swapped) == 0 and flags.value == 0
    repeated = indices.copy()
    repeated[indptr[r] + 1] = repeated[indptr[r]]
    assert check(indptr, repeated) == 0 and flags.value == 0
    assert product(indptr, swapped)[0] == 0                    # still a product one can compute

    bad_cases = []
    for bad_col in (cols, -1, 2**31 - 1):
        idx = indices.copy(); idx[nnz // 2] = bad_col
        bad_cases.append((indptr, idx, nnz))
    ptr = indptr.copy(); ptr[rows // 2] = ptr[rows // 2 + 1] + 3          # decreasing
    bad_cases.append((ptr, indices, nnz))
    ptr = indptr.copy(); ptr[0] = 1                                         # does not start at 0
    bad_cases.append((ptr, indices, nnz))
    ptr = indptr.copy(); ptr[-1] = nnz + 1000                               # runs past the arrays
    bad_cases.append((ptr, indices, nnz))
    bad_cases.append((indptr, indices, nnz - 1))                            # nnz does not match
    ptr = indptr.copy(); ptr[3] = -4
    bad_cases.append((ptr, indices, nnz))
    for ptr_, idx_, n in bad_cases:
        assert check(ptr_, idx_, n) == L.LF_ERR_INVALID
        rc, out = product(ptr_, idx_, n)
        assert rc == L.LF_ERR_INVALID and "lf_csr_spmm" in L.last_error()
        assert float(out.min()) == 7.0 and float(out.max()) == 7.0          # nothing was written
    # no scratch, no check: refused rather than run unchecked
    p, i = dev(torch, indptr, np.int32), dev(torch, indices, np.int32)
    out = torch.empty((rows, feat), device="cuda")
    assert lib.lf_csr_spmm(p.data_ptr(), i.data_ptr(), dV.data_ptr(), rows, cols, nnz, feat, 0, dB.data_ptr(),
                           out.data_ptr(), None, None) == L.LF_ERR_INVALID

    # BSR: the block structure is a CSR of blocks
    mb, nb, bs, bfeat = 12, 9, 32, 64
    bdeg = rng.integers(0, 4, size=mb)
    bptr = np.concatenate(([0], np.cumsum(bdeg))).astype(np.int32)
    nnzb = int(bptr[-1])
    bidx = np.concatenate([np.sort(rng.choice(nb, size=d, replace=False)) for d in bdeg]).astype(np.int32)
    data = (torch.rand(nnzb * bs * bs, device="cuda") - 0.5).to(torch.float16)
    X = (torch.rand((nb * bs, bfeat), device="cuda") - 0.5).to(torch.float16)

    def bsr(ptr_, idx_, n=nnzb):
        p, i = dev(torch, ptr_, np.int32), dev(torch, idx_, np.int32)
        Y = torch.full((mb * bs, bfeat), 3.0, device="cuda", dtype=torch.float16)
        rc = lib.lf_bsr_spmm(p.data_ptr(), i.data_ptr(), data.data_ptr(), mb, nb, n, bs, bfeat, X.data_ptr(),
                             Y.data_ptr(), scratch.data_ptr(), None)
        torch.cuda.synchronize()
        return rc, Y

    assert bsr(bptr, bidx)[0] == 0
    for bad in (nb, -2):
        idx = bidx.copy(); idx[nnzb // 2] = bad
        rc, Y = bsr(bptr, idx)
        assert rc == L.LF_ERR_INVALID and "lf_bsr_spmm" in L.last_error()
        assert float(Y.float().min()) == 3.0 and float(Y.float().max()) == 3.0
    ptr = bptr.copy(); ptr[-1] += 5
    assert bsr(ptr, bidx)[0] == L.LF_ERR_INVALID
    assert bsr(bptr, bidx, nnzb + 1)[0] == L.LF_ERR_INVALID
