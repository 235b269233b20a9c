"""Full-size checks of the remaining benchmark workloads, at the shape the benchmark runs:

  cfg2  170k x 170k power-law graph, N = 128, two column partitions
  cfg4  27-point stencil on a 100^3 grid, N = 256 (the row-group kernel must serve it)
  cfg5  500k x 2M skewed matrix with 50 rows of 100k entries, bf16 B, N = 512

The oracle's Python loops cannot run at these sizes, so (as for the 2.45M-row graph) the
format is checked through size-independent properties on the GPU - every nonzero exactly
once and in its column partition, padding (0, 0), ascending rows, the bucket rule
(format_algos.py:275-279), split rows only in a partition's widest bucket
(format_algos.py:286-305) - the statistics against numpy, and the product through
run-to-run identity and a slice of rows against scipy CSR(f64) @ dense(f64) with the bound
1e-5 * sum|a||b|."""
import numpy as np
import pytest
import scipy.sparse as sp

from oracle import liteform_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-5


def seg_degrees(indptr, indices, rows, cols, parts):
    """deg[p][r]: entries of row r in column partition p."""
    psize = -(-cols // parts)
    if parts == 1:
        return np.diff(indptr).astype(np.int64).reshape(1, rows), psize
    row_of = np.repeat(np.arange(rows, dtype=np.int64), np.diff(indptr))
    key = (indices // psize).astype(np.int64) * rows + row_of
    return np.bincount(key, minlength=parts * rows).reshape(parts, rows), psize


def check_statistics(fa, g, parts):
    rows, cols = g.coo_mtx.shape
    indptr, indices, _ = g.adj_tensors("csr")
    stats, hist = fa.bucket_statistics(g, parts)
    deg_all, psize = seg_degrees(indptr, indices, rows, cols, parts)
    for p in range(parts):
        deg = deg_all[p]
        deg = deg[deg > 0]
        cls = np.where(deg <= 1, 0, np.ceil(np.log2(np.maximum(deg, 1))).astype(np.int64))
        cost_rows = np.where(cls > 10, 1 << np.maximum(cls - 10, 0), 1)
        cls = np.minimum(cls, 10)
        for k in range(11):
            m = cls == k
            assert stats[p, k, 0] == cost_rows[m].sum()
            assert stats[p, k, 1] == deg[m].sum()
            assert stats[p, k, 2] == m.sum()
        lo, hi = p * psize, min(cols, (p + 1) * psize)
        assert hist[p].sum() == max(0, hi - lo)
        touched = np.zeros(cols, dtype=bool)
        touched[indices] = True
        assert hist[p, 1:].sum() == touched[lo:hi].sum()
    return stats


def check_round_trip(fa, torch, g, cfg):
    rows, cols = g.coo_mtx.shape
    parts = len(cfg)
    fmt = fa.build_hyb_format_device(g, cfg)
    indptr, indices, data = g.adj_tensors("csr")
    deg_all, psize = seg_degrees(indptr, indices, rows, cols, parts)
    d_deg = torch.from_numpy(deg_all).cuda()
    keys, vals = [], []
    for k in range(fmt.num_buckets):
        W = fmt.flat_widths[k]
        R = int(fmt.ell_rows[k])
        if R == 0:
            continue
        p = fmt.part_of[k]
        r, c, v, meta = fmt.slab(k)[:4]
        c = c.view(R, W)
        v = v.view(R, W)
        ln = (meta & 0x7FF).to(torch.int64)
        valid = torch.arange(W, device="cuda").view(1, W) < ln.view(R, 1)
        assert bool((c[~valid] == 0).all()) and bool((v[~valid] == 0).all())      # padding is (0, 0)
        assert bool((ln >= 1).all()) and bool((ln <= W).all())
        assert bool((r[1:] >= r[:-1]).all())                                      # ascending source rows
        cv = c[valid].to(torch.int64)
        assert bool((cv // psize == p).all())                                     # right column partition
        widths = fmt.bucket_widths[p]
        b = widths.index(W)
        is_last = b + 1 == len(widths)
        if not is_last:
            assert bool((r[1:] > r[:-1]).all())                                   # split rows only in the widest
        # bucket rule: first width >= degree, else the last
        deg = d_deg[p][r.to(torch.int64)]
        assert bool((deg > (widths[b - 1] if b else 0)).all())
        if not is_last:
            assert bool((deg <= W).all())
        rr = r.to(torch.int64).view(R, 1).expand(R, W)[valid]
        keys.append(rr * cols + cv)
        vals.append(v[valid])
    keys = torch.cat(keys)
    vals = torch.cat(vals)
    assert keys.numel() == g.num_edges()
    order = torch.argsort(keys)
    d_indptr = torch.from_numpy(indptr.astype(np.int64)).cuda()
    want_rows = torch.repeat_interleave(torch.arange(rows, device="cuda"), d_indptr[1:] - d_indptr[:-1])
    want = want_rows * cols + torch.from_numpy(indices.astype(np.int64)).cuda()
    assert torch.equal(keys[order], want)                       # every nonzero exactly once
    assert torch.equal(vals[order], torch.from_numpy(np.asarray(data, dtype=np.float32)).cuda())
    return fmt


def check_rows_against_scipy(g, C_dev, B_host, row_ids, feat_slices):
    """C[row_ids][:, features] against scipy in float64 with the 1e-5 * sum|a||b| bound."""
    rows, cols = g.coo_mtx.shape
    indptr, indices, data = g.adj_tensors("csr")
    csr = sp.csr_matrix((np.asarray(data, dtype=np.float32), indices, indptr), shape=(rows, cols))
    sub = csr[row_ids]
    for sl in feat_slices:
        Bs = np.ascontiguousarray(B_host[:, sl])
        ref = O.spmm_csr_f64(sub.indptr, sub.indices, sub.data, sub.shape, Bs)
        bound = O.spmm_abs_bound(sub.indptr, sub.indices, sub.data, sub.shape, Bs)
        got = C_dev[row_ids][:, sl].cpu().numpy().astype(np.float64)
        excess = float((np.abs(got - ref) - TOL * bound).max())
        assert excess <= 0, f"outside 1e-5 * sum|a||b| by {excess} (features {sl})"


@pytest.fixture(scope="module")
def env():
    import torch
    from liteform_ae_amd import format_algos as fa
    from liteform_ae_amd.synthetic import make_workload
    return fa, torch, make_workload


def test_cfg2_full_size_two_partitions(env):
    fa, torch, make_workload = env
    wl = make_workload("cfg2")
    g = wl.matrix
    rows, cols = wl.shape
    feat, parts = 128, 2
    assert (rows, cols) == (170_000, 170_000) and wl.num_parts == parts and wl.feat_size == feat
    check_statistics(fa, g, parts)
    for model in ("reference", "gfx950"):
        cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts, cost_model=model))
        assert len(cfg) == parts
        fmt = check_round_trip(fa, torch, g, cfg)
        plan = fa.HybSpMM(fmt, feat)
        assert plan.info["launches"] == parts
        gen = torch.Generator(device="cuda").manual_seed(2)
        B = torch.rand((cols, feat), device="cuda", generator=gen) * 2 - 1
        C1 = plan.run(B).clone()
        assert torch.equal(C1, plan.run(B))                               # bit reproducible
        plan.close()
        # every row: the matrix is small enough for scipy in float64
        check_rows_against_scipy(g, C1, B.cpu().numpy(), np.arange(rows), [slice(0, feat)])


def test_cfg4_full_size_row_groups(env, monkeypatch):
    fa, torch, make_workload = env
    wl = make_workload("cfg4")
    g = wl.matrix
    rows, cols = wl.shape
    feat = 256
    assert rows == 100 ** 3 and wl.nnz == 26_463_592 and wl.feat_size == feat
    check_statistics(fa, g, 1)
    cfg = fa.search_bucket_config(g, 1, fa.CostModelSettings(feat, 1, cost_model="gfx950"))
    fmt = check_round_trip(fa, torch, g, cfg)
    gen = torch.Generator(device="cuda").manual_seed(4)
    B = torch.rand((cols, feat), device="cuda", generator=gen) * 2 - 1
    plan = fa.HybSpMM(fmt, feat)
    assert plan.info["row_group_buckets"] >= 1                           # the stencil takes the shared-gather path
    assert plan.info["cell_buckets"] >= 1                                # ... as 16-row cells at fp32, N = 256
    C1 = plan.run(B).clone()
    assert torch.equal(C1, plan.run(B))
    plan.close()
    # the same product without row groups: same terms per row in the same (ascending column)
    # order, so for finite B the two paths agree to rounding of the fused multiply-adds
    monkeypatch.setenv("LF_ROW_GROUPS", "0")
    plain = fa.HybSpMM(fmt, feat)
    assert plain.info["row_group_buckets"] == 0
    C0 = plain.run(B).clone()
    plain.close()
    monkeypatch.delenv("LF_ROW_GROUPS")
    indptr, _, data = g.adj_tensors("csr")                                # no empty rows in the stencil
    row_abs = np.add.reduceat(np.abs(np.asarray(data, dtype=np.float64)), indptr[:-1])
    row_abs = torch.from_numpy(row_abs.astype(np.float32)).cuda().view(rows, 1)       # sum|a| >= sum|a||b|: |b| < 1
    assert bool(((C1 - C0).abs() <= 2e-5 * row_abs).all())
    # two feature windows (the shape the benchmark picks for this workload)
    win = fa.HybSpMM(fmt, feat, windows=2)
    Cw = win.run(B).clone()
    win.close()
    assert bool(((Cw - C0).abs() <= 2e-5 * row_abs).all())
    # rows from the grid's corner, faces and interior against scipy in float64
    rng = np.random.default_rng(4)
    row_ids = np.unique(np.concatenate([np.arange(0, 30_000), rng.integers(0, rows, size=30_000),
                                        np.arange(rows - 10_000, rows)]))
    Bh = B.cpu().numpy()
    check_rows_against_scipy(g, C1, Bh, row_ids, [slice(0, feat)])
    check_rows_against_scipy(g, Cw, Bh, row_ids, [slice(0, feat)])


def test_cfg5_full_size_bf16_heavy_rows(env):
    fa, torch, make_workload = env
    wl = make_workload("cfg5")
    g = wl.matrix
    rows, cols = wl.shape
    feat = 512
    assert (rows, cols) == (500_000, 2_000_000) and wl.b_dtype == "bf16" and wl.feat_size == feat
    indptr = g.adj_tensors("csr")[0]
    deg = np.diff(indptr)
    dense_rows = np.nonzero(deg == 100_000)[0]
    assert len(dense_rows) == 50
    check_statistics(fa, g, 1)
    gen = torch.Generator(device="cuda").manual_seed(5)
    B = (torch.rand((cols, feat), device="cuda", generator=gen) * 2 - 1).to(torch.bfloat16)
    # the features checked on the host (the whole of B in float64 would be 8 GB): both ends and
    # the seam between the two feature windows
    slices = [slice(0, 32), slice(240, 272), slice(480, 512)]
    Bh = np.zeros((cols, feat), dtype=np.float32)
    for sl in slices:
        Bh[:, sl] = B[:, sl].to(torch.float32).cpu().numpy()
    rng = np.random.default_rng(5)
    row_ids = np.unique(np.concatenate([dense_rows, np.arange(0, 20_000), rng.integers(0, rows, size=20_000)]))
    for parts in (1, 2):
        cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts, cost_model="gfx950"))
        fmt = check_round_trip(fa, torch, g, cfg)
        plan = fa.HybSpMM(fmt, feat, "bf16")
        assert plan.info["heavy_rows"] >= 50 * parts                      # the 100k-entry rows take the chunked tail
        C1 = plan.run(B).clone()
        assert torch.equal(C1, plan.run(B))
        plan.close()
        check_rows_against_scipy(g, C1, Bh, row_ids, slices)
        if parts == 1:
            # the shape the launch-shape model picks for this workload: two feature windows of 256
            assert fa.predict_launch_shape(g, feat, "bf16") == (1, 2)
            win = fa.HybSpMM(fmt, feat, "bf16", windows=2)
            assert win.info["launches"] == 2
            Cw = win.run(B).clone()
            assert torch.equal(Cw, win.run(B))
            win.close()
            check_rows_against_scipy(g, Cw, Bh, row_ids, slices)
            del Cw
        del fmt, plan, C1
