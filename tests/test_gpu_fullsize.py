"""Full-size checks on the headline workload (2.45M x 2.45M power-law graph, ~81.6M nnz).

The oracle's Python loops cannot run at this size, so the format is checked through
size-independent properties computed with torch on the GPU (round trip to CSR, bucket
rule, ordering), the statistics against numpy, and the product through linearity,
run-to-run identity and a slice of rows against scipy in float64."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def big():
    import torch
    from liteform_ae_amd import format_algos as fa
    from liteform_ae_amd.synthetic import make_workload
    wl = make_workload("cfg3")
    return wl, fa, torch


def test_statistics_full_size(big):
    wl, fa, torch = big
    g = wl.matrix
    stats, hist = fa.bucket_statistics(g, 1)
    indptr, indices, _ = g.adj_tensors("csr")
    deg = np.diff(indptr).astype(np.int64)
    deg = deg[deg > 0]
    cls = np.where(deg <= 1, 0, np.ceil(np.log2(np.maximum(deg, 1))).astype(np.int64))
    cost_rows = np.where(cls > 10, 1 << np.maximum(cls - 10, 0), 1)
    cls = np.minimum(cls, 10)
    for k in range(11):
        m = cls == k
        assert stats[0, k, 0] == cost_rows[m].sum()
        assert stats[0, k, 1] == deg[m].sum()
        assert stats[0, k, 2] == m.sum()
    assert hist[0].sum() == g.num_dst_nodes()
    # columns touched by at least one row = columns with a nonzero mask
    touched = np.zeros(g.num_dst_nodes(), dtype=bool)
    touched[indices] = True
    assert hist[0, 1:].sum() == touched.sum()
    # class-k column set size against numpy for two classes (the cheap ones)
    row_cls = np.full(g.num_src_nodes(), -1, dtype=np.int64)
    row_cls[np.diff(indptr) > 0] = cls
    for k in (9, 10):
        rows_k = np.nonzero(row_cls == k)[0]
        cols_k = np.unique(np.concatenate([indices[indptr[r]:indptr[r + 1]] for r in rows_k]))
        assert sum(int(hist[0, m]) for m in range(2048) if m >> k & 1) == len(cols_k)


@pytest.mark.parametrize("parts", [1, 2])
def test_column_set_histogram_full_size(big, parts):
    """Every bin of the class-mask histogram against numpy: per partition and class, the
    columns touched by rows of that class, then one mask per column."""
    wl, fa, torch = big
    g = wl.matrix
    rows, cols = wl.shape
    stats, hist = fa.bucket_statistics(g, parts)
    indptr, indices, _ = g.adj_tensors("csr")
    psize = -(-cols // parts)
    row_of = np.repeat(np.arange(rows, dtype=np.int32), np.diff(indptr))
    part_of = indices // psize
    for p in range(parts):
        sel = part_of == p
        idx_p, row_p = indices[sel], row_of[sel]
        deg = np.bincount(row_p, minlength=rows).astype(np.int64)
        cls = np.where(deg <= 1, 0, np.ceil(np.log2(np.maximum(deg, 1))).astype(np.int64))
        cls = np.minimum(cls, 10)
        cls_of_nnz = cls[row_p]
        mask = np.zeros(cols, dtype=np.int64)
        for k in range(11):
            touched = np.zeros(cols, dtype=bool)
            touched[idx_p[cls_of_nnz == k]] = True
            mask[touched] |= 1 << k
        lo, hi = p * psize, min(cols, (p + 1) * psize)
        want = np.bincount(mask[lo:hi], minlength=2048)
        np.testing.assert_array_equal(hist[p], want)
        for k in range(11):
            m = (cls == k) & (deg > 0)
            assert stats[p, k, 1] == deg[m].sum() and stats[p, k, 2] == m.sum()


@pytest.mark.parametrize("parts,model", [(1, "reference"), (2, "gfx950")])
def test_format_round_trip_full_size(big, parts, model):
    wl, fa, torch = big
    g = wl.matrix
    rows, cols = wl.shape
    cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(128, parts, cost_model=model))
    fmt = fa.build_hyb_format_device(g, cfg)
    indptr, indices, data = g.adj_tensors("csr")
    d_indptr = torch.from_numpy(indptr.astype(np.int64)).cuda()
    psize = -(-cols // parts)
    keys, vals = [], []
    for k in range(fmt.num_buckets):
        W = fmt.flat_widths[k]
        R = int(fmt.ell_rows[k])
        if R == 0:
            continue
        r, c, v, meta = fmt.slab(k)[:4]
        c = c.view(R, W)
        v = v.view(R, W)
        ln = (meta & 0x7FF).to(torch.int64)
        valid = torch.arange(W, device="cuda").view(1, W) < ln.view(R, 1)
        assert bool((c[~valid] == 0).all()) and bool((v[~valid] == 0).all())      # padding is (0, 0)
        assert bool((ln >= 1).all()) and bool((ln <= W).all())
        assert bool((r[1:] >= r[:-1]).all())                                      # ascending source rows
        p = fmt.part_of[k]
        cv = c[valid].to(torch.int64)
        assert bool((cv // psize == p).all())                                     # right column partition
        is_last = k + 1 == fmt.num_buckets or fmt.part_of[k + 1] != p
        if not is_last:
            assert bool((r[1:] > r[:-1]).all())                                   # split rows only in the widest
        rr = r.to(torch.int64).view(R, 1).expand(R, W)[valid]
        keys.append(rr * cols + cv)
        vals.append(v[valid])
        if parts == 1:
            # bucket rule: first width >= degree, else the last
            deg = (d_indptr[1:] - d_indptr[:-1])[r.to(torch.int64)]
            lo = fmt.bucket_widths[0][fmt.bucket_widths[0].index(W) - 1] if fmt.bucket_widths[0].index(W) else 0
            assert bool((deg > lo).all())
            if not is_last:
                assert bool((deg <= W).all())
    keys = torch.cat(keys)
    vals = torch.cat(vals)
    assert keys.numel() == g.num_edges()
    order = torch.argsort(keys)
    keys = keys[order]
    vals = vals[order]
    want_rows = torch.repeat_interleave(torch.arange(rows, device="cuda"), d_indptr[1:] - d_indptr[:-1])
    want = want_rows * cols + torch.from_numpy(indices.astype(np.int64)).cuda()
    assert torch.equal(keys, want)                      # every nonzero exactly once
    assert torch.equal(vals, torch.from_numpy(np.asarray(data, dtype=np.float32)).cuda())


def test_spmm_full_size_properties(big):
    wl, fa, torch = big
    from oracle import liteform_oracle as O
    g = wl.matrix
    rows, cols = wl.shape
    feat = 128
    for parts in (1, 2):
        cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts, cost_model="gfx950"))
        fmt = fa.build_hyb_format_device(g, cfg)
        plan = fa.HybSpMM(fmt, feat)
        gen = torch.Generator(device="cuda").manual_seed(3)
        B1 = torch.rand((cols, feat), device="cuda", generator=gen) * 2 - 1
        B2 = torch.rand((cols, feat), device="cuda", generator=gen) * 2 - 1
        C1 = plan.run(B1).clone()
        C1b = plan.run(B1)
        assert torch.equal(C1, C1b)                                   # bit reproducible
        C2 = plan.run(B2).clone()
        C12 = plan.run(B1 + B2)
        # linearity: A(B1 + B2) = A B1 + A B2 up to rounding; values are in [0, 1), |B| < 2
        deg = torch.from_numpy(np.diff(g.adj_tensors("csr")[0]).astype(np.float32)).cuda().view(rows, 1)
        assert bool(((C12 - (C1 + C2)).abs() <= 4e-5 * (deg + 1)).all())
        # a slice of rows against scipy in float64 with the stated tolerance
        take = 150_000
        indptr, indices, data = g.adj_tensors("csr")
        sub = int(indptr[take])
        Bh = B1.cpu().numpy()
        ref = O.spmm_csr_f64(indptr[:take + 1], indices[:sub], data[:sub], (take, cols), Bh)
        bound = O.spmm_abs_bound(indptr[:take + 1], indices[:sub], data[:sub], (take, cols), Bh)
        got = C1[:take].cpu().numpy()
        assert (np.abs(got - ref) <= 1e-5 * bound).all()
        plan.close()
        del fmt, plan


def _check_product(fa, torch, g, plan, feat, seed, take=150_000, slices=None):
    """Run-to-run identity, and the first `take` rows against scipy in float64 with the bound
    1e-5 * sum|a||b| (on the feature slices given, else on all features)."""
    from oracle import liteform_oracle as O
    rows, cols = g.num_src_nodes(), g.num_dst_nodes()
    gen = torch.Generator(device="cuda").manual_seed(seed)
    B = torch.rand((cols, feat), device="cuda", generator=gen) * 2 - 1
    C1 = plan.run(B).clone()
    assert torch.equal(C1, plan.run(B))                               # bit reproducible
    indptr, indices, data = g.adj_tensors("csr")
    sub = int(indptr[take])
    for sl in slices or [slice(0, feat)]:
        Bh = np.ascontiguousarray(B[:, sl].cpu().numpy())
        ref = O.spmm_csr_f64(indptr[:take + 1], indices[:sub], data[:sub], (take, cols), Bh)
        bound = O.spmm_abs_bound(indptr[:take + 1], indices[:sub], data[:sub], (take, cols), Bh)
        got = C1[:take, sl].cpu().numpy()
        excess = float((np.abs(got - ref) - 1e-5 * bound).max())
        assert excess <= 0, f"outside 1e-5 * sum|a||b| by {excess} (features {sl})"
    return B, C1


def test_headline_shape_one_partition_two_windows(big):
    """The shape the benchmark runs for N = 128: one column partition, two feature windows of 64.
    Checked like the single pass, and against it: windows change the lane count a row is summed
    with, so split and cooperatively reduced rows may differ in the last bits, other rows not."""
    wl, fa, torch = big
    g = wl.matrix
    feat = 128
    assert fa.predict_launch_shape(g, feat) == (1, 2)
    cfg = fa.search_bucket_config(g, 1, fa.CostModelSettings(feat, 1, cost_model="gfx950"))
    fmt = fa.build_hyb_format_device(g, cfg)
    plan = fa.HybSpMM(fmt, feat, windows=2)
    assert plan.info["launches"] == 2 and plan.info["windows"] == 2
    B, C2 = _check_product(fa, torch, g, plan, feat, seed=3)
    plan.close()
    single = fa.HybSpMM(fmt, feat)
    C1 = single.run(B)
    single.close()
    deg = torch.from_numpy(np.diff(g.adj_tensors("csr")[0]).astype(np.float32)).cuda().view(-1, 1)
    assert bool(((C2 - C1).abs() <= 2e-6 * (deg + 1)).all())
    short = (deg.view(-1) <= 64).nonzero().view(-1)[:500_000]         # one ELL row, summed slot by slot
    assert torch.equal(C2[short], C1[short])


@pytest.mark.parametrize("feat,shape", [(32, (1, 1)), (64, (1, 1)), (256, (1, 4))])
def test_feature_sweep_full_size(big, feat, shape):
    """The other feature sizes of the sweep (N = 32, 64, 256) at 2.45M rows, each with the launch
    shape the model picks for it: the tile and grid arithmetic at ~100k workgroups."""
    wl, fa, torch = big
    g = wl.matrix
    assert fa.predict_launch_shape(g, feat) == shape
    parts, windows = shape
    cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(feat, parts, cost_model="gfx950"))
    fmt = fa.build_hyb_format_device(g, cfg)
    plan = fa.HybSpMM(fmt, feat, windows=windows)
    slices = None if feat <= 64 else [slice(0, 32), slice(96, 160), slice(feat - 32, feat)]
    _check_product(fa, torch, g, plan, feat, seed=10 + feat, take=100_000, slices=slices)
    plan.close()


def test_launch_shape_model_on_the_headline_graph(big):
    """The model's choice for the 2.45M-row graph: one pass at 64 features, two feature windows
    at 128 (B is 1.25 GB against a 256 MB memory-side cache), as the measurements say."""
    wl, fa, torch = big
    g = wl.matrix
    assert fa.row_overlap_device(g) < 0.01
    assert fa.predict_launch_shape(g, 64) == (1, 1)
    best, table = fa.predict_launch_shape(g, 128, return_predictions=True)
    assert best == (1, 2)
    assert 5.0 < table[best] < 8.0            # predicted milliseconds (measured: 6.2)


