"""Shared helpers for the test-suite (not collected by pytest)."""
import numpy as np

from liteform_ae_amd.format_matrix_market import MTX
from oracle import liteform_oracle as O


def mtx_from_rows(rows_to_cols, shape):
    r, c = [], []
    for i, cols in enumerate(rows_to_cols):
        for j in cols:
            r.append(i)
            c.append(j)
    return MTX.from_coo(np.array(r, dtype=np.int64), np.array(c, dtype=np.int64), shape)


def skewed_matrix(rng, nr, nc, mean_deg=6.0, heavy_rows=2, heavy_len=None, values=True):
    """Random CSR with log-normal row lengths plus a few very long rows."""
    deg = np.clip(np.rint(rng.lognormal(np.log(mean_deg), 1.0, size=nr)), 0, nc).astype(np.int64)
    for _ in range(heavy_rows):
        deg[rng.integers(nr)] = heavy_len or min(nc, max(8, nc // 2))
    rows = np.repeat(np.arange(nr), deg)
    cols = rng.integers(0, nc, size=len(rows))
    key = np.unique(rows * nc + cols)
    rows, cols = key // nc, key % nc
    data = rng.uniform(-1, 1, size=len(rows)).astype(np.float32) if values else None
    return MTX.from_coo(rows, cols, (nr, nc), data=data)


def stats_from_oracle(g, num_parts, width_limit=1024):
    """What lf_bucket_stats must return, derived from the oracle's initial buckets."""
    pools = O.get_init_buckets_sequential(g, num_parts, width_limit)
    stats = np.zeros((num_parts, 11, 4), np.int64)
    hist = np.zeros((num_parts, 2048), np.int64)
    ncols = g.num_dst_nodes()
    psize = -(-ncols // num_parts)
    for p, pool in enumerate(pools):
        colmask = {}
        for w, b in pool.items():
            k = w.bit_length() - 1
            stats[p, k, :3] = (b.num_rows, b.nnz, len(b.row_indices))
            for col in b.col_indices:
                colmask[col] = colmask.get(col, 0) | (1 << k)
        lo, hi = p * psize, min(ncols, (p + 1) * psize)
        if hi > lo:
            masks = np.zeros(hi - lo, np.int64)
            for col, m in colmask.items():
                masks[col - lo] = m
            hist[p] = np.bincount(masks, minlength=2048)
    return stats, hist


def assert_hyb_equal(got, want):
    """Bit-exact comparison of two (rows, cols, mask) results, shapes included."""
    for name, a_parts, b_parts in zip(("rows", "cols", "mask"), got, want):
        assert len(a_parts) == len(b_parts), name
        for p, (ab, bb) in enumerate(zip(a_parts, b_parts)):
            assert len(ab) == len(bb), (name, p)
            for b, (x, y) in enumerate(zip(ab, bb)):
                assert x.shape == y.shape, (name, p, b, x.shape, y.shape)
                np.testing.assert_array_equal(x, y, err_msg=f"{name}[{p}][{b}]")
