"""Pins the CPU oracle (oracle/liteform_oracle.py) without running the reference.

The reference ships no tests, golden vectors or result files for this path, so the
oracle is pinned by (1) known answers evaluated by hand from the reference's source
(format_algos.py:226-385, 623-648, 709-774, 819-954, 1035-1166), (2) brute force on
tiny inputs, (3) invariants, and (4) agreement of two independent formulations.
"""
import itertools

import numpy as np
import pytest
import scipy.sparse as sp

from liteform_ae_amd.format_matrix_market import MTX
from oracle import liteform_oracle as O


def mtx_from_rows(rows_to_cols, shape):
    r, c = [], []
    for i, cols in enumerate(rows_to_cols):
        for j in cols:
            r.append(i)
            c.append(j)
    return MTX.from_coo(np.array(r, dtype=np.int64), np.array(c, dtype=np.int64), shape)


HAND = [[0, 1, 2, 5], [1], [], [0, 1, 2, 3, 4, 6], [2, 7], [0, 3, 4, 5, 6]]


def keys(pool):
    return {w: b.key() for w, b in pool.items()}


# ------------------------------------------------------------------ hand-worked example A
def test_hand_example_init_buckets():
    g = mtx_from_rows(HAND, (6, 8))
    pools = O.get_init_buckets_sequential(g, 2)
    #            width: (width, cost rows, nnz, |rows|, |cols|)
    assert keys(pools[0]) == {1: (1, 2, 2, 2, 2), 2: (2, 1, 2, 1, 2), 4: (4, 2, 7, 2, 4)}
    assert keys(pools[1]) == {1: (1, 2, 2, 2, 2), 2: (2, 1, 2, 1, 2), 4: (4, 1, 3, 1, 3)}
    assert pools[0][1].row_indices == [1, 4] and pools[0][1].col_indices == {1, 2}
    assert pools[0][2].row_indices == [5] and pools[0][2].col_indices == {0, 3}
    assert pools[0][4].row_indices == [0, 3] and pools[0][4].col_indices == {0, 1, 2, 3}
    assert pools[1][4].row_indices == [5] and pools[1][4].col_indices == {4, 5, 6}


def test_hand_example_single_row_fixup():
    g = mtx_from_rows(HAND, (6, 8))
    pools = O.get_init_buckets_sequential(g, 2)
    O.modify_single_row_buckets(pools)
    assert list(pools[0].keys()) == [1, 4]
    assert keys(pools[0]) == {1: (1, 4, 4, 3, 4), 4: (4, 2, 7, 2, 4)}
    assert pools[0][1].row_indices == [1, 4, 5]
    assert list(pools[1].keys()) == [1, 2]
    assert keys(pools[1]) == {1: (1, 2, 2, 2, 2), 2: (2, 3, 5, 2, 3)}
    assert pools[1][2].row_indices == [3, 5] and pools[1][2].col_indices == {4, 5, 6}


def test_hand_example_costs_and_config():
    g = mtx_from_rows(HAND, (6, 8))
    cfg = O.OracleCostModelSettings(32, 2)
    tr = O.search_cost_trace(g, 2, cfg)
    assert tr[0] == [([1, 4], 472.0), ([1, 2], 536.0), ([1], 536.0)]
    assert tr[1] == [([1, 2], 336.0), ([1], 400.0)]
    assert O.search_bucket_config(g, 2, cfg) == [[1, 4], [1, 2]]


def test_hand_example_hyb_slabs():
    g = mtx_from_rows(HAND, (6, 8))
    for build in (O.build_hyb_format_sequential, O.build_hyb_format_closed_form):
        rows, cols, mask = build(g, [[1, 4], [1, 2]])
        assert rows[0][0].tolist() == [1, 4]
        assert cols[0][0].tolist() == [[1], [2]]
        assert mask[0][0].tolist() == [[1], [1]]
        assert rows[0][1].tolist() == [0, 3, 5]
        assert cols[0][1].tolist() == [[0, 1, 2, 0], [0, 1, 2, 3], [0, 3, 0, 0]]
        assert mask[0][1].tolist() == [[1, 1, 1, 0], [1, 1, 1, 1], [1, 1, 0, 0]]
        assert rows[1][0].tolist() == [0, 4]
        assert cols[1][0].tolist() == [[5], [7]]
        assert rows[1][1].tolist() == [3, 5, 5]          # row 5 split over two ELL rows
        assert cols[1][1].tolist() == [[4, 6], [4, 5], [6, 0]]
        assert mask[1][1].tolist() == [[1, 1], [1, 1], [1, 0]]


# ------------------------------------------------------------------ hand-worked example B
def test_stale_snapshot_makes_zero_row_bucket():
    """Widths {8 (one row), 1 (one row)}: 8 folds into a new width 4; the width-1 fix-up
    then looks for a target in the *old* key list, finds 8 (already deleted) and
    re-creates it with ratio 1 // 8 = 0 cost-model rows (format_algos.py:638-641, 917)."""
    g = mtx_from_rows([[0, 1, 2, 3, 4, 5], [7]], (2, 8))
    pools = O.get_init_buckets_sequential(g, 1)
    assert keys(pools[0]) == {1: (1, 1, 1, 1, 1), 8: (8, 1, 6, 1, 6)}
    O.modify_single_row_buckets(pools)
    assert list(pools[0].keys()) == [4, 8]              # insertion order, not sorted
    assert keys(pools[0]) == {4: (4, 2, 6, 1, 6), 8: (8, 0, 1, 1, 1)}
    cfg = O.OracleCostModelSettings(32, 1)
    tr = O.search_cost_trace(g, 1, cfg)[0]
    # base: w4 non-atomic 16+192+32=240 ; w8 atomic with 0 padded rows 0+32+0=32
    assert tr == [([4, 8], 272.0), ([4], 304.0), ([2], 368.0), ([1], 496.0)]
    assert O.search_bucket_config(g, 1, cfg) == [[4, 8]]
    rows, cols, mask = O.build_hyb_format_sequential(g, [[4, 8]])
    assert rows[0][0].tolist() == [1] and cols[0][0].tolist() == [[7, 0, 0, 0]]
    assert rows[0][1].tolist() == [0] and cols[0][1].tolist() == [[0, 1, 2, 3, 4, 5, 0, 0]]


def test_width_one_merges_into_existing_bucket_with_ratio_zero():
    g = mtx_from_rows([[0, 1, 2], [1, 2, 3], [5], [0, 2, 4, 6]], (4, 8))
    pools = O.get_init_buckets_sequential(g, 1)
    assert keys(pools[0]) == {1: (1, 1, 1, 1, 1), 4: (4, 3, 10, 3, 6)}
    O.modify_single_row_buckets(pools)
    # rows unchanged (3 + 1*0), nnz and index sets merged
    assert keys(pools[0]) == {4: (4, 3, 11, 4, 7)}
    assert pools[0][4].row_indices == [0, 1, 3, 2]


def test_single_nonzero_partition_raises():
    g = mtx_from_rows([[3]], (1, 8))
    with pytest.raises(ValueError, match="only having 1 non-zero element"):
        O.search_bucket_config(g, 1, O.OracleCostModelSettings(32, 1))
    # second partition holds a single nonzero
    g = mtx_from_rows([[0, 1], [0, 2, 6]], (2, 8))
    with pytest.raises(ValueError):
        O.search_bucket_config(g, 2, O.OracleCostModelSettings(32, 2))


def test_empty_partition_gives_empty_width_list():
    g = mtx_from_rows([[0, 1], [0, 2], [1, 3]], (3, 8))
    cfgs = O.search_bucket_config(g, 2, O.OracleCostModelSettings(64, 2))
    assert cfgs[1] == []
    rows, cols, mask = O.build_hyb_format_sequential(g, cfgs)
    assert rows[1] == [] and cols[1] == []


def test_long_row_above_width_limit():
    # degree 2500 -> next pow2 4096 -> width 1024, 4 cost-model rows (format_algos.py:878-882)
    assert O.initial_width(2500) == (1024, 4)
    assert O.initial_width(1024) == (1024, 1)
    assert O.initial_width(1025) == (1024, 2)
    assert O.initial_width(1) == (1, 1) and O.initial_width(3) == (4, 1)
    for d in list(range(1, 70)) + [2**k + e for k in range(6, 20) for e in (-1, 0, 1)]:
        import math
        assert O.initial_width(d, 1 << 40)[0] == int(2 ** math.ceil(math.log2(d)))


# ------------------------------------------------------------------ brute force / invariants
def random_mtx(rng, nr, nc, density, heavy=0):
    a = rng.random((nr, nc)) < density
    for _ in range(heavy):
        a[rng.integers(nr)] = rng.random(nc) < 0.9
    return a


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("parts", [1, 2, 3])
def test_init_buckets_brute_force(seed, parts):
    rng = np.random.default_rng(seed)
    nr, nc = 23, 37
    a = random_mtx(rng, nr, nc, 0.12, heavy=1)
    r, c = np.nonzero(a)
    g = MTX.from_coo(r, c, (nr, nc))
    psize = -(-nc // parts)
    pools = O.get_init_buckets_sequential(g, parts, width_limit=8)
    stats = O.init_bucket_stats_closed_form(g, parts, width_limit=8)
    for p in range(parts):
        sub = a[:, p * psize:(p + 1) * psize]
        expect = {}
        for i in range(nr):
            d = int(sub[i].sum())
            if d == 0:
                continue
            w = 1
            while w < d:
                w *= 2
            mr = 1
            if w > 8:
                mr, w = w // 8, 8
            e = expect.setdefault(w, [0, 0, [], set()])
            e[0] += mr
            e[1] += d
            e[2].append(i)
            e[3] |= set((np.nonzero(sub[i])[0] + p * psize).tolist())
        assert list(pools[p].keys()) == sorted(expect)
        for w, (mr, nnz, rl, cs) in expect.items():
            assert pools[p][w].key() == (w, mr, nnz, len(rl), len(cs))
            assert pools[p][w].row_indices == rl and pools[p][w].col_indices == cs
            assert stats[p][w] == (w, mr, nnz, len(rl), len(cs))


def pow2_configs(max_w, rng, k):
    ws = [1 << i for i in range(max_w.bit_length())]
    out = []
    for _ in range(k):
        n = rng.integers(1, len(ws) + 1)
        out.append(sorted(rng.choice(ws, size=n, replace=False).tolist()))
    return out


@pytest.mark.parametrize("seed", range(8))
def test_builder_round_trip_and_two_formulations(seed):
    rng = np.random.default_rng(100 + seed)
    nr, nc = 40, 53
    parts = int(rng.integers(1, 5))
    a = random_mtx(rng, nr, nc, 0.15, heavy=2)
    r, c = np.nonzero(a)
    g = MTX.from_coo(r, c, (nr, nc))
    psize = -(-nc // parts)
    widths = [pow2_configs(16, rng, 1)[0] for _ in range(parts)]
    rows, cols, mask = O.build_hyb_format_sequential(g, widths)
    rows2, cols2, mask2 = O.build_hyb_format_closed_form(g, widths)
    recon = np.zeros_like(a, dtype=np.int64)
    for p in range(parts):
        for b, w in enumerate(widths[p]):
            assert rows[p][b].shape == (len(rows[p][b]),)
            assert cols[p][b].shape == (len(rows[p][b]), w) == mask[p][b].shape
            np.testing.assert_array_equal(rows[p][b], rows2[p][b])
            np.testing.assert_array_equal(cols[p][b], cols2[p][b])
            np.testing.assert_array_equal(mask[p][b], mask2[p][b])
            # padding is (0, 0) and only at the tail of an ELL row
            assert (cols[p][b][mask[p][b] == 0] == 0).all()
            assert (np.diff(mask[p][b], axis=1) <= 0).all()
            assert (np.diff(rows[p][b]) >= 0).all()
            if b + 1 < len(widths[p]):
                assert (np.diff(rows[p][b]) > 0).all()      # split rows only in the widest bucket
            e, s = np.nonzero(mask[p][b])
            cc = cols[p][b][e, s]
            assert ((cc // psize) == p).all()
            np.add.at(recon, (rows[p][b][e], cc), 1)
            # entries of a row come out in ascending column order (CSR order)
            for row in np.unique(rows[p][b]):
                seq = cols[p][b][rows[p][b] == row][mask[p][b][rows[p][b] == row] == 1]
                assert (np.diff(seq) > 0).all()
    np.testing.assert_array_equal(recon, a.astype(np.int64))   # every nonzero exactly once
    # exact product with small integers
    B = rng.integers(-3, 4, size=(nc, 5)).astype(np.float64)
    vals = [[m.astype(np.float64) for m in mp] for mp in mask]
    np.testing.assert_array_equal(O.spmm_from_hyb(rows, cols, vals, nr, B), a.astype(np.float64) @ B)


def test_builder_bucket_choice_rule():
    """degree d goes to the first width >= d, else to the last (format_algos.py:275-279)."""
    g = mtx_from_rows([[0], [0, 1], [0, 1, 2], [0, 1, 2, 3, 4], list(range(9))], (5, 16))
    rows, cols, mask = O.build_hyb_format_sequential(g, [[2, 4]])
    assert rows[0][0].tolist() == [0, 1]
    assert rows[0][1].tolist() == [2, 3, 3, 4, 4, 4]
    assert cols[0][1].tolist() == [[0, 1, 2, 0], [0, 1, 2, 3], [4, 0, 0, 0],
                                   [0, 1, 2, 3], [4, 5, 6, 7], [8, 0, 0, 0]]


def test_duplicate_coo_entries_count_in_degree_not_in_fill():
    """Degrees come from raw COO triplets, the fill from the de-duplicated CSR
    (format_algos.py:250-254)."""
    g = MTX.from_coo([0, 0, 0, 1], [1, 1, 2, 3], (2, 4))     # (0,1) twice
    rows, cols, mask = O.build_hyb_format_sequential(g, [[2, 4]])
    assert rows[0][0].tolist() == [1]              # degree 1 -> width 2
    assert rows[0][1].tolist() == [0]              # COO degree 3 -> width 4, but 2 entries
    assert cols[0][1].tolist() == [[1, 2, 0, 0]]
    r2 = O.build_hyb_format_closed_form(g, [[2, 4]])
    np.testing.assert_array_equal(r2[1][0][1], cols[0][1])


# ------------------------------------------------------------------ search properties
def independent_cost(state, feat, parts):
    """Cost of a state given as {width: (cost_rows, n_out_rows, n_cols)}, summed in the
    given order, written from the formula in the paper's terms rather than the code:
    2*I*K + |cols|*J + (atomic ? I : |rows|)*J with I padded to the widest block."""
    max_w = max(state)
    tot = 0
    for w, (mr, n_out, n_cols) in state.items():
        blk = max_w // w
        I = -(-mr // blk) * blk
        tot += 2 * I * w + n_cols * feat + ((I / n_out) * n_out * feat if (parts > 1 or w == max_w) else n_out * feat)
    return tot


@pytest.mark.parametrize("seed", range(10))
def test_search_returns_strict_minimum_of_fold_chain(seed):
    rng = np.random.default_rng(500 + seed)
    nr, nc = 60, 64
    parts = int(rng.integers(1, 4))
    feat = int(rng.choice([32, 64, 128, 512]))
    a = random_mtx(rng, nr, nc, 0.1, heavy=3)
    r, c = np.nonzero(a)
    g = MTX.from_coo(r, c, (nr, nc))
    cfg = O.OracleCostModelSettings(feat, parts)
    try:
        result = O.search_bucket_config(g, parts, cfg)
    except ValueError:
        pytest.skip("single-nonzero partition")
    traces = O.search_cost_trace(g, parts, cfg)
    for p, tr in enumerate(traces):
        if not tr:
            assert result[p] == []
            continue
        costs = [c for _, c in tr]
        best = min(costs)
        first = costs.index(best)                      # strict <: the earliest minimum wins
        assert result[p] == tr[first][0]
        assert all(w & (w - 1) == 0 for w in result[p]) and result[p] == sorted(result[p])
        # last state is the single width-1 bucket holding everything
        assert tr[-1][0] == [1] or len(tr) == 1
    # recompute every state's cost from scratch, independently of get_memory_cost
    pools = O.get_init_buckets_sequential(g, parts)
    O.modify_single_row_buckets(pools)
    for p, pool in enumerate(pools):
        if not pool:
            continue
        k = 0
        state = {w: (b.num_rows, len(b.row_indices), len(b.col_indices)) for w, b in pool.items()}
        assert independent_cost(state, feat, parts) == traces[p][k][1]
        pre = max(pool)
        new = pre // 2
        while new >= 1:
            O.move_largest_bucket(pool, pre, new)
            k += 1
            state = {w: (b.num_rows, len(b.row_indices), len(b.col_indices)) for w, b in pool.items()}
            assert independent_cost(state, feat, parts) == traces[p][k][1]
            pre, new = new, new // 2


def test_spmm_anchors():
    rng = np.random.default_rng(7)
    n = 50
    B = rng.standard_normal((n, 8))
    eye = sp.identity(n, format="csr")
    np.testing.assert_array_equal(O.spmm_csr_f64(eye.indptr, eye.indices, eye.data, (n, n), B), B)
    dense_row = sp.csr_matrix(np.ones((1, n)))
    np.testing.assert_allclose(
        O.spmm_csr_f64(dense_row.indptr, dense_row.indices, dense_row.data, (1, n), B),
        B.sum(0, keepdims=True), rtol=1e-13)
    a = sp.random(n, n, 0.1, random_state=3, format="csr")
    np.testing.assert_allclose(O.spmm_csr_f64(a.indptr, a.indices, a.data, (n, n), B),
                               a.toarray() @ B, rtol=1e-12, atol=1e-12)
    g = MTX(None)
    g.coo_mtx = a.tocoo()
    np.testing.assert_allclose(O.spmm_reference_f64(g, B), a.toarray() @ B, rtol=1e-12, atol=1e-12)


def test_bsr_oracle_against_dense():
    rng = np.random.default_rng(2)
    blocks = rng.uniform(-1, 1, size=(5, 32, 32)).astype(np.float32)
    a = sp.bsr_matrix((blocks, np.array([0, 2, 1, 0, 2]), np.array([0, 2, 3, 5])), shape=(96, 96))
    x = rng.uniform(-1, 1, size=(96, 7))
    np.testing.assert_allclose(O.spmm_bsr_f64(a, x), a.toarray().astype(np.float64) @ x, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(O.spmm_bsr_abs_bound(a, x), np.abs(a.toarray()).astype(np.float64) @ np.abs(x),
                               rtol=1e-12, atol=1e-12)
    eye = sp.identity(64, format="csr").tobsr(blocksize=(32, 32))
    np.testing.assert_array_equal(O.spmm_bsr_f64(eye, x[:64]), x[:64])
