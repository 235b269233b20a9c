"""Host part of the bucket-width search (lf_search_bucket_config) against the oracle.

The statistics are taken from the oracle's initial buckets here, so these tests need no
GPU; the GPU tests check that lf_bucket_stats produces the same statistics."""
import numpy as np
import pytest

from liteform_ae_amd.format_algos import CostModelSettings, search_from_statistics
from oracle import liteform_oracle as O

from helpers import mtx_from_rows, skewed_matrix, stats_from_oracle

HAND = [[0, 1, 2, 5], [1], [], [0, 1, 2, 3, 4, 6], [2, 7], [0, 3, 4, 5, 6]]


def both(g, parts, feat, cfg_parts=None, limit=1024):
    cfg_parts = parts if cfg_parts is None else cfg_parts
    stats, hist = stats_from_oracle(g, parts, limit)
    got = search_from_statistics(stats, hist, CostModelSettings(feat, cfg_parts), width_limit=limit,
                                 return_trace=True)
    ocfg = O.OracleCostModelSettings(feat, cfg_parts)
    pools = O.get_init_buckets_sequential(g, parts, limit)
    O.modify_single_row_buckets(pools)
    want_cfg = O.get_bucket_config([dict(p) for p in _clone(pools)], ocfg)
    want_trace = []
    for pool in _clone(pools):
        tr = []
        if pool:
            tr.append(O.get_memory_cost(pool, ocfg)["cost"])
            pre = max(pool)
            new = pre // 2
            while new >= 1:
                O.move_largest_bucket(pool, pre, new)
                tr.append(O.get_memory_cost(pool, ocfg)["cost"])
                pre, new = new, new // 2
        want_trace.append(tr)
    return got, (want_cfg, want_trace)


def _clone(pools):
    return [{w: O.OracleBucket(b.bucket_width, b.num_rows, b.nnz, list(b.row_indices), set(b.col_indices))
             for w, b in pool.items()} for pool in pools]


def test_hand_example():
    g = mtx_from_rows(HAND, (6, 8))
    (cfg, trace), (wcfg, wtrace) = both(g, 2, 32)
    assert cfg == [[1, 4], [1, 2]] == wcfg
    assert trace == [[472.0, 536.0, 536.0], [336.0, 400.0]] == wtrace


def test_stale_snapshot_case():
    g = mtx_from_rows([[0, 1, 2, 3, 4, 5], [7]], (2, 8))
    (cfg, trace), (wcfg, wtrace) = both(g, 1, 32)
    assert cfg == [[4, 8]] == wcfg
    assert trace == [[272.0, 304.0, 368.0, 496.0]] == wtrace


def test_single_nonzero_partition_is_value_error():
    g = mtx_from_rows([[3]], (1, 8))
    stats, hist = stats_from_oracle(g, 1)
    with pytest.raises(ValueError, match="The partition is too small, only having 1 non-zero element."):
        search_from_statistics(stats, hist, CostModelSettings(32, 1))


def test_empty_partition():
    g = mtx_from_rows([[0, 1], [0, 2], [1, 3]], (3, 8))
    stats, hist = stats_from_oracle(g, 2)
    assert search_from_statistics(stats, hist, CostModelSettings(64, 2))[1] == []


@pytest.mark.parametrize("seed", range(12))
def test_random_matrices_bit_exact(seed):
    rng = np.random.default_rng(900 + seed)
    nr = int(rng.integers(50, 900))
    nc = int(rng.integers(50, 900))
    parts = int(rng.choice([1, 1, 2, 3, 5, 8]))
    feat = int(rng.choice([32, 64, 128, 256, 512]))
    g = skewed_matrix(rng, nr, nc, mean_deg=float(rng.choice([2, 5, 12])), heavy_rows=int(rng.integers(0, 4)),
                      values=False)
    try:
        (cfg, trace), (wcfg, wtrace) = both(g, parts, feat)
    except ValueError:
        stats, hist = stats_from_oracle(g, parts)
        with pytest.raises(ValueError):
            search_from_statistics(stats, hist, CostModelSettings(feat, parts))
        return
    assert cfg == wcfg
    assert trace == wtrace          # every visited state's cost, bit for bit


@pytest.mark.parametrize("limit", [4, 16, 64])
def test_small_width_limit_exercises_row_splitting(limit):
    rng = np.random.default_rng(limit)
    g = skewed_matrix(rng, 300, 400, mean_deg=9, heavy_rows=3, values=False)
    (cfg, trace), (wcfg, wtrace) = both(g, 2, 128, limit=limit)
    assert cfg == wcfg and trace == wtrace
    assert max(max(c) for c in cfg if c) <= limit


def test_cfg_num_parts_may_differ_from_partition_count():
    # the driver passes the same number twice, but the two are separate arguments
    # (format_algos.py:988-993 vs 45-49); a 1-partition matrix priced as if it had 4
    rng = np.random.default_rng(3)
    g = skewed_matrix(rng, 200, 200, values=False)
    (cfg, trace), (wcfg, wtrace) = both(g, 1, 64, cfg_parts=4)
    assert cfg == wcfg and trace == wtrace


def test_gfx950_model_returns_valid_config():
    rng = np.random.default_rng(5)
    g = skewed_matrix(rng, 500, 500, mean_deg=10, heavy_rows=2, values=False)
    stats, hist = stats_from_oracle(g, 1)
    cfg = search_from_statistics(stats, hist, CostModelSettings(128, 1, cost_model="gfx950"))
    assert cfg[0] == sorted(cfg[0]) and all(w & (w - 1) == 0 for w in cfg[0])
