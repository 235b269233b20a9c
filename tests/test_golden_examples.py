"""The hand-derived known answers of tests/golden/hand_examples.json against the oracle and
the C search (CPU), and against the GPU pipeline (marked gpu)."""
import json
import os

import numpy as np
import pytest

from liteform_ae_amd.format_algos import CostModelSettings, search_from_statistics
from oracle import liteform_oracle as O

from helpers import mtx_from_rows, stats_from_oracle

CASES = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "hand_examples.json")))


def as_arrays(slabs, key):
    return [[np.asarray(b, dtype=np.int64) for b in part] for part in slabs[key]]


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_hand_example(name):
    c = CASES[name]
    g = mtx_from_rows(c["rows_to_cols"], tuple(c["shape"]))
    P, feat = c["num_parts"], c["feat_size"]
    pools = O.get_init_buckets_sequential(g, P)
    for p, want in enumerate(c["init_buckets"]):
        assert {str(w): list(b.key()[1:]) for w, b in pools[p].items()} == want
    O.modify_single_row_buckets(pools)
    for p, want in enumerate(c["fixed_buckets_in_dict_order"]):
        assert [[w, list(b.key()[1:])] for w, b in pools[p].items()] == want
    trace = O.search_cost_trace(g, P, O.OracleCostModelSettings(feat, P))
    assert [[[ws, cost] for ws, cost in part] for part in trace] == c["search_trace"]
    assert O.search_bucket_config(g, P, O.OracleCostModelSettings(feat, P)) == c["config"]
    for build in (O.build_hyb_format_sequential, O.build_hyb_format_closed_form):
        rows, cols, mask = build(g, c["config"])
        for got, key in ((rows, "rows"), (cols, "cols"), (mask, "mask")):
            want = as_arrays(c["slabs"], key)
            for p in range(P):
                for b in range(len(c["config"][p])):
                    np.testing.assert_array_equal(got[p][b], want[p][b])


@pytest.mark.parametrize("name", sorted(CASES))
def test_c_search_reproduces_hand_example(name):
    c = CASES[name]
    g = mtx_from_rows(c["rows_to_cols"], tuple(c["shape"]))
    stats, hist = stats_from_oracle(g, c["num_parts"])
    cfg, trace = search_from_statistics(stats, hist, CostModelSettings(c["feat_size"], c["num_parts"]),
                                        return_trace=True)
    assert cfg == c["config"]
    assert trace == [[cost for _, cost in part] for part in c["search_trace"]]


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_gpu_pipeline_reproduces_hand_example(name):
    import torch
    from liteform_ae_amd import format_algos as fa
    c = CASES[name]
    g = mtx_from_rows(c["rows_to_cols"], tuple(c["shape"]))
    P, feat = c["num_parts"], c["feat_size"]
    assert fa.search_bucket_config(g, P, fa.CostModelSettings(feat, P)) == c["config"]
    rows, cols, mask = fa.build_hyb_format(g, c["config"])
    for got, key in ((rows, "rows"), (cols, "cols"), (mask, "mask")):
        want = as_arrays(c["slabs"], key)
        for p in range(P):
            for b in range(len(c["config"][p])):
                assert got[p][b].shape == want[p][b].shape
                np.testing.assert_array_equal(got[p][b], want[p][b])
    # all-ones A times ones: every output element is the row's nonzero count
    x = torch.ones((c["shape"][1], feat), device="cuda")
    out = fa.spmm_hyb(fa.build_hyb_format_device(g, c["config"]), x).cpu().numpy()
    np.testing.assert_array_equal(out[:, 0], [len(r) for r in c["rows_to_cols"]])
