"""Oracle, C search and GPU pipeline against vectors produced by the reference's own functions
(tests/golden/make_search_vectors.py wrote them once, where the reference checkout is
available; nothing here reads the reference).  21 seeded matrices - skewed rows, rows above
the 1024 width limit, 1 to 8 column partitions, repeated COO coordinates, a partition with a
single entry - with the reference's initial buckets, single-row fix-up, the float cost of every
state of the fold chain, the chosen widths and a digest of the hyb slabs."""
import hashlib
import json
import os

import numpy as np
import pytest

from liteform_ae_amd.format_algos import CostModelSettings, search_from_statistics
from liteform_ae_amd.format_matrix_market import MTX
from oracle import liteform_oracle as O

from helpers import stats_from_oracle

HERE = os.path.join(os.path.dirname(__file__), "golden")
VECTORS = json.load(open(os.path.join(HERE, "search_vectors.json")))["cases"]
ARRAYS = np.load(os.path.join(HERE, "search_vectors.npz"))


def matrix(name):
    c = VECTORS[name]
    rows = ARRAYS[name + "_row"].astype(np.int64)
    cols = ARRAYS[name + "_col"].astype(np.int64)
    assert len(rows) == c["coo_entries"]
    return MTX.from_coo(rows, cols, tuple(c["shape"]), name=name)


def digest(nested):
    h = hashlib.sha256()
    shapes = []
    for part in nested:
        shapes.append([list(a.shape) for a in part])
        for a in part:
            h.update(np.ascontiguousarray(a, dtype=np.int64).tobytes())
    return shapes, h.hexdigest()


def pool_rows(pool):
    return [[int(w)] + [int(x) for x in b.key()[1:]] for w, b in pool.items()]


GOOD = sorted(n for n, c in VECTORS.items() if "raises" not in c)
BAD = sorted(n for n, c in VECTORS.items() if "raises" in c)


@pytest.mark.parametrize("name", GOOD)
def test_oracle_matches_the_reference(name):
    c = VECTORS[name]
    g = matrix(name)
    P, feat = c["num_parts"], c["feat_size"]
    cfg = O.OracleCostModelSettings(feat, P)
    pools = O.get_init_buckets_sequential(g, P)
    assert [pool_rows(p) for p in pools] == c["init_buckets"]
    O.modify_single_row_buckets(pools)
    assert [pool_rows(p) for p in pools] == c["fixed_buckets_in_dict_order"]
    trace = O.search_cost_trace(g, P, cfg)
    assert [[[ws, float(cost).hex()] for ws, cost in part] for part in trace] == c["search_trace"]
    config = O.search_bucket_config(g, P, cfg)
    assert config == c["config"]
    for build in (O.build_hyb_format_sequential, O.build_hyb_format_closed_form):
        rows, cols, mask = build(g, config)
        for key, nested in (("rows", rows), ("cols", cols), ("mask", mask)):
            shapes, sha = digest(nested)
            assert shapes == c["slabs"][key]["shapes"], (build.__name__, key)
            assert sha == c["slabs"][key]["sha256"], (build.__name__, key)


@pytest.mark.parametrize("name", GOOD)
def test_c_search_matches_the_reference(name):
    c = VECTORS[name]
    g = matrix(name)
    stats, hist = stats_from_oracle(g, c["num_parts"])
    config, trace = search_from_statistics(stats, hist, CostModelSettings(c["feat_size"], c["num_parts"]),
                                           return_trace=True)
    assert config == c["config"]
    assert [[float(x).hex() for x in part] for part in trace] == [[cost for _, cost in part] for part in c["search_trace"]]


@pytest.mark.parametrize("name", BAD)
def test_single_entry_partition_raises_like_the_reference(name):
    c = VECTORS[name]
    g = matrix(name)
    kind, message = c["raises"]
    assert kind == "ValueError"
    with pytest.raises(ValueError, match="only having 1 non-zero element") as err:
        O.search_bucket_config(g, c["num_parts"], O.OracleCostModelSettings(c["feat_size"], c["num_parts"]))
    assert str(err.value) == message
    stats, hist = stats_from_oracle(g, c["num_parts"])
    with pytest.raises(ValueError) as err:
        search_from_statistics(stats, hist, CostModelSettings(c["feat_size"], c["num_parts"]))
    assert str(err.value) == message


@pytest.mark.gpu
@pytest.mark.parametrize("name", GOOD + BAD)
def test_gpu_pipeline_matches_the_reference(name):
    from liteform_ae_amd import format_algos as fa
    c = VECTORS[name]
    g = matrix(name)
    P, feat = c["num_parts"], c["feat_size"]
    if "raises" in c:
        with pytest.raises(ValueError) as err:
            fa.search_bucket_config(g, P, fa.CostModelSettings(feat, P))
        assert str(err.value) == c["raises"][1]
        return
    assert fa.search_bucket_config(g, P, fa.CostModelSettings(feat, P)) == c["config"]
    rows, cols, mask = fa.build_hyb_format(g, c["config"])
    for key, nested in (("rows", rows), ("cols", cols), ("mask", mask)):
        shapes, sha = digest(nested)
        assert shapes == c["slabs"][key]["shapes"], key
        assert sha == c["slabs"][key]["sha256"], key
