#!/usr/bin/env python3
"""Writes tests/golden/search_vectors.{json,npz}: inputs and outputs of the reference's own
format-selection functions on seeded matrices.

Runs only where the reference checkout is present (here: /root/reference; pass another path as
the first argument); the tests read the two files it writes and never the reference.  The
reference's module cannot be imported as it stands - it pulls in tvm / SparseTIR, dgl and ogb at
import time and uses numpy.str - so those modules are replaced by inert placeholders before the
import.  None of the functions called below touches them: they are pure Python over numpy, scipy
and bisect (playground_pipline/format_algos.py:226-385, 623-648, 709-816, 819-954, 988-1166).

Per case the files hold: the matrix (COO triplets, npz), the partition count and feature size,
and what the reference computes - the initial buckets, the buckets after the single-row
fix-up in dict order, the cost of every state of the fold chain (as float hex strings), the
chosen widths, and shapes plus a SHA-256 of the hyb slabs.
"""
import copy
import hashlib
import json
import os
import sys
import types

import numpy as np
import scipy.sparse as sp

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"


class _Placeholder(types.ModuleType):
    """Stands in for a module the reference imports but the functions used here never call:
    any attribute is another placeholder, calling one returns its single callable argument
    (so it works as a decorator) or another placeholder."""

    def __getattr__(self, name):
        if name.startswith("__"):
            raise AttributeError(name)
        return _Placeholder(f"{self.__name__}.{name}")

    def __call__(self, *args, **kwargs):
        if len(args) == 1 and callable(args[0]) and not kwargs and not isinstance(args[0], _Placeholder):
            return args[0]
        return _Placeholder(f"{self.__name__}()")

    def __getitem__(self, item):
        return _Placeholder(f"{self.__name__}[]")


def import_reference():
    for name in ("tvm", "tvm.testing", "tvm.tir", "tvm.script", "tvm.sparse", "tvm.runtime",
                 "sparsetir_artifact", "dgl", "dgl.data", "ogb", "ogb.nodeproppred"):
        sys.modules.setdefault(name, _Placeholder(name))
    if not hasattr(np, "str"):
        np.str = str                       # format_algos.py:50 annotates with np.str
    sys.path.insert(0, os.path.join(REFERENCE, "playground_pipline"))
    import format_algos as FA              # noqa: E402
    import format_matrix_market as FM      # noqa: E402
    return FA, FM


def skewed(rng, nr, nc, mean_deg, heavy, heavy_len, dup=0):
    deg = np.clip(np.rint(rng.lognormal(np.log(mean_deg), 1.1, size=nr)), 0, nc).astype(np.int64)
    for _ in range(heavy):
        deg[rng.integers(nr)] = min(nc, heavy_len)
    rows = np.repeat(np.arange(nr), deg)
    cols = rng.integers(0, nc, size=len(rows))
    key = np.unique(rows * nc + cols)
    rows, cols = key // nc, key % nc
    if dup:                                # repeated coordinates: degrees count them, the CSR merges them
        pick = rng.integers(0, len(rows), size=dup)
        rows = np.concatenate([rows, rows[pick]])
        cols = np.concatenate([cols, cols[pick]])
    order = rng.permutation(len(rows))     # unsorted triplets, like a file
    return rows[order].astype(np.int32), cols[order].astype(np.int32)


CASES = [
    # name, seed, rows, cols, mean degree, heavy rows, heavy length, duplicates, partitions, feature size
    ("skew_p1_a", 1, 600, 900, 5, 2, 700, 0, 1, 32),
    ("skew_p1_b", 2, 1500, 1500, 9, 3, 1400, 0, 1, 128),
    ("skew_p1_wide", 3, 400, 6000, 12, 2, 5000, 0, 1, 64),      # rows above the 1024 width limit
    ("skew_p2_a", 4, 800, 1200, 6, 2, 900, 0, 2, 32),
    ("skew_p2_b", 5, 2500, 2500, 7, 4, 2400, 0, 2, 128),
    ("skew_p2_wide", 6, 500, 8000, 10, 3, 7000, 0, 2, 256),
    ("skew_p4_a", 7, 1000, 2000, 8, 2, 1500, 0, 4, 64),
    ("skew_p4_b", 8, 3000, 3000, 11, 5, 2900, 0, 4, 128),
    ("skew_p4_wide", 9, 300, 12000, 20, 2, 11000, 0, 4, 512),
    ("skew_p8_a", 10, 1200, 4000, 9, 3, 3500, 0, 8, 32),
    ("skew_p8_b", 11, 2000, 2000, 14, 4, 1900, 0, 8, 128),
    ("skew_p8_wide", 12, 350, 16000, 30, 2, 15000, 0, 8, 256),
    ("dense_rows_p1", 13, 200, 3000, 3, 12, 2800, 0, 1, 128),   # many rows in the widest bucket
    ("dense_rows_p3", 14, 200, 3000, 3, 12, 2800, 0, 3, 64),
    ("sparse_p1", 15, 4000, 4000, 1.5, 1, 300, 0, 1, 32),       # mostly 1-2 entries: width-1 paths
    ("sparse_p2", 16, 4000, 4000, 1.5, 1, 300, 0, 2, 128),
    ("dups_p1", 17, 700, 700, 6, 2, 600, 400, 1, 64),
    ("dups_p2", 18, 900, 1100, 7, 2, 900, 600, 2, 128),
    ("tiny_p1", 19, 12, 40, 4, 1, 30, 0, 1, 32),
    ("tiny_p2", 20, 16, 64, 5, 1, 50, 0, 2, 32),
    # the second column partition holds a single entry: the reference raises ValueError (920-921)
    ("one_entry_partition", 21, 30, 40, 3, 0, 0, 0, 2, 32),
]


def bucket_rows(pool):
    return [[int(w), int(b.num_rows), int(b.nnz), len(b.row_indices), len(b.col_indices)] for w, b in pool.items()]


def digest(nested):
    h = hashlib.sha256()
    shapes = []
    for part in nested:
        shapes.append([list(a.shape) for a in part])
        for a in part:
            h.update(np.ascontiguousarray(a, dtype=np.int64).tobytes())
    return shapes, h.hexdigest()


def main():
    FA, FM = import_reference()
    arrays, out = {}, {}
    for name, seed, nr, nc, mean_deg, heavy, heavy_len, dup, parts, feat in CASES:
        rng = np.random.default_rng(seed)
        rows, cols = skewed(rng, nr, nc, mean_deg, heavy, heavy_len, dup)
        if name == "one_entry_partition":
            keep = cols < nc // 2
            rows, cols = np.append(rows[keep], 7).astype(np.int32), np.append(cols[keep], nc - 3).astype(np.int32)
        arrays[name + "_row"], arrays[name + "_col"] = rows.astype(np.uint16), cols.astype(np.uint16)
        g = FM.MTX(None)                                   # format_matrix_market.py:44-46
        g.name = name
        g.coo_mtx = sp.coo_matrix((np.ones(len(rows)), (rows, cols)), shape=(nr, nc))
        cfg = FA.CostModelSettings(feat_size=feat, num_parts=parts)
        case = {"shape": [nr, nc], "num_parts": parts, "feat_size": feat, "coo_entries": int(len(rows))}
        try:
            pools = FA.get_init_buckets(g, parts)
            case["init_buckets"] = [bucket_rows(p) for p in pools]
            FA.modify_single_row_buckets(pools)
            case["fixed_buckets_in_dict_order"] = [bucket_rows(p) for p in pools]
            trace = []
            for pool in copy.deepcopy(pools):              # the loop of modify_bucket_widths (709-774), state by state
                tr = []
                if pool:
                    tr.append([sorted(int(w) for w in pool), float(FA.get_memory_cost(pool, cfg)["cost"]).hex()])
                    pre = max(pool.keys())
                    new = pre // 2
                    while new >= 1:
                        FA.move_largest_bucket(pool, pre, new)
                        tr.append([sorted(int(w) for w in pool), float(FA.get_memory_cost(pool, cfg)["cost"]).hex()])
                        pre, new = new, new // 2
                trace.append(tr)
            case["search_trace"] = trace
            config = FA.search_bucket_config(g, parts, cfg)          # the reference's own end-to-end answer
            case["config"] = [[int(w) for w in ws] for ws in config]
            hyb_rows, hyb_cols, hyb_mask = FA.build_hyb_format(g, config)
            case["slabs"] = {}
            for key, nested in (("rows", hyb_rows), ("cols", hyb_cols), ("mask", hyb_mask)):
                shapes, sha = digest(nested)
                case["slabs"][key] = {"shapes": shapes, "sha256": sha}
        except ValueError as exc:                            # format_algos.py:920-921
            case["raises"] = ["ValueError", str(exc)]
        out[name] = case
        print(name, case.get("config", case.get("raises")))
    np.savez_compressed(os.path.join(HERE, "search_vectors.npz"), **arrays)
    with open(os.path.join(HERE, "search_vectors.json"), "w") as f:
        json.dump({"comment": "written by make_search_vectors.py from the reference's functions; costs are float.hex()",
                   "cases": out}, f, indent=1)


if __name__ == "__main__":
    main()
