"""Measures, on a GPU, the kernel time of every state of the width search's fold chain:

    python tests/golden/measure_fold_chains.py measure OUT.jsonl [--matrices deg9,ppi_like,...] [--feats 32,128,512]
    python tests/golden/measure_fold_chains.py merge OUT.jsonl SECTION

A state of the chain is a list of bucket widths: the initial one holds every power of two up to
the longest row's class, each further one folds the widest bucket into the next narrower width
(format_algos.py:623-648 of the reference).  `measure` composes the hyb format of one column
partition for every state, times the product in one pass (median of 7 runs, HIP events) and
writes one JSON line per state together with the degree-class statistics the MI355X fold cost
is computed from.  `merge` puts such a file into section SECTION of
tests/golden/launch_shape_measurements.json ("fold_validation": matrices the fold cost's
constants were never fitted to), in the layout of its "fold_chains" section plus the statistics.

Matrices: `degK` = 2^20-column matrices with exactly K entries in every row (uniform columns),
otherwise a name of liteform_ae_amd/synthetic.py.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
FIXTURE = os.path.join(HERE, "launch_shape_measurements.json")

UNIFORM_ROWS = {9: 1_000_000, 24: 1_000_000, 50: 600_000, 70: 400_000, 260: 150_000}
DEFAULT_MATRICES = "deg9,deg24,deg50,deg70,deg260,ppi_like,graph_400k_d120,rect_150k_600k_d200"


def uniform_degree(deg):
    from liteform_ae_amd.format_matrix_market import MTX
    from liteform_ae_amd.synthetic import csr_from_row_degrees
    rows = UNIFORM_ROWS.get(deg, 400_000)
    rng = np.random.default_rng(7000 + deg)
    indptr, indices = csr_from_row_degrees(np.full(rows, deg), 1 << 20, rng)
    data = rng.random(len(indices), dtype=np.float32)
    return MTX.from_csr(indptr, indices, (rows, 1 << 20), data=data, name=f"deg{deg}"), "f32"


def fold_chain(first):
    """Every state from the initial widths down to [1]."""
    state = list(first)
    yield list(state)
    while state[-1] > 1:
        top = state[-1]
        state = [w for w in state if w < top]
        if not state or state[-1] != top // 2:
            state.append(top // 2)
        yield list(state)


def measure(out_path, matrices, feats):
    import torch
    from liteform_ae_amd import format_algos as fa
    from liteform_ae_amd.synthetic import make_workload
    out = open(out_path, "a")
    for name in matrices:
        if name.startswith("deg"):
            g, dt = uniform_degree(int(name[3:]))
        else:
            wl = make_workload(name)
            g, dt = wl.matrix, wl.b_dtype
        rows, cols, nnz = g.num_src_nodes(), g.num_dst_nodes(), g.num_edges()
        stats, _ = fa.bucket_statistics(g, 1, with_columns=False)
        first = [1 << k for k in range(stats.shape[1]) if stats[0, k, 2] > 0]
        print(f"# {name}: {rows} x {cols}, nnz {nnz}, initial widths {first}", flush=True)
        for feat in feats:
            want = torch.float32 if dt == "f32" else torch.bfloat16
            B = (torch.rand((cols, feat), dtype=torch.float32, device="cuda") - 0.5).to(want)
            C = torch.empty((rows, feat), dtype=torch.float32, device="cuda")
            pick = fa.search_from_statistics(stats, None, fa.CostModelSettings(feat, 1, cost_model="gfx950"))[0]
            states = list(fold_chain(first))
            if pick not in states:                       # (the single-row fix-up can leave a state off this chain)
                states.append(pick)
            for state in states:
                fmt = fa.build_hyb_format_device(g, [state])
                plan = fa.HybSpMM(fmt, feat, dt, windows=1)
                ms = float(np.median(plan.time_ms(B, C, warmup=2, repeat=7)))
                plan.close()
                del fmt
                rec = {"name": name, "feat": feat, "dt": dt, "widths": state, "ms": ms, "picked": state == pick,
                       "rows": rows, "cols": cols, "nnz": nnz, "stats": stats[0].tolist()}
                out.write(json.dumps(rec) + "\n")
                out.flush()
                print(json.dumps({k: v for k, v in rec.items() if k != "stats"}), flush=True)
            del B, C
        del g


def merge(jsonl_path, section):
    fixture = json.load(open(FIXTURE))
    cases = fixture.setdefault(section, {})
    for line in open(jsonl_path):
        r = json.loads(line)
        key = f"{r['name']}/N{r['feat']}"
        c = cases.setdefault(key, {"rows": r["rows"], "cols": r["cols"], "nnz": r["nnz"], "feat_size": r["feat"],
                                   "b_dtype": r["dt"], "stats": r["stats"], "chain": []})
        c["chain"] = [s for s in c["chain"] if s["widths"] != r["widths"]]
        c["chain"].append({"widths": r["widths"], "ms": round(r["ms"], 5)})
    json.dump(fixture, open(FIXTURE, "w"), separators=(",", ":"))
    print(f"{section}: {len(cases)} chains")


if __name__ == "__main__":
    if len(sys.argv) >= 3 and sys.argv[1] == "measure":
        opts = dict(zip(sys.argv[3::2], sys.argv[4::2]))
        measure(sys.argv[2], opts.get("--matrices", DEFAULT_MATRICES).split(","),
                [int(x) for x in opts.get("--feats", "32,128,512").split(",")])
    elif len(sys.argv) == 4 and sys.argv[1] == "merge":
        merge(sys.argv[2], sys.argv[3])
    else:
        print(__doc__)
        sys.exit(2)
