"""Measures what tests/golden/launch_shape_measurements.json holds, on a GPU:

    python tests/golden/measure_launch_shapes.py measure OUT.jsonl --workloads ppi_like,reddit_like \\
           [--feats 32,64,128,256,512] [--parts 1,2,4,8,16,32]
    python tests/golden/measure_launch_shapes.py merge OUT.jsonl SECTION

`measure` composes the hyb format of every workload for every partition count (MI355X cost
model), times the product for every feature-window count (median of 7 runs, HIP events) and
appends one JSON line per shape with the bucket statistics of that partition count and the
model's prediction at the time of the run.  `merge` folds such a file into section SECTION of
the fixture ("cases", "dense_cases", "validation_cases"), in the layout the tests read:
ms["PxW"], stats["P"], rows, cols, feat_size, b_dtype.
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


def measure(out_path, workloads, feats, parts_list):
    import torch
    from liteform_ae_amd import format_algos as fa
    from liteform_ae_amd.synthetic import make_workload
    out = open(out_path, "a")
    for name in workloads:
        wl = make_workload(name)
        g = wl.matrix
        rows, cols = wl.shape
        print(f"# {name}: {rows} x {cols}, nnz {wl.nnz}", flush=True)
        for feat in feats:
            want = torch.float32 if wl.b_dtype == "f32" else torch.bfloat16
            B = (torch.rand((cols, feat), dtype=torch.float32, device="cuda") - 0.5).to(want)
            C = torch.empty((rows, feat), dtype=torch.float32, device="cuda")
            for p in parts_list:
                try:
                    stats, _ = fa.bucket_statistics(g, p, with_columns=False)
                    cfg = fa.search_from_statistics(stats, None, fa.CostModelSettings(feat, p, cost_model="gfx950"))
                except ValueError as e:                  # a partition with a single entry
                    print(f"# skipped {name} N={feat} P={p}: {e}", flush=True)
                    continue
                fmt = fa.build_hyb_format_device(g, cfg)
                for w in fa._window_candidates(feat, wl.b_dtype):
                    plan = fa.HybSpMM(fmt, feat, wl.b_dtype, windows=w)
                    ms = float(np.median(plan.time_ms(B, C, warmup=2, repeat=7)))
                    plan.close()
                    rec = {"name": name, "feat": feat, "dt": wl.b_dtype, "P": p, "W": w, "ms": ms,
                           "pred": fa.model_spmm_ms(stats, w, rows, cols, feat, wl.b_dtype),
                           "rows": rows, "cols": cols, "nnz": wl.nnz, "stats": stats.tolist()}
                    out.write(json.dumps(rec) + "\n")
                    out.flush()
                    print(json.dumps({k: v for k, v in rec.items() if k != "stats"}), flush=True)
                del fmt
            del B, C
        del wl, g


def merge(jsonl_path, section):
    fixture = json.load(open(FIXTURE))
    cases = fixture.setdefault(section, {})
    for line in open(jsonl_path):
        r = json.loads(line)
        key = f"{r['name']}/N{r['feat']}/{r.get('dt', 'f32')}"
        c = cases.setdefault(key, {"rows": r["rows"], "cols": r["cols"], "nnz": r["nnz"], "feat_size": r["feat"],
                                   "b_dtype": r.get("dt", "f32"), "ms": {}, "stats": {}})
        c["ms"][f"{r['P']}x{r['W']}"] = round(r["ms"], 5)
        c["stats"][str(r["P"])] = r["stats"]
    json.dump(fixture, open(FIXTURE, "w"), separators=(",", ":"))
    print(f"{section}: {len(cases)} groups")


if __name__ == "__main__":
    if len(sys.argv) >= 3 and sys.argv[1] == "measure":
        opts = dict(zip(sys.argv[3::2], sys.argv[4::2]))
        measure(sys.argv[2],
                opts.get("--workloads", "ppi_like,proteins_like,reddit_like").split(","),
                [int(x) for x in opts.get("--feats", "32,64,128,256,512").split(",")],
                [int(x) for x in opts.get("--parts", "1,2,4,8,16,32").split(",")])
    elif len(sys.argv) == 4 and sys.argv[1] == "merge":
        merge(sys.argv[2], sys.argv[3])
    else:
        print(__doc__)
        sys.exit(2)
