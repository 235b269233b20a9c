"""End-to-end flow of the reference's driver for matrices that use the CELL (hyb) format.

Mirrors the CELL branch of ``playground_pipline/proc05.spmm.end-to-end.py:127-190`` and its
result table (proc05.spmm.end-to-end.py:273-286): for every matrix and every feature size
the column-partition count is chosen, the bucket-width search is timed (``time_bucket(s)``),
the hyb format is composed and the fused kernel is timed (``time_exe_our(ms)``).

Differences: the reference predicts the format (CELL or BCSR) and the partition count with
RandomForest models, of which the partition model is not distributed.  Here the format is
CELL unless ``select_format`` says otherwise (the BSR and CSR branches of the reference's
driver, proc05.spmm.end-to-end.py:191-261, run through ``bench_bsrmm`` / ``bench_naive``), and
the partition count comes, together with the number of feature windows, from the launch-shape
model (``predict_launch_shape``), or is given.  ``num_parts_override`` stands where the
reference's driver overrides its predictor by matrix name (proc05.spmm.end-to-end.py:145-148).
Extra columns report GFLOP/s, feature windows and compose time.

    python -m liteform_ae_amd.driver --synthetic cfg2 --feat 32 64 128
    python -m liteform_ae_amd.driver --dataset path/to/matrix.mtx
"""
from __future__ import annotations

import argparse
import math
import sys
import time

import numpy as np
import scipy.sparse as sp

from .format_matrix_market import MTX

FEAT_SIZES = (32, 64, 128, 256, 512)        # proc05.spmm.end-to-end.py:141
# the partition counts the reference's driver sets by hand, whatever its predictor says
# (proc05.spmm.end-to-end.py:145-148)
REFERENCE_NUM_PARTS_OVERRIDE = {"ppi": 16, "proteins": 32}


def _run_block_or_csr(g, fa, feat, fmt_name):
    """The reference's branch for matrices its selector sends away from CELL
    (proc05.spmm.end-to-end.py:191-261): pad to a multiple of 32 and run the fp16 BSR kernel;
    if that fails, or when CSR is asked for, run the row-parallel CSR kernel."""
    import torch
    bsize = 32                                                         # proc05:205
    num_src, num_dst = g.num_src_nodes(), g.num_dst_nodes()
    side = -(-max(num_src, num_dst) // bsize) * bsize                  # proc05:198-210
    if fmt_name == "BSR":
        try:
            bsr_weight = g.tobsr_with_padding(shape=(side, side), blocksize=(bsize, bsize))
            x = torch.rand(bsr_weight.shape[1], feat).half()           # proc05:221
            return "BSR", fa.bench_bsrmm(bsr_weight, x, block_size=bsize)
        except Exception as e:                                         # proc05:232-234
            print(e, file=sys.stderr)
            print(f"name {g.name} in BSR failed. Do CSR then.")
    try:
        x = torch.rand((num_dst, feat))                                # proc05:239
        y_ndarray = g.dot(x.numpy())
        return "CSR", fa.bench_naive(g, x, y_ndarray, feat_size=feat, coarsening_factor=2)
    except Exception as e2:                                            # proc05:254-261
        print(e2, file=sys.stderr)
        return "CRASHED", 0


def run_end_to_end(matrices, feat_sizes=FEAT_SIZES, num_parts=None, cost_model="reference",
                   check_correctness=False, out_csv=None, keep_values=False, select_format=None,
                   num_parts_override=None):
    """Runs the flow for an iterable of MTX objects and returns a pandas DataFrame with the
    reference's columns.  ``num_parts``: None = from the launch-shape model per (matrix, feature size); an int;
    or a callable ``(g, feat_size) -> int``.  ``num_parts_override``: a mapping from matrix name
    to a partition count that replaces whatever ``num_parts`` gave for that matrix, as the
    reference's driver does for two of its graphs (``REFERENCE_NUM_PARTS_OVERRIDE``; such a
    matrix runs in one feature window).  ``select_format``: None = CELL for every
    matrix; or a callable ``g -> "CELL" | "BSR" | "CSR"`` standing in for the reference's
    format-selection model (proc05.spmm.end-to-end.py:133)."""
    import pandas as pd
    import torch

    from . import format_algos as fa

    table = {k: [] for k in ("name", "format", "feat_size", "num_parts", "time_select(s)",
                             "time_num_parts(s)", "time_bucket(s)", "time_exe_our(ms)",
                             "time_compose(ms)", "GFLOP/s", "feature_windows", "bucket_config")}
    for g in matrices:
        print(f"\nGo to name {g.name} ...")
        fa._device_csr(g)          # the matrix goes to the GPU when it is loaded, before any timed step
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fmt_name = select_format(g) if select_format else "CELL"
        time_select = time.perf_counter() - t0
        if fmt_name != "CELL":
            for feat in feat_sizes:
                ran_as, exe_time = _run_block_or_csr(g, fa, feat, fmt_name)
                row = {"name": g.name, "format": ran_as, "feat_size": feat, "num_parts": 0,
                       "time_select(s)": time_select, "time_num_parts(s)": 0, "time_bucket(s)": 0,
                       "time_exe_our(ms)": exe_time, "time_compose(ms)": float("nan"),
                       "GFLOP/s": 2.0 * g.num_edges() * feat / (exe_time * 1e-3) / 1e9 if exe_time > 0 else 0.0,
                       "feature_windows": 1, "bucket_config": ""}
                for k, v in row.items():
                    table[k].append(v)
            continue
        for feat in feat_sizes:
            t0 = time.perf_counter()
            if num_parts is None:
                parts, windows = fa.predict_launch_shape(g, feat)
            elif callable(num_parts):
                parts, windows = int(num_parts(g, feat)), 1
            else:
                parts, windows = int(num_parts), 1
            if num_parts_override and g.name in num_parts_override:    # proc05:145-148
                parts, windows = int(num_parts_override[g.name]), 1
            time_parts = time.perf_counter() - t0
            print(f"name: {g.name} num_parts: {parts} feature_windows: {windows} time(s): {time_parts}")

            print("Configuring ...", flush=True)
            t0 = time.perf_counter()                                   # proc05:153-157
            cfg = fa.CostModelSettings(feat_size=feat, num_parts=parts, cost_model=cost_model)
            bucket_config = fa.search_bucket_config(g, parts, cfg)
            time_bucket = time.perf_counter() - t0

            x = torch.ones((g.num_dst_nodes(), feat))                  # proc05:162
            y_ndarray = None
            if check_correctness:
                # the expected product has to use the values the format is composed with: the
                # matrix's own, or ones (the reference's matrices hold nothing else,
                # format_matrix_market.py:63-64)
                if keep_values:
                    y_ndarray = g.dot(x.numpy())
                else:
                    indptr, indices, _ = g.adj_tensors("csr")
                    ones = sp.csr_matrix((np.ones(len(indices), dtype=np.float32), indices, indptr), shape=(g.num_src_nodes(), g.num_dst_nodes()))
                    y_ndarray = ones.dot(x.numpy())
            compose_ms = float("nan")
            try:
                if keep_values:
                    hyb = fa.build_hyb_format_device(g, bucket_config)
                else:
                    hyb = fa.build_hyb_format_device(g, bucket_config, with_values=False)
                compose_ms = hyb.compose_ms
                exe_time = fa.bench_hyb_with_config(g, x, y_ndarray, feat_size=feat, bucket_widths=bucket_config,
                                                    bucketing_format=hyb, coarsening_factor=2,
                                                    num_col_parts=parts, use_implicit_unroll=True,
                                                    check_correctness=check_correctness,
                                                    feature_windows=windows)
                print(f"[{g.name}] {fmt_name} N={feat} partitions={parts} windows={windows} widths={bucket_config} "
                      f"search={time_bucket * 1e3:.3f} ms compose={compose_ms:.3f} ms kernel={exe_time:.4f} ms", flush=True)
            except Exception as e:                                     # proc05:178-180
                exe_time = math.inf
                print(e, file=sys.stderr)
            table["name"].append(g.name)
            table["format"].append(fmt_name)
            table["feat_size"].append(feat)
            table["num_parts"].append(parts)
            table["feature_windows"].append(windows)
            table["time_select(s)"].append(time_select)
            table["time_num_parts(s)"].append(time_parts)
            table["time_bucket(s)"].append(time_bucket)
            table["time_exe_our(ms)"].append(exe_time)
            table["time_compose(ms)"].append(compose_ms)
            table["GFLOP/s"].append(2.0 * g.num_edges() * feat / (exe_time * 1e-3) / 1e9 if exe_time > 0 else 0.0)
            table["bucket_config"].append(str(bucket_config))
    df = pd.DataFrame(data=table)
    print(df.to_string())
    if out_csv:
        df.to_csv(out_csv, index=False)
    return df


def main(argv=None):
    ap = argparse.ArgumentParser("CELL-format SpMM end to end")
    ap.add_argument("--dataset", "-d", nargs="*", default=[], help="MatrixMarket (.mtx) files")
    ap.add_argument("--synthetic", nargs="*", default=[], help="synthetic workloads: cfg1 .. cfg5")
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--feat", type=int, nargs="*", default=list(FEAT_SIZES))
    ap.add_argument("--num-parts", type=int, default=0,
                    help="column partitions for every matrix (0 = from the launch-shape model)")
    ap.add_argument("--reference-overrides", action="store_true",
                    help="partition counts the reference's driver sets by matrix name (ppi: 16, proteins: 32)")
    ap.add_argument("--cost-model", default="reference", choices=["reference", "gfx950"])
    ap.add_argument("--format", default="CELL", choices=["CELL", "BSR", "CSR"],
                    help="format to run every matrix in (the reference chooses it with a model)")
    ap.add_argument("--check", action="store_true", help="compare with scipy (rtol 1e-4) as the reference can")
    ap.add_argument("--csv", default="", help="write the table to this file")
    args = ap.parse_args(argv)
    mats = [MTX(path) for path in args.dataset]
    if args.synthetic:
        from .synthetic import make_workload
        for name in args.synthetic:
            wl = make_workload(name, args.scale)
            indptr, indices, _ = wl.matrix.adj_tensors("csr")   # the reference's matrices are unweighted
            mats.append(MTX.from_csr(indptr, indices, wl.shape, name=wl.matrix.name))
    if not mats:
        ap.print_help(sys.stderr)
        return 2
    run_end_to_end(mats, feat_sizes=args.feat, num_parts=args.num_parts or None, cost_model=args.cost_model,
                   check_correctness=args.check, out_csv=args.csv or None,
                   select_format=(lambda g: args.format) if args.format != "CELL" else None,
                   num_parts_override=REFERENCE_NUM_PARTS_OVERRIDE if args.reference_overrides else None)
    return 0


if __name__ == "__main__":
    sys.exit(main())
