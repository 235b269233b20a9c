#!/usr/bin/env python3
"""Benchmark of the fused hyb SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3] [--feat 128] [--parts 1] [--windows 1]

A step is one SpMM  C = A_hyb . B  over the whole synthetic matrix, with A's hyb slabs, B and
C resident in HBM.  The default workload is the 2.45M-row power-law graph at N = 128, the
configuration the headline metric is quoted on.  Prints one JSON line:

  value            GFLOP/s = 2 * nnz * N / t, from the wall time of K back-to-back steps
  roofline         HBM: algorithmic bytes per step / average kernel time of a step measured
                   with HIP events on the launch stream (a step is one launch per column
                   partition and feature window; bytes and time are both summed over them, so
                   the ratio is also the per-launch one); traffic = L2<->fabric bytes per step from rocprofv3
                   counters when a measurement is on file
  format_compose   bucket-width search and slab build times (GPU), reported beside it
  cpu_baseline     scipy CSR @ dense (the reference's own CPU product, one thread) on a
                   bounded sample of rows of the same matrix
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(nnz, rows, cols, feat, b_bytes):
    """A as CSR once, B once, C once."""
    return nnz * 8 + (rows + 1) * 4 + cols * feat * b_bytes + rows * feat * 4


def gather_bytes(nnz, rows, feat, b_bytes):
    """The same with one B row fetched per nonzero (no reuse of B)."""
    return nnz * 8 + (rows + 1) * 4 + nnz * feat * b_bytes + rows * feat * 4


# L2 <-> fabric bytes per step (all launches of a step; /W2 = two feature windows) from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE, FETCH_SIZE scaled by 2.000 as calibrated on a 1 GiB copy in the same runs;
# source: profiles/spmm_partition_kernel.cfg3_N128.md
MEASURED_TRAFFIC = {
    "cfg3/N128/P1": 44157630417,
    "cfg3/N128/P2": 46512630501,
    "cfg3/N128/P3": 48665180588,
    "cfg3/N128/P1/W2": 45234112102,
    "cfg3/N128/P2/W2": 47336937882,
}


def recorded_traffic(workload, feat, parts, windows):
    return MEASURED_TRAFFIC.get(f"{workload}/N{feat}/P{parts}" + (f"/W{windows}" if windows > 1 else ""))


def cpu_baseline(wl, B_host, feat, budget_s=20.0):
    """scipy CSR(f32) @ dense(f32) on the first rows of the matrix, sized to ~budget_s."""
    import scipy.sparse as sp
    indptr, indices, data = wl.matrix.adj_tensors("csr")
    rows = wl.shape[0]
    nnz = int(indptr[-1])
    # ~1 GFLOP/s is typical for scipy's single-threaded csr_matvecs at this width
    target_nnz = int(budget_s * 1.0e9 / (2 * feat))
    if nnz <= target_nnz:
        take = rows
    else:
        take = int(np.searchsorted(indptr, target_nnz))
        take = max(1, min(rows, take))
    sub_nnz = int(indptr[take])
    A = sp.csr_matrix((np.asarray(data[:sub_nnz], dtype=np.float32), indices[:sub_nnz], indptr[:take + 1]),
                      shape=(take, wl.shape[1]))
    Bf = np.ascontiguousarray(B_host, dtype=np.float32)
    t0 = time.perf_counter()
    out = A @ Bf
    dt = time.perf_counter() - t0
    res = {
        "value": round(2.0 * sub_nnz * feat / dt / 1e9, 3),
        "unit": "GFLOP/s",
        "cores": 1,
        "kind": "port",
        "sample": f"scipy csr_matrix(f32) @ dense(f32), first {take} of {rows} rows "
                  f"({sub_nnz} nnz), 1 run, {dt:.2f} s",
    }
    # the same sample through torch's threaded CPU CSR product, as a multi-core figure
    try:
        import warnings
        import torch
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            At = torch.sparse_csr_tensor(torch.from_numpy(np.asarray(A.indptr, dtype=np.int64)),
                                         torch.from_numpy(np.asarray(A.indices, dtype=np.int64)),
                                         torch.from_numpy(A.data), size=A.shape)
        Bt = torch.from_numpy(Bf)
        At @ Bt                                             # warm-up (thread pool, first touch)
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            At @ Bt
            times.append(time.perf_counter() - t0)
        res["threaded"] = {"value": round(2.0 * sub_nnz * feat / float(np.median(times)) / 1e9, 3),
                           "unit": "GFLOP/s", "cores": int(torch.get_num_threads()),
                           "host_cpus": os.cpu_count(),
                           "sample": "torch.sparse_csr_tensor(f32) @ dense(f32), same rows, median of 3"}
    except Exception as exc:                                # a baseline only: report, do not fail the bench
        res["threaded"] = {"value": None, "error": f"{type(exc).__name__}: {exc}"}
    return res, out, take


def bench_bsr(args):
    """Block-sparse fp16 side path (bench_bsrmm's kernel): random 32 x 32 block structure."""
    import scipy.sparse as sp
    import torch
    from liteform_ae_amd import format_algos as fa

    feat = args.feat or 128
    mb = nb = max(8, int(round(32768 * args.scale)))
    per_row = 8
    rng = np.random.default_rng(1006)
    cols = np.sort(rng.integers(0, nb, size=(mb, per_row)), axis=1)
    keep = np.ones_like(cols, dtype=bool)
    keep[:, 1:] = cols[:, 1:] != cols[:, :-1]
    indptr = np.zeros(mb + 1, dtype=np.int32)
    indptr[1:] = np.cumsum(keep.sum(1))
    indices = cols[keep].astype(np.int32)
    nnzb = len(indices)
    dev = fa._DeviceBSR.__new__(fa._DeviceBSR)
    dev.block_size, dev.mb, dev.nb, dev.nnzb = 32, mb, nb, nnzb
    dev.indptr = torch.from_numpy(indptr).cuda()
    dev.indices = torch.from_numpy(indices).cuda()
    dev.data = (torch.rand(nnzb * 1024, device="cuda") - 0.5).to(torch.float16)
    x = (torch.rand((nb * 32, feat), device="cuda") - 0.5).to(torch.float16)
    for _ in range(args.warmup):
        fa.spmm_bsr(dev, x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y = fa.spmm_bsr(dev, x)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    ev = []
    for _ in range(args.steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fa.spmm_bsr(dev, x)
        b.record()
        b.synchronize()
        ev.append(a.elapsed_time(b))
    kernel_ms = float(np.mean(ev))
    flops = 2.0 * nnzb * 1024 * feat
    algo = nnzb * 2048 + nnzb * 4 + (mb + 1) * 4 + nb * 32 * feat * 2 + mb * 32 * feat * 2
    gath = nnzb * 2048 + nnzb * 4 + (mb + 1) * 4 + nnzb * 32 * feat * 2 + mb * 32 * feat * 2
    print(json.dumps({
        "metric": "BSR (32x32, fp16) SpMM GFLOP/s", "value": round(flops / (ms * 1e-3) / 1e9, 1), "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 in, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": f"bsr: {mb * 32} x {nb * 32}, {nnzb} dense 32x32 blocks (~{per_row} per block row)",
                   "feat_size": feat},
        "roofline": {"bound": "hbm", "achieved": round(algo / (kernel_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(algo / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": None, "kernel_ms": round(kernel_ms, 4), "algorithmic_bytes": algo,
                     "gather_bytes": gath, "gather_GBps": round(gath / (kernel_ms * 1e-3) / 1e9, 1),
                     "mfma_TFLOPs": round(flops / (kernel_ms * 1e-3) / 1e12, 1)},
    }))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg3")
    ap.add_argument("--feat", type=int, default=0, help="dense columns N (default: the workload's)")
    ap.add_argument("--parts", type=int, default=0,
                    help="column partitions (default: the workload's; measured choice where it names none)")
    ap.add_argument("--windows", type=int, default=0,
                    help="feature windows per step (0 = by measurement together with the partitions)")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the matrix (testing only)")
    ap.add_argument("--b-dtype", default="", choices=["", "f32", "bf16"], help="dtype of B (default: the workload's)")
    ap.add_argument("--cost-model", default="gfx950", choices=["reference", "gfx950"],
                    help="cost function of the bucket-width search (the reference's, or the MI355X one)")
    ap.add_argument("--widths", default="", help="bucket widths instead of the searched ones, "
                    "e.g. '1,2,4,8;1,2,4' (partitions separated by ';')")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy, so a counter run reads a known size")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from liteform_ae_amd import _lib
    from liteform_ae_amd import format_algos as fa
    from liteform_ae_amd.synthetic import make_dense, make_workload

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    _lib.load()
    torch.cuda.set_device(0)
    if args.workload == "bsr":
        return bench_bsr(args)

    t0 = time.perf_counter()
    wl = make_workload(args.workload, args.scale)
    if args.b_dtype:
        wl.b_dtype = args.b_dtype
    feat = args.feat or wl.feat_size
    parts = args.parts or wl.num_parts
    g = wl.matrix
    rows, cols = wl.shape
    nnz = wl.nnz
    t_gen = time.perf_counter() - t0
    print(f"[bench] {wl.name}: {rows} x {cols}, nnz {nnz}, N {feat}, P {parts or 'auto'}, B {wl.b_dtype} "
          f"(generated in {t_gen:.1f} s)", file=sys.stderr, flush=True)

    B_host = make_dense(cols, feat, wl.seed)
    if wl.b_dtype == "bf16":
        B_dev = torch.from_numpy(B_host).cuda().to(torch.bfloat16)
        B_host = B_dev.to(torch.float32).cpu().numpy()      # what the kernel really reads
        b_bytes = 2
    else:
        B_dev = torch.from_numpy(B_host).cuda()
        b_bytes = 4
    C_dev = torch.empty((rows, feat), dtype=torch.float32, device="cuda")

    # ---- format composition (GPU): search = what the reference times as time_bucket
    t0 = time.perf_counter()
    fa._device_csr(g)                       # COO upload + canonical CSR on the GPU, once, outside the timed parts
    torch.cuda.synchronize()
    ingest_ms = (time.perf_counter() - t0) * 1e3
    part_timings = None
    windows = args.windows
    if not parts or not windows:            # left open: partition count and feature windows by measurement
        t0 = time.perf_counter()
        (parts, windows), shape_timings = fa.choose_launch_shape(
            g, feat, wl.b_dtype, candidates=(parts,) if parts else (1, 2, 3, 4),
            windows=(windows,) if windows else None, cost_model=args.cost_model, return_timings=True)
        part_timings = {f"P{p}xW{w}": round(t, 4) for (p, w), t in shape_timings.items()}
        print(f"[bench] launch shape chosen by measurement: {parts} partition(s) x {windows} feature window(s) "
              f"from {part_timings} ({time.perf_counter() - t0:.2f} s)", file=sys.stderr, flush=True)
    cfg_obj = fa.CostModelSettings(feat, parts, cost_model=args.cost_model)
    fa.search_bucket_config(g, parts, cfg_obj)            # warm
    t0 = time.perf_counter()
    config = fa.search_bucket_config(g, parts, cfg_obj)
    search_ms = (time.perf_counter() - t0) * 1e3
    if args.widths:
        config = [[int(w) for w in part.split(",") if w] for part in args.widths.split(";")]
        if len(config) == 1 and parts > 1:
            config = config * parts
    fa.build_hyb_format_device(g, config)                 # warm
    t0 = time.perf_counter()
    fmt = fa.build_hyb_format_device(g, config)
    build_ms = (time.perf_counter() - t0) * 1e3
    fa.HybSpMM(fmt, feat, wl.b_dtype, windows=windows).close()     # warm
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    plan = fa.HybSpMM(fmt, feat, wl.b_dtype, windows=windows)
    torch.cuda.synchronize()
    plan_ms = (time.perf_counter() - t0) * 1e3
    print(f"[bench] config {config}; search {search_ms:.2f} ms, build {build_ms:.2f} ms, "
          f"kernel plan {plan_ms:.2f} ms; plan {plan.info}",
          file=sys.stderr, flush=True)

    # ---- timed region: K steps, inputs resident, synchronize on both sides
    for _ in range(args.warmup):
        plan.run(B_dev, C_dev)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        plan.run(B_dev, C_dev)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3

    # per-step kernel time from HIP events on the launch stream (warm caches, then flushed)
    ev_ms = plan.time_ms(B_dev, C_dev, warmup=0, repeat=args.steps)
    flush = torch.empty(int(512e6), dtype=torch.int8, device="cuda")
    ev_cold_ms = plan.time_ms(B_dev, C_dev, warmup=0, repeat=max(3, args.steps // 3), flush=flush)
    del flush
    kernel_ms = float(np.mean(ev_ms))

    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")      # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    flops = 2.0 * nnz * feat
    algo = algorithmic_bytes(nnz, rows, cols, feat, b_bytes)
    gath = gather_bytes(nnz, rows, feat, b_bytes)
    achieved = algo / (kernel_ms * 1e-3) / 1e9
    traffic = recorded_traffic(wl.name if args.scale == 1.0 else "", feat, parts, windows)

    result = {
        "metric": "SpMM GFLOP/s & % HBM roofline at N=128; format-compose ms",
        "value": round(flops / (ms_per_step * 1e-3) / 1e9, 2),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if wl.b_dtype == "f32" else "bf16 B, f32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": f"{wl.name}: {wl.description}" + ("" if args.scale == 1.0 else f" (scale {args.scale})"),
            "rows": rows, "cols": cols, "nnz": nnz, "feat_size": feat, "num_parts": parts, "feature_windows": windows,
            "bucket_widths": config, "cost_model": args.cost_model,
            "launch_shape_candidates_ms": part_timings,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 5),
            "traffic": traffic,
            "launches_per_step": parts * windows,
            "kernel_ms": round(kernel_ms, 4),
            "kernel_ms_median": round(float(np.median(ev_ms)), 4),
            "kernel_ms_min": round(float(np.min(ev_ms)), 4),
            "kernel_ms_cold": round(float(np.mean(ev_cold_ms)), 4),
            "algorithmic_bytes": algo,
            "gather_bytes": gath,
            "gather_GBps": round(gath / (kernel_ms * 1e-3) / 1e9, 1),
        },
        "format_compose": {
            "search_ms": round(search_ms, 3),
            "build_ms": round(build_ms, 3),
            "total_ms": round(search_ms + build_ms, 3),
            "kernel_plan_ms": round(plan_ms, 3),        # tile tables of the fused kernel (the reference: TVM build)
            "coo_upload_and_csr_ms": round(ingest_ms, 1),
            "slab_slots": fmt.total_slots(),
            "ell_rows": int(np.sum(fmt.ell_rows)),
        },
    }

    if not args.no_cpu:
        base, ref_rows, take = cpu_baseline(wl, B_host, feat, args.cpu_seconds)
        base["host_cpus"] = os.cpu_count()
        result["cpu_baseline"] = base
        # the same rows from the GPU, against the 1e-5 * sum|a||b| bound
        from oracle import liteform_oracle as O
        indptr, indices, data = g.adj_tensors("csr")
        sub = int(indptr[take])
        bound = O.spmm_abs_bound(indptr[:take + 1], indices[:sub], data[:sub], (take, cols), B_host)
        gpu_rows = C_dev[:take].cpu().numpy()
        exact = O.spmm_csr_f64(indptr[:take + 1], indices[:sub], np.asarray(data[:sub], dtype=np.float32),
                               (take, cols), B_host)
        excess = float((np.abs(gpu_rows - exact) - 1e-5 * bound).max())
        result["parity"] = {"rows_checked": take, "within_1e-5_bound": bool(excess <= 0),
                            "max_abs_err": float(np.abs(gpu_rows - exact).max())}
    plan.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
