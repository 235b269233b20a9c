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
                   the ratio is also the per-launch one); traffic = L2<->fabric bytes per step from
                   the rocprofv3 counter runs on file for exactly these kernel sources, else null
  format_compose   launch-shape choice, bucket-width search, slab build and kernel plan times
                   (GPU), their sum with the upload as end_to_end_ms, and the same search and
                   build through the CPU restatement on the two small workloads
  cpu_baseline     scipy CSR @ dense (the reference's own CPU product, one thread) on a
                   bounded sample of rows of the same matrix, 1 warm-up + median of 3
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


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.md")
KERNEL_SOURCES = ("lf_spmm.hip", "lf_cells.hip", "lf_spmm_device.h")


def kernel_source_id():
    """Identity of the SpMM kernel sources, joined: sha1 of each file with comments and white
    space taken out (so that rewording a comment does not disown a measurement).  What a
    counter measurement on file has to name to be reported for this build."""
    import hashlib
    import re
    ids = []
    for name in KERNEL_SOURCES:
        text = open(os.path.join(ROOT, "liteform_ae_amd", "csrc", name), "r", encoding="utf-8").read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        text = re.sub(r"\s+", "", text)
        ids.append(hashlib.sha1(text.encode("utf-8")).hexdigest()[:12])
    return "+".join(ids)


def recorded_traffic(workload, feat, parts, windows):
    """L2 <-> fabric bytes per step from the rocprofv3 counter runs summarised in
    profiles/hbm_traffic.md (FETCH_SIZE and WRITE_SIZE, calibrated on a plain copy).  A row
    counts only if it was taken with the kernel sources of this build (their ids are
    in the row); otherwise the figure is unknown and reported as null."""
    key = f"{workload}/N{feat}/P{parts}/W{windows}"
    try:
        lines = open(TRAFFIC_FILE).read().splitlines()
    except OSError:
        return None
    here = kernel_source_id()
    for line in lines:
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 4 and cells[0] == key and cells[3] == here:
            try:
                return int(cells[2].replace(",", ""))
            except ValueError:
                return None
    return None


def cpu_baseline(wl, B_host, feat, budget_s=20.0):
    """scipy CSR(f32) @ dense(f32) - the reference's own CPU product, one thread - on the first
    rows of the matrix: one warm-up and three timed runs, sized so that the four together take
    about budget_s; the median is reported."""
    import scipy.sparse as sp
    indptr, indices, data = wl.matrix.adj_tensors("csr")
    rows = wl.shape[0]
    nnz = int(indptr[-1])
    # ~3 GFLOP/s is typical for scipy's single-threaded csr_matvecs at this width
    target_nnz = int(budget_s / 4 * 3.0e9 / (2 * feat))
    if nnz <= target_nnz:
        take = rows
    else:
        take = int(np.searchsorted(indptr, target_nnz))
        take = max(1, min(rows, take))
    sub_nnz = int(indptr[take])
    A = sp.csr_matrix((np.asarray(data[:sub_nnz], dtype=np.float32), indices[:sub_nnz], indptr[:take + 1]),
                      shape=(take, wl.shape[1]))
    Bf = np.ascontiguousarray(B_host, dtype=np.float32)
    out = A @ Bf                                            # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        out = A @ Bf
        times.append(time.perf_counter() - t0)
    dt = float(np.median(times))
    res = {
        "value": round(2.0 * sub_nnz * feat / dt / 1e9, 3),
        "unit": "GFLOP/s",
        "cores": 1,
        "kind": "port",
        "sample": f"scipy csr_matrix(f32) @ dense(f32), first {take} of {rows} rows "
                  f"({sub_nnz} nnz), 1 warm-up + median of 3 runs, {dt:.2f} s each",
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


def compose_cpu_baseline(fa, make_workload, cost_model):
    """Format composition on the CPU beside the GPU, on the two workloads the CPU restatement
    finishes in seconds: the oracle's search_bucket_config (the reference's pure-Python
    algorithm: what its driver times as time_bucket) and its closed-form numpy builder, against
    search + slab build through the library on the same matrices.  Beyond these sizes the
    Python search takes minutes: not run, never extrapolated."""
    from oracle import liteform_oracle as O
    out = {}
    for name in ("cfg1", "cfg2"):
        wl = make_workload(name)
        g, parts, feat = wl.matrix, wl.num_parts or 1, wl.feat_size
        t0 = time.perf_counter()
        want = O.search_bucket_config(g, parts, O.OracleCostModelSettings(feat, parts))
        cpu_search = (time.perf_counter() - t0) * 1e3
        t0 = time.perf_counter()
        O.build_hyb_format_closed_form(g, want)
        cpu_build = (time.perf_counter() - t0) * 1e3
        cfg_obj = fa.CostModelSettings(feat, parts, cost_model="reference")
        fa.search_bucket_config(g, parts, cfg_obj)          # warm (uploads the matrix)
        t0 = time.perf_counter()
        got = fa.search_bucket_config(g, parts, cfg_obj)
        gpu_search = (time.perf_counter() - t0) * 1e3
        fa.build_hyb_format_device(g, got)
        t0 = time.perf_counter()
        fa.build_hyb_format_device(g, got)
        gpu_build = (time.perf_counter() - t0) * 1e3
        out[name] = {"nnz": wl.nnz, "num_parts": parts, "same_config": got == want,
                     "cpu_search_ms": round(cpu_search, 2), "cpu_build_ms": round(cpu_build, 2),
                     "gpu_search_ms": round(gpu_search, 3), "gpu_build_ms": round(gpu_build, 3)}
    out["note"] = ("cpu = oracle/liteform_oracle.py (pure-Python search, numpy closed-form builder), 1 core; "
                   "reference cost model on both sides; cfg3-cfg5: not run (the Python search takes minutes)")
    return out


def bench_bsr(args):
    """Block-sparse fp16 side path (bench_bsrmm's kernel): random block structure, blocks of
    --bsr-block rows and columns, the same number of matrix rows whatever the block size."""
    import torch
    from liteform_ae_amd import format_algos as fa

    feat = args.feat or 128
    bs = args.bsr_block
    mb = nb = max(8, int(round(32768 * 32 // bs * args.scale)))
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
    dev.block_size, dev.mb, dev.nb, dev.nnzb = bs, mb, nb, nnzb
    dev.indptr = torch.from_numpy(indptr).cuda()
    dev.indices = torch.from_numpy(indices).cuda()
    dev.data = (torch.rand(nnzb * bs * bs, device="cuda") - 0.5).to(torch.float16)
    dev.checked = False                       # the first product checks the index arrays on the GPU
    x = (torch.rand((nb * bs, feat), device="cuda") - 0.5).to(torch.float16)
    for _ in range(max(1, args.warmup)):
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
    flops = 2.0 * nnzb * bs * bs * feat
    blk = bs * bs * 2
    algo = nnzb * blk + nnzb * 4 + (mb + 1) * 4 + nb * bs * feat * 2 + mb * bs * feat * 2
    gath = nnzb * blk + nnzb * 4 + (mb + 1) * 4 + nnzb * bs * feat * 2 + mb * bs * feat * 2
    print(json.dumps({
        "metric": f"BSR ({bs}x{bs}, fp16) SpMM GFLOP/s", "value": round(flops / (ms * 1e-3) / 1e9, 1), "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 in, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": f"bsr: {mb * bs} x {nb * bs}, {nnzb} dense {bs}x{bs} blocks (~{per_row} per block row)",
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
                    help="column partitions (default: the workload's; chosen by --shape where it names none)")
    ap.add_argument("--windows", type=int, default=0,
                    help="feature windows per step (0 = chosen together with the partitions)")
    ap.add_argument("--shape", default="model", choices=["model", "measured"],
                    help="how an open partition / window count is chosen: the launch-shape model "
                         "(default) or by composing and timing the candidates")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the matrix (testing only)")
    ap.add_argument("--b-dtype", default="", choices=["", "f32", "bf16"], help="dtype of B (default: the workload's)")
    ap.add_argument("--cost-model", default="gfx950", choices=["reference", "gfx950"],
                    help="cost function of the bucket-width search (the reference's, or the MI355X one)")
    ap.add_argument("--widths", default="", help="bucket widths instead of the searched ones, "
                    "e.g. '1,2,4,8;1,2,4' (partitions separated by ';')")
    ap.add_argument("--bsr-block", type=int, default=32, choices=[16, 32, 64], help="--workload bsr: block size")
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
    # The matrix goes to the GPU once, outside the timed parts.  The synthetic workloads are
    # canonical CSR arrays and go up as they are (upload + structural check on the GPU).
    t0 = time.perf_counter()
    dev_csr = fa._device_csr(g)
    torch.cuda.synchronize()
    ingest_ms = (time.perf_counter() - t0) * 1e3
    ingest_path = dev_csr.path
    part_timings = None
    windows = args.windows
    shape_ms = 0.0
    shape_how = "given"
    if not parts or not windows:            # left open: partition count and feature windows
        cands = (parts,) if parts else fa.PARTITION_CANDIDATES
        wins = (windows,) if windows else None
        if args.shape == "model":
            fa.predict_launch_shape(g, feat, wl.b_dtype, candidates=cands, windows=wins)          # warm
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            (parts, windows), table = fa.predict_launch_shape(g, feat, wl.b_dtype, candidates=cands, windows=wins,
                                                              return_predictions=True)
            shape_ms = (time.perf_counter() - t0) * 1e3
            shape_how = "model"
        else:
            t0 = time.perf_counter()
            (parts, windows), table = fa.choose_launch_shape(g, feat, wl.b_dtype, candidates=cands, windows=wins,
                                                             cost_model=args.cost_model, return_timings=True)
            shape_ms = (time.perf_counter() - t0) * 1e3
            shape_how = "measured"
        part_timings = {f"P{p}xW{w}": round(t, 4) for (p, w), t in table.items()}
        print(f"[bench] launch shape ({shape_how}): {parts} partition(s) x {windows} feature window(s) "
              f"from {part_timings or 'the row-overlap rule'} ({shape_ms:.2f} ms)", file=sys.stderr, flush=True)
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
    traffic = recorded_traffic(wl.name if args.scale == 1.0 and not args.widths else "", feat, parts, windows)

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
            "launch_shape": shape_how,
            "launch_shape_candidates_ms": part_timings,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 5),
            "traffic": traffic,
            "traffic_source": "profiles/hbm_traffic.md" if traffic is not None else None,
            "kernel_source_id": kernel_source_id(),
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
            "launch_shape_ms": round(shape_ms, 3),      # choosing partitions x windows (model, or measurement)
            "ingest_ms": round(ingest_ms, 1),           # matrix to the GPU as canonical CSR (once per matrix)
            "ingest_path": {"csr": "CSR arrays uploaded and checked on the GPU (lf_csr_check)",
                            "coo": "COO triplets uploaded, sorted and merged on the GPU (lf_coo_to_csr)"}[ingest_path],
            # everything between "matrix on the host" and "first product can start"
            "end_to_end_ms": round(ingest_ms + shape_ms + search_ms + build_ms + plan_ms, 2),
            "slab_slots": fmt.total_slots(),
            "ell_rows": int(np.sum(fmt.ell_rows)),
        },
    }

    if not args.no_cpu:
        # the other way in, for comparison: the same matrix as COO triplets (what a MatrixMarket
        # file or the reference's container holds), sorted and merged on the GPU
        from liteform_ae_amd.format_matrix_market import MTX
        coo = g.coo_mtx
        g_coo = MTX.from_coo(coo.row, coo.col, coo.shape, data=coo.data)
        t0 = time.perf_counter()
        dev_coo = fa._DeviceCSR(g_coo)
        torch.cuda.synchronize()
        result["format_compose"]["coo_upload_and_csr_ms"] = round((time.perf_counter() - t0) * 1e3, 1)
        result["format_compose"]["coo_route_same_arrays"] = bool(
            dev_coo.nnz == dev_csr.nnz and torch.equal(dev_coo.indptr, dev_csr.indptr)
            and torch.equal(dev_coo.indices, dev_csr.indices) and torch.equal(dev_coo.values, dev_csr.values))
        del dev_coo, g_coo
        result["format_compose"]["cpu_baseline"] = compose_cpu_baseline(fa, make_workload, args.cost_model)
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
