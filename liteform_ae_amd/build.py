"""Builds liblfhip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m liteform_ae_amd.build            # compile into liteform_ae_amd/liblfhip.so

hipcc cross-compiles without a GPU.  The library links only against the HIP runtime.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblfhip.so")

SOURCES = ["lf_error.cpp", "lf_search.cpp", "lf_format.hip", "lf_spmm.hip", "lf_cells.hip", "lf_bsr.hip", "lf_ingest.hip"]

# -ffp-contract=off: the width search must add and multiply doubles exactly like CPython.
# packed-fp32-ops is switched off for device code on purpose (scalar fp32 FMAs only).
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def build(verbose: bool = True, extra_flags=(), out: str = LIB, objdir: str | None = None) -> str:
    """Compile every source and link `out`.  `extra_flags` (e.g. "-DLF_UNROLL=16") are for
    kernel-tuning builds loaded through the LITEFORM_HIP_LIB environment variable."""
    hipcc = hipcc_path()
    objdir = objdir or os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-I", os.path.join(ROOT, "include"), "-I", CSRC]
        if src.endswith(".cpp"):
            cmd += ["-x", "hip"]
        cmd += ["-c", os.path.join(CSRC, src), "-o", obj]
        _run(cmd, verbose)
        objs.append(obj)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *objs], verbose)
    return out


def _run(cmd, verbose):
    if verbose:
        print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if out.strip() and (verbose or proc.returncode):
        print(out)
    if proc.returncode:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}")


if __name__ == "__main__":
    build()
    print("built", LIB)
    sys.exit(0)
