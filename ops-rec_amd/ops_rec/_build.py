"""Builds the HIP library for gfx950 with hipcc (explicit, in-tree; no JIT cache)."""

from __future__ import annotations

import os
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

_PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_PKG), "csrc")
LIB_DIR = os.path.join(_PKG, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libhstu_mi355.so")

# the host side, and the kernels by input type and direction: one translation unit each, compiled side by side
SOURCES = [
    "hstu_mi355.hip",
    "ln_mul_mi355.hip",
    "in_linear_silu_mi355.hip",
    "hstu_kernels_fwd_bf16.hip",
    "hstu_kernels_fwd_f16.hip",
    "hstu_kernels_fwd_f8.hip",
    "hstu_kernels_fwd_f32.hip",
    "hstu_kernels_fwd_short.hip",
    "hstu_kernels_bwd_bf16.hip",
    "hstu_kernels_bwd_f16.hip",
]
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]  # fmt: skip


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the HIP library cannot be built")


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}): {' '.join(cmd)}\n{res.stdout}")


def build(verbose: bool = False, jobs: int | None = None, extra_flags: tuple = (), lib_path: str | None = None) -> str:
    """Compile ``csrc/*.hip`` into ``ops_rec/_lib/libhstu_mi355.so`` (always recompiles every source).
    ``extra_flags`` / ``lib_path`` build a variant elsewhere (the timeline example builds one with ``-DHSTU_TIMELINE``)."""
    target = lib_path or LIB_PATH
    os.makedirs(os.path.dirname(target), exist_ok=True)
    hipcc = hipcc_path()
    jobs = jobs or max(1, min(len(SOURCES), os.cpu_count() or 1, int(os.environ.get("MAX_JOBS", "16"))))
    with tempfile.TemporaryDirectory(prefix="hstu_build_") as obj_dir:
        objects = [os.path.join(obj_dir, os.path.splitext(s)[0] + ".o") for s in SOURCES]
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            jobs_done = [
                pool.submit(_run, [hipcc, *HIPCC_FLAGS, *extra_flags, "-c", os.path.join(CSRC, s), "-o", o], verbose)
                for s, o in zip(SOURCES, objects)
            ]
            for j in jobs_done:
                j.result()
        tmp = target + ".tmp"
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objects], verbose)
    os.replace(tmp, target)
    return target
