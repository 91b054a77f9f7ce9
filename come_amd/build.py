"""Builds ``come_amd/lib/libcome_hip.so`` from ``come_amd/csrc/*.hip`` with hipcc for gfx950.

Usage: ``python -m come_amd.build`` (cross-compiles; no GPU needed).
"""

from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcome_hip.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["abi.hip", "merge_kernels.hip", "select_kernels.hip", "attn_fwd.hip", "attn_fwd_hd.hip", "qk_prologue.hip", "suffix_kernels.hip"]

# Packed-FP32 VALU forms are switched off for all device code.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                # MFMA accumulators in ordinary VGPRs: no v_accvgpr_read/write copies around the softmax
                "-mllvm", "-amdgpu-mfma-vgpr-form=1"]
COMMON_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-Wall",
                "-Wno-unused-function"] + DEVICE_FLAGS


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(line for line in res.stdout.splitlines()
                    if "is not a recognized feature for this target" not in line)
    if res.returncode != 0:
        raise RuntimeError(f"command failed ({res.returncode}): {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out, flush=True)


def build_library(verbose: bool = True, extra_flags: list[str] | None = None) -> str:
    """Compiles every source and links the shared library; returns its path."""
    hipcc = _hipcc()
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    flags = COMMON_FLAGS + (extra_flags or [])
    objs = []
    jobs = []
    for src in SOURCES:
        obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        jobs.append([hipcc, *flags, "-c", os.path.join(CSRC, src), "-o", obj])
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        list(pool.map(lambda c: _run(c, verbose), jobs))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(verbose="-q" not in sys.argv)
    print(path)
