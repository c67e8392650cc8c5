"""Build libverl_amd.so (gfx950) from the HIP sources in this directory.

    python -m verl_amd.csrc.build        # or: python verl_amd/csrc/build.py

hipcc cross-compiles without a GPU.  The library links only the HIP runtime; it is loaded with
ctypes after ``import torch`` so that the runtime torch already mapped is the one it binds to.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libverl_amd.so")
SOURCES = ["runtime.hip", "lce.hip", "policy_math.hip", "gae.hip", "returns_scan.hip", "otb.hip", "metrics.hip", "rollout_corr.hip", "response_window.hip", "cov_select.hip", "row_softmax.hip"]
HEADERS = ["common.h", "gemm_core.h", "rowchunk.h", os.path.join("..", "..", "include", "verl_amd.h")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-mcode-object-version=5",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # the LDS-direct loads set M0 from inline assembly and say so in the clobber list
    "-Wno-inline-asm",
]


def _compile(src: str) -> str:
    obj = os.path.join(HERE, "build", os.path.splitext(src)[0] + ".o")
    os.makedirs(os.path.dirname(obj), exist_ok=True)
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    """Compile every source and link the shared library; always recompiles."""
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH) >> 10} KiB)")
    return LIB_PATH


if __name__ == "__main__":
    build()
