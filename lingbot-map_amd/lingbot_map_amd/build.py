"""Compile the HIP library for gfx950 in-tree (``_lib/liblbm_paged_attn.so``).

hipcc cross-compiles without a GPU.  The packed-FP32 VALU forms are switched off for all
device code; the host pass prints a harmless "not a recognized feature" note for that flag.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "csrc")
LIB_DIR = os.path.join(HERE, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "liblbm_paged_attn.so")
SOURCES = ["c_abi.hip", "tables_gfx950.hip", "append_gfx950.hip", "qkv_prepare_gfx950.hip", "residual_norm_gfx950.hip", "linear_gfx950.hip",
           "paged_attn_gfx950.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no NaN-quieting moves around the row-maximum chains of the attention kernel; the
    # only NaN test in the library (fp32 -> bf16 append) is done on the integer bits
    "-fno-honor-nans",
]


def build(verbose: bool = False) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [HIPCC, *FLAGS, "-o", LIB_PATH, *[os.path.join(CSRC, s) for s in SOURCES]]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
