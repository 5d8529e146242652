"""Compiles the HIP attention library for gfx950 with hipcc (no torch headers).

`python -m oregon_gpt_oss_patching_amd.build` or `build_library()`; the result,
libgptoss_attn.so, is placed beside this file and loaded by `_lib.py`.
"""
from __future__ import annotations

import os
import shutil
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
SOURCE = os.path.join(_HERE, "csrc", "gptoss_attn.hip")
LIBRARY = os.path.join(_HERE, "libgptoss_attn.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 VALU ops are kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results stay in ordinary vector registers unless a kernel pins an accumulator to the AGPR half
    # itself (the 64-key dK/dV kernel does, through inline assembly)
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


def build_library(verbose: bool = False) -> str:
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-o", LIBRARY, SOURCE]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{proc.stdout}\n{proc.stderr}")
    return LIBRARY


if __name__ == "__main__":
    print(build_library(verbose=True))
