"""Builds lib/libm26s_b1.so (HIP, gfx950) in-tree with hipcc. No GPU is needed to compile."""
from __future__ import annotations

import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "lib", "libm26s_b1.so")
SOURCES = ["csrc/b1_abi.hip", "csrc/glue_abi.hip", "csrc/probe_abi.hip", "csrc/frame_abi.hip"]
DEPENDS = ["csrc/b1_kernels.h", "csrc/b1_tile.h", "csrc/b1_layout.h", "csrc/glue_kernels.h", "../include/m26s_b1.h",
           "../include/m26c_glue.h", "../include/m26_probe.h", "../include/m26w_frame.h"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
         # packed FP32 instructions stay off on this target
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wextra"]


def hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the gfx950 library cannot be built")


def build_library(verbose: bool = False) -> str:
    """Compile unconditionally and return the library path."""
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    cmd = [hipcc(), *FLAGS, *[os.path.join(HERE, s) for s in SOURCES], "-o", LIB]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return LIB


def stale() -> bool:
    if not os.path.exists(LIB):
        return True
    built = os.path.getmtime(LIB)
    return any(os.path.getmtime(os.path.join(HERE, f)) > built for f in SOURCES + DEPENDS)
