"""Builds the HIP libraries (gfx950) in-tree with hipcc. No GPU is needed to compile.

lib/libm26s_b1.so   the serving library: the expert FFN, the coordinator-side kernels, the frame adapter
lib/libm26_probe.so measurement aids only (what the GPU sustains on the two rooflines); the serving
                    library does not carry them, and only the benchmark and one test load them
"""
from __future__ import annotations

import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "lib", "libm26s_b1.so")
PROBE_LIB = os.path.join(HERE, "lib", "libm26_probe.so")
SOURCES = ["csrc/b1_abi.hip", "csrc/glue_abi.hip", "csrc/frame_abi.hip"]
DEPENDS = ["csrc/b1_kernels.h", "csrc/b1_tile.h", "csrc/b1_conform.h", "csrc/b1_layout.h", "csrc/glue_kernels.h",
           "../include/m26s_b1.h", "../include/m26c_glue.h", "../include/m26w_frame.h"]
PROBE_SOURCES = ["csrc/probe_abi.hip"]
PROBE_DEPENDS = ["../include/m26_probe.h"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
         # packed FP32 instructions stay off on this target
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wextra"]


def hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the gfx950 libraries cannot be built")


def _compile(sources, target: str, verbose: bool) -> str:
    os.makedirs(os.path.dirname(target), exist_ok=True)
    cmd = [hipcc(), *FLAGS, *[os.path.join(HERE, s) for s in sources], "-o", target]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return target


def build_library(verbose: bool = False) -> str:
    """Compile the serving library unconditionally, check the tile kernels' generated code around
    their hand-issued loads (a library that fails the check is removed again), return its path."""
    _compile(SOURCES, LIB, verbose)
    from . import codegen_check
    try:
        seen = codegen_check.run()
    except Exception:
        os.remove(LIB)
        raise
    if verbose:
        print(f"codegen check of the tile kernels: {seen}")
    return LIB


def build_probe(verbose: bool = False) -> str:
    return _compile(PROBE_SOURCES, PROBE_LIB, verbose)


def _older(target: str, files) -> bool:
    if not os.path.exists(target):
        return True
    built = os.path.getmtime(target)
    return any(os.path.getmtime(os.path.join(HERE, f)) > built for f in files)


def stale() -> bool:
    """True when the serving library is missing or older than one of its sources."""
    return _older(LIB, SOURCES + DEPENDS)


def probe_stale() -> bool:
    return _older(PROBE_LIB, PROBE_SOURCES + PROBE_DEPENDS)
