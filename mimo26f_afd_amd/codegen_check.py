"""Check of the tile kernels' generated code around their hand-issued loads.

The k-loop of csrc/b1_tile.h issues its scale loads and LDS reads as `asm` statements and orders them
with explicit s_waitcnt, because a load the compiler knows of makes it drain the direct-to-LDS
prefetch. The price: to the compiler such a register holds its value the moment the instruction has
issued. Two things must therefore hold in the generated code, and this module checks them on the
assembly hipcc emits (no GPU needed):

 1. a register with a hand-issued load in flight is read by nothing but an MFMA (behind the waits the
    source places), and
 2. it is not written by a compiler instruction before an MFMA has read it or a closing
    `s_waitcnt vmcnt(0)` / `lgkmcnt(0)` has passed: the data in flight would land on top of the new
    value (an address, say).

Each tile kernel is walked in layout order, twice (loops wrap), which is conservative for the
straight-line tails. `python -m mimo26f_afd_amd.codegen_check` compiles and checks.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile

from . import build

NO_DEST = ("global_load_lds", "global_store", "ds_write", "v_readfirstlane", "v_cmp", "s_", "buffer_store",
           "scratch_store", "global_atomic")


def _regs(tok: str) -> set:
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def check(asm_text: str) -> tuple[dict, list]:
    """Returns ({kernel: hand-issued loads seen}, [problem lines])."""
    funcs, name = {}, None
    for line in asm_text.split("\n"):
        m = re.match(r"^(_ZN4m26g\w*tile_kernel\w*):", line)
        if m:
            name = m.group(1)
            funcs[name] = []
            continue
        if line.startswith(".Lfunc_end"):
            name = None
        if name:
            funcs[name].append(line)
    seen, problems = {}, []
    for fn, body in funcs.items():
        flying_vm, flying_lds, inasm, loads = set(), set(), False, 0
        for line in body + body:
            if "ASMSTART" in line:
                inasm = True
                continue
            if "ASMEND" in line:
                inasm = False
                continue
            tok = line.strip().replace(",", " ").split()
            if not tok or tok[0].startswith(";") or tok[0].startswith("."):
                continue
            op = tok[0]
            if op == "s_waitcnt":
                if "vmcnt(0)" in line:
                    flying_vm.clear()
                if "lgkmcnt(0)" in line:
                    flying_lds.clear()
                continue
            if inasm:
                if op.startswith("ds_read"):
                    flying_lds |= _regs(tok[1])
                    loads += 1
                elif op == "global_load_dword":
                    flying_vm |= _regs(tok[1])
                    loads += 1
                elif op.startswith("v_mfma"):
                    for t in tok[2:]:
                        flying_vm -= _regs(t)
                        flying_lds -= _regs(t)
                continue
            nodest = op.startswith(NO_DEST)
            dest = set() if nodest or len(tok) < 2 else _regs(tok[1])
            srcs = set()
            for t in tok[(1 if nodest else 2):]:
                srcs |= _regs(t)
            flying = flying_vm | flying_lds
            if srcs & flying:
                problems.append(f"{fn}: reads a register with a hand-issued load in flight: {line.strip()}")
            if dest & flying:
                problems.append(f"{fn}: writes a register with a hand-issued load in flight: {line.strip()}")
        seen[fn] = loads // 2
    return seen, problems


def compile_to_asm() -> str:
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "b1_abi.s")
        flags = [f for f in build.FLAGS if f not in ("-fPIC", "-shared")]
        cmd = [build.hipcc(), *flags, "--cuda-device-only", "-S", os.path.join(build.HERE, build.SOURCES[0]), "-o", out]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("hipcc -S failed:\n" + proc.stderr)
        with open(out) as f:
            return f.read()


def run() -> dict:
    """Compile, check, raise on any problem; returns the per-kernel count of hand-issued loads."""
    seen, problems = check(compile_to_asm())
    if len(seen) < 2 or min(seen.values()) < 100:
        raise RuntimeError(f"codegen check: tile kernels not found in the assembly ({seen})")
    if problems:
        raise RuntimeError("codegen check failed:\n" + "\n".join(problems[:12]))
    return seen


if __name__ == "__main__":
    print(run())
    sys.exit(0)
