"""Check of the tile kernels' generated code around their hand-issued loads.

The k-loops of csrc/b1_tile.h issue their scale loads and LDS
reads as `asm` statements and order them with explicit s_waitcnt, because a load the compiler knows
of makes it drain the direct-to-LDS prefetch. The price: to the compiler such a register holds its
value the moment the instruction has issued. Two things must therefore hold in the generated code,
and this module checks them on the assembly hipcc emits (no GPU needed):

 1. a register with a hand-issued load in flight is not read, and
 2. it is not written: the data in flight would land on top of the new value (an address, say).

"In flight" follows the hardware's counters. Vector-memory operations (loads, stores, direct-to-LDS
loads, whoever issued them) complete in issue order, and `s_waitcnt vmcnt(N)` returns when at most N
are outstanding: the checker keeps them in a queue and retires all but the newest N at such a wait.
LDS reads retire at `lgkmcnt(0)`, the only form the kernels use. An MFMA also retires the registers
it reads: the sources place every MFMA behind the wait for its operands, and the queue model then
agrees.

Each kernel is walked in layout order, twice (loops wrap), which is conservative for the
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


VM_PREFIX = ("global_load", "global_store", "global_atomic", "buffer_", "scratch_", "flat_")
KERNELS = r"^(_ZN4m26g\w*tile_kernel\w*):"


def check(asm_text: str) -> tuple[dict, list]:
    """Returns ({kernel: hand-issued loads seen}, [problem lines])."""
    funcs, name = {}, None
    for line in asm_text.split("\n"):
        m = re.match(KERNELS, line)
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
        vm_queue, flying_lds, inasm, loads = [], set(), False, 0
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
                m = re.search(r"vmcnt\((\d+)\)", line)
                if m:
                    del vm_queue[:max(0, len(vm_queue) - int(m.group(1)))]
                if "lgkmcnt(0)" in line:
                    flying_lds.clear()
                continue
            flying = flying_lds.union(*vm_queue) if vm_queue else set(flying_lds)
            if inasm:
                if op.startswith("ds_read"):
                    flying_lds |= _regs(tok[1])
                    loads += 1
                elif op.startswith("global_load_dword") and not op.startswith("global_load_lds"):
                    vm_queue.append(_regs(tok[1]))
                    loads += 1
                elif op.startswith(VM_PREFIX):
                    vm_queue.append(set())
                elif op.startswith("v_mfma"):
                    used = set()
                    for t in tok[2:]:
                        used |= _regs(t)
                    flying_lds -= used
                    for entry in vm_queue:
                        entry -= used
                elif op.startswith(("ds_write", "v_accvgpr")):
                    srcs = set()
                    for t in tok[1:]:
                        srcs |= _regs(t)
                    if srcs & flying:
                        problems.append(f"{fn}: hand-written instruction reads a register with a load in flight: {line.strip()}")
                continue
            if op.startswith(VM_PREFIX):
                vm_queue.append(set())  # the compiler's own: it waits for them itself, but they hold a place in the order
            nodest = op.startswith(NO_DEST)
            dest = set() if nodest or len(tok) < 2 else _regs(tok[1])
            srcs = set()
            for t in tok[(1 if nodest else 2):]:
                srcs |= _regs(t)
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
