"""Check of the tile kernels' generated code around their hand-issued loads.

The k-loops of csrc/b1_tile.h issue their scale loads and LDS
reads as `asm` statements and order them with explicit s_waitcnt, because a load the compiler knows
of makes it drain the direct-to-LDS prefetch. The price: to the compiler such a register holds its
value the moment the instruction has issued. Two things must therefore hold in the generated code,
and this module checks them on the assembly hipcc emits (no GPU needed):

 1. a register with a hand-issued load in flight is not read, and
 2. it is not written: the data in flight would land on top of the new value (an address, say).

 3. a hand-written MFMA's accumulator is not touched by anything but another MFMA until the matrix pipe
    has written it back. The MFMAs are `asm` statements too (the accumulator must stay in place), so the
    compiler does not know that their result arrives eight passes later: a register copy it places
    right behind the last MFMA of a loop (to hand the accumulator to the code after the loop in another
    register) reads the value from before that MFMA. The sources put `s_nop` runs where such code can
    follow; the check counts wait states (one per instruction, N + 1 for `s_nop N`) between a
    hand-written MFMA and the next non-MFMA access to its destination, and wants at least 16
    (the compiler's own hazard tables hold 8 passes + 3 for this MFMA; the rest is margin).

 4. in every kernel of the library, a store of more than eight bytes written as an `asm` statement is
    followed, inside the same statement, by at least two wait states (`s_nop 1`). Such a store reads the
    upper half of its data a little after it issues; the compiler keeps the next instructions off those
    registers for the stores it emits itself, and cannot for one it does not recognise (it reused the
    registers at once, and two of four stored columns came out wrong now and then).

"In flight" follows the hardware's counters. Vector-memory operations (loads, stores, direct-to-LDS
loads, whoever issued them) complete in issue order, and `s_waitcnt vmcnt(N)` returns when at most N
are outstanding: an operation has landed behind such a wait exactly when at least N younger ones were
issued after it, so the checker keeps, per register in flight, the number of vector-memory operations
issued since its load. LDS reads retire at `lgkmcnt(0)`, the only form the kernels use. An MFMA also
retires the registers it reads: the sources place every MFMA behind the wait for its operands.

The walk follows the control flow: the kernel is cut into basic blocks at labels and branches, the state
at a block's entry is the join over its predecessors (a register is in flight if it is on any path, with
the smallest count of younger operations any path gives it), iterated to a fixed point, and every
instruction is then judged against the state that can reach it. `python -m mimo26f_afd_amd.codegen_check`
compiles and checks.
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


MFMA_WAIT_STATES = 16


def _aregs(tok: str) -> set:
    m = re.match(r"a\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"a(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def _regs(tok: str) -> set:
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


VM_PREFIX = ("global_load", "global_store", "global_atomic", "buffer_", "scratch_", "flat_")
KERNELS = r"^(_ZN4m26g\w*tile_kernel\w*):"


BRANCH = re.compile(r"^(s_branch|s_cbranch_\w+)\s+(\.L\w+)")
CAP = 64  # vmcnt holds six bits: beyond that many younger operations an entry cannot be told apart


def _blocks(body: list) -> tuple[list, dict]:
    """Basic blocks [(label or None, [(line, inasm)])] in layout order and label -> block index."""
    blocks, cur, label, inasm = [], [], None, False
    for line in body:
        text = line.strip()
        if "ASMSTART" in text:
            inasm = True
            continue
        if "ASMEND" in text:
            inasm = False
            continue
        m = re.match(r"^(\.L\w+):", text)
        if m:
            if cur or label is not None:
                blocks.append((label, cur))
            cur, label = [], m.group(1)
            continue
        if not text or text.startswith(";") or text.startswith("."):
            continue
        cur.append((text, inasm))
        if BRANCH.match(text) or text.startswith("s_endpgm"):
            blocks.append((label, cur))
            cur, label = [], None
    if cur or label is not None:
        blocks.append((label, cur))
    return blocks, {lab: i for i, (lab, _) in enumerate(blocks) if lab is not None}


def _step(state, text: str, inasm: bool, fn: str, problems):
    """One instruction on (vm: {reg: younger operations}, lds: set of regs, hot: {accumulator register: wait
    states since the hand-written MFMA that writes it}); reports into `problems` if given."""
    vm, lds, hot = state
    tok = text.replace(",", " ").split()
    op = tok[0]
    mfma = inasm and op.startswith("v_mfma")
    if hot and not mfma:
        touched = set()
        for t in tok[1:]:
            touched |= _aregs(t)
        if problems is not None and touched & set(hot):
            problems.append(f"{fn}: touches an accumulator {min(hot[r] for r in touched & set(hot))} wait states "
                            f"after the hand-written MFMA that writes it: {text}")
    states = int(tok[1]) + 1 if op == "s_nop" and len(tok) > 1 and tok[1].isdigit() else 1
    for r in list(hot):
        hot[r] += states
        if hot[r] >= MFMA_WAIT_STATES:
            del hot[r]
    if mfma:
        for r in _aregs(tok[1]):
            hot[r] = 0

    def issue(regs):
        for r in list(vm):
            vm[r] = min(CAP, vm[r] + 1)
        for r in regs:
            vm[r] = 0

    if op == "s_waitcnt":
        m = re.search(r"vmcnt\((\d+)\)", text)
        if m:
            n = int(m.group(1))
            for r in [r for r, y in vm.items() if y >= n]:
                del vm[r]
        if "lgkmcnt(0)" in text:
            lds.clear()
        return
    flying = set(vm) | lds
    if inasm:
        if op.startswith("ds_read"):
            lds.update(_regs(tok[1]))
            return "load"
        if op.startswith("global_load_dword") and not op.startswith("global_load_lds"):
            issue(_regs(tok[1]))
            return "load"
        if op.startswith(VM_PREFIX):
            issue(())
        elif op.startswith("v_mfma"):
            used = set()
            for t in tok[2:]:
                used |= _regs(t)
            lds.difference_update(used)
            for r in used:
                vm.pop(r, None)
        elif op.startswith(("ds_write", "v_accvgpr")):
            srcs = set()
            for t in tok[1:]:
                srcs |= _regs(t)
            if problems is not None and srcs & flying:
                problems.append(f"{fn}: hand-written instruction reads a register with a load in flight: {text}")
        return
    if op.startswith(VM_PREFIX):
        issue(())  # the compiler's own: it waits for them itself, but they hold a place in the order
    nodest = op.startswith(NO_DEST)
    dest = set() if nodest or len(tok) < 2 else _regs(tok[1])
    srcs = set()
    for t in tok[(1 if nodest else 2):]:
        srcs |= _regs(t)
    if problems is not None:
        if srcs & flying:
            problems.append(f"{fn}: reads a register with a hand-issued load in flight: {text}")
        if dest & flying:
            problems.append(f"{fn}: writes a register with a hand-issued load in flight: {text}")


def _join(into, other) -> bool:
    """Joins `other` into `into`; True if `into` changed."""
    changed = False
    for r, y in other[0].items():
        if r not in into[0] or y < into[0][r]:
            into[0][r] = y
            changed = True
    if not other[1] <= into[1]:
        into[1].update(other[1])
        changed = True
    for r, y in other[2].items():
        if r not in into[2] or y < into[2][r]:
            into[2][r] = y
            changed = True
    return changed


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
        blocks, index = _blocks(body)
        succ = []
        for i, (_, ins) in enumerate(blocks):
            last = ins[-1][0] if ins else ""
            m = BRANCH.match(last)
            nxt = []
            if m:
                if m.group(2) in index:
                    nxt.append(index[m.group(2)])
                if m.group(1) != "s_branch" and i + 1 < len(blocks):
                    nxt.append(i + 1)
            elif not last.startswith("s_endpgm") and i + 1 < len(blocks):
                nxt.append(i + 1)
            succ.append(nxt)
        entry = [None] * len(blocks)
        if blocks:
            entry[0] = ({}, set(), {})
        work = [0] if blocks else []
        while work:
            i = work.pop()
            state = (dict(entry[i][0]), set(entry[i][1]), dict(entry[i][2]))
            for text, inasm in blocks[i][1]:
                _step(state, text, inasm, fn, None)
            for j in succ[i]:
                if entry[j] is None:
                    entry[j] = (dict(state[0]), set(state[1]), dict(state[2]))
                    work.append(j)
                elif _join(entry[j], state):
                    work.append(j)
        loads, found = 0, []
        for i, (_, ins) in enumerate(blocks):
            if entry[i] is None:
                continue  # unreachable
            state = (dict(entry[i][0]), set(entry[i][1]), dict(entry[i][2]))
            for text, inasm in ins:
                if _step(state, text, inasm, fn, found) == "load":
                    loads += 1
        problems += list(dict.fromkeys(found))
        seen[fn] = loads
    return seen, problems


WIDE_STORE = re.compile(r"^(global|buffer|flat|scratch)_store_dwordx[34]\b")


def check_asm_stores(asm_text: str) -> tuple[int, list]:
    """Rule 4 over the whole file: (wide stores found inside asm statements, problems)."""
    found, problems, inasm, lines = 0, [], False, asm_text.splitlines()
    for n, line in enumerate(lines):
        text = line.strip()
        if "ASMSTART" in text:
            inasm = True
        elif "ASMEND" in text:
            inasm = False
        elif inasm and WIDE_STORE.match(text):
            found += 1
            nxt = lines[n + 1].strip() if n + 1 < len(lines) else ""
            m = re.match(r"s_nop\s+(\d+)", nxt)
            if not m or int(m.group(1)) < 1:
                problems.append(f"line {n + 1}: asm store of more than eight bytes without its wait states: {text}")
    return found, problems


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
    text = compile_to_asm()
    seen, problems = check(text)
    if len(seen) < 3 or min(seen.values()) < 100:
        raise RuntimeError(f"codegen check: tile kernels not found in the assembly ({seen})")
    stores, store_problems = check_asm_stores(text)
    if not stores:
        raise RuntimeError("codegen check: the asm stores of the per-route rows were not found in the assembly")
    problems += store_problems
    seen["asm stores of more than eight bytes"] = stores
    if problems:
        raise RuntimeError("codegen check failed:\n" + "\n".join(problems[:12]))
    return seen


if __name__ == "__main__":
    print(run())
    sys.exit(0)
