"""The tile kernels order hand-issued loads with explicit waits; the generated code must keep every
register such a load fills away from compiler instructions until the data has landed. Checked on
the assembly (no GPU): the checker on synthetic cases of both hazards, then on what hipcc emits."""
from mimo26f_afd_amd import codegen_check

HEAD = "_ZN4m26g15fc1_tile_kernelENS_7Fc1ArgsE:\n"
TAIL = ".Lfunc_end0:\n"


def asm(*lines):
    return HEAD + "\n".join(lines) + "\n" + TAIL


def hand(instr):
    return "\t;;#ASMSTART\n\t" + instr + "\n\t;;#ASMEND"


def test_checker_flags_reads_and_writes_under_a_load_in_flight():
    load = hand("global_load_dword v7, v[2:3], off offset:256")
    mfma = hand("v_mfma_scale_f32_16x16x128_f8f6f4 a[0:3], v[10:13], v[20:27], a[0:3], v7, v8 op_sel_hi:[0,0,0] cbsz:4")
    wait = hand("s_waitcnt vmcnt(0)")
    _, p = codegen_check.check(asm(load, wait, mfma, "\tv_mov_b32_e32 v7, v1"))
    assert p == []
    _, p = codegen_check.check(asm(load, "\tv_add_u32_e32 v9, v7, v1", wait, mfma))
    assert len(p) == 1 and "reads" in p[0]
    _, p = codegen_check.check(asm(load, "\tv_lshl_add_u64 v[6:7], v[4:5], 0, s[2:3]", wait))
    assert p and "writes" in p[0]                                        # a dead load's register reused
    lds = hand("ds_read_b128 v[20:23], v30 offset:1024")
    _, p = codegen_check.check(asm(lds, "\tv_mov_b32_e32 v21, 0", hand("s_waitcnt lgkmcnt(0)")))
    assert p and "writes" in p[0]
    _, p = codegen_check.check(asm(lds, hand("s_waitcnt lgkmcnt(0)"), "\tv_mov_b32_e32 v21, 0"))
    assert p == []


def test_checker_retires_vector_memory_operations_in_issue_order():
    """`vmcnt(N)` leaves the newest N operations in flight, stores and direct-to-LDS loads included."""
    a = hand("global_load_dword v7, v[2:3], off")
    b = hand("global_load_dword v8, v[2:3], off offset:4")
    store = "\tglobal_store_dword v[2:3], v1, off"
    one = hand("s_waitcnt vmcnt(1)")
    done = hand("s_waitcnt vmcnt(0)")
    _, p = codegen_check.check(asm(a, b, one, "\tv_add_u32_e32 v9, v7, v1", done))
    assert p == []                                                       # the older load has landed
    _, p = codegen_check.check(asm(a, b, one, "\tv_add_u32_e32 v9, v8, v1", done))
    assert p and "reads" in p[0]                                         # the younger one has not
    _, p = codegen_check.check(asm(a, b, store, one, "\tv_add_u32_e32 v9, v8, v1", done))
    assert p == []                                                       # the store is the one left in flight
    lds_load = hand("global_load_lds_dwordx4 v[2:3], off")
    _, p = codegen_check.check(asm(a, lds_load, lds_load, hand("s_waitcnt vmcnt(2)"), "\tv_add_u32_e32 v9, v7, v1", done))
    assert p == []
    _, p = codegen_check.check(asm(a, lds_load, lds_load, hand("s_waitcnt vmcnt(3)"), "\tv_add_u32_e32 v9, v7, v1", done))
    assert p and "reads" in p[0]


def test_checker_keeps_everything_but_mfmas_off_a_fresh_accumulator():
    """A hand-written MFMA's result is eight passes away and the compiler does not know: an accumulator copy
    or read it places right behind one (as it does behind a loop, to hand the accumulator on in another
    register) is a hazard until sixteen wait states have passed; another MFMA on the same accumulator is not."""
    mfma = hand("v_mfma_scale_f32_16x16x128_f8f6f4 a[64:67], v[10:13], v[20:27], a[64:67], v7, v8 op_sel_hi:[0,0,0] cbsz:4")
    copy = "\tv_accvgpr_mov_b32 a60, a64"
    _, p = codegen_check.check(asm(mfma, "\ts_add_i32 s35, s35, 3", copy))
    assert len(p) == 1 and "accumulator" in p[0]
    _, p = codegen_check.check(asm(mfma, hand("s_nop 15"), copy))
    assert p == []
    _, p = codegen_check.check(asm(mfma, hand("s_nop 13"), copy))          # fourteen wait states: too few
    assert len(p) == 1
    _, p = codegen_check.check(asm(mfma, mfma, hand("s_nop 15"), "\tv_accvgpr_read_b32 v1, a65"))
    assert p == []
    _, p = codegen_check.check(asm(mfma, hand("ds_write_b128 v3, a[64:67] offset:1024")))
    assert len(p) == 1
    # behind a loop: the exit block is reached from the loop's last MFMA whatever lies between them in the file
    _, p = codegen_check.check(asm(".LBB0_1:", mfma, "\ts_cbranch_scc1 .LBB0_1", copy, "\ts_endpgm"))
    assert len(p) == 1
    _, p = codegen_check.check(asm(".LBB0_1:", mfma, hand("s_nop 15"), "\ts_cbranch_scc1 .LBB0_1", copy, "\ts_endpgm"))
    assert p == []


def test_checker_follows_the_control_flow():
    """A register in flight is judged along the paths that can reach an instruction, not along the layout:
    code that merely follows a branch in the file is not reached from it, a loop's back edge is."""
    load = hand("global_load_dword v7, v[2:3], off offset:256")
    wait = hand("s_waitcnt vmcnt(0)")
    # the load's block jumps over a neighbour in the layout that overwrites v7: not a hazard
    _, p = codegen_check.check(asm(load, "\ts_branch .LBB0_2", ".LBB0_1:", "\tv_mov_b32_e32 v7, 0", "\ts_endpgm",
                                   ".LBB0_2:", wait, "\tv_add_u32_e32 v9, v7, v1", "\ts_endpgm"))
    assert p == []
    # the same neighbour on the fall-through path of a conditional branch is one
    _, p = codegen_check.check(asm(load, "\ts_cbranch_scc1 .LBB0_2", ".LBB0_1:", "\tv_mov_b32_e32 v7, 0", "\ts_endpgm",
                                   ".LBB0_2:", wait, "\ts_endpgm"))
    assert len(p) == 1 and "writes" in p[0]
    # a load issued at the bottom of a loop body is still in flight at its top
    _, p = codegen_check.check(asm(".LBB0_1:", "\tv_add_u32_e32 v9, v7, v1", wait, load, "\ts_cbranch_scc1 .LBB0_1", "\ts_endpgm"))
    assert len(p) == 1 and "reads" in p[0]
    _, p = codegen_check.check(asm(".LBB0_1:", wait, "\tv_add_u32_e32 v9, v7, v1", load, "\ts_cbranch_scc1 .LBB0_1", wait, "\ts_endpgm"))
    assert p == []
    # two paths join: the register is in flight if it is on either, with the fewer younger operations of the two
    other = hand("global_load_dword v8, v[2:3], off")
    _, p = codegen_check.check(asm("\ts_cbranch_scc1 .LBB0_2", load, other, other, "\ts_branch .LBB0_3", ".LBB0_2:", load, other,
                                   ".LBB0_3:", hand("s_waitcnt vmcnt(2)"), "\tv_add_u32_e32 v9, v7, v1", wait, "\ts_endpgm"))
    assert len(p) == 1 and "reads" in p[0]                                # on the second path only one operation is younger
    _, p = codegen_check.check(asm("\ts_cbranch_scc1 .LBB0_2", load, other, other, "\ts_branch .LBB0_3", ".LBB0_2:", load, other,
                                   ".LBB0_3:", hand("s_waitcnt vmcnt(1)"), "\tv_add_u32_e32 v9, v7, v1", wait, "\ts_endpgm"))
    assert p == []


def test_checker_wants_wait_states_inside_an_asm_store_of_more_than_eight_bytes():
    """A store of more than eight bytes reads the upper half of its data after it issues; written as an asm
    statement it has to bring its own two wait states, inside the statement."""
    bare = ";;#ASMSTART\n\tglobal_store_dwordx4 v[0:1], v[14:17], off sc1\n\t;;#ASMEND\n\tv_mov_b32_e32 v16, 0"
    n, p = codegen_check.check_asm_stores(bare)
    assert n == 1 and len(p) == 1 and "wait states" in p[0]
    for nop, problems in (("s_nop 1", 0), ("s_nop 0", 1), ("s_nop 3", 0)):
        good = f";;#ASMSTART\n\tglobal_store_dwordx4 v[0:1], v[14:17], off sc1\n\t{nop}\n\t;;#ASMEND"
        n, p = codegen_check.check_asm_stores(good)
        assert n == 1 and len(p) == problems
    # stores the compiler emitted itself (outside asm statements) and narrow asm stores are not its business
    n, p = codegen_check.check_asm_stores("\tglobal_store_dwordx4 v[0:1], v[14:17], off\n;;#ASMSTART\n\tglobal_store_dwordx2 v[0:1], v[2:3], off sc1\n;;#ASMEND")
    assert n == 0 and p == []


def test_built_tile_kernels_pass():
    seen = codegen_check.run()
    stores = seen.pop("asm stores of more than eight bytes")
    assert stores >= 4                                                    # the per-route rows' stores of every FC2 body
    assert len(seen) == 3 and all(n >= 100 for n in seen.values())
