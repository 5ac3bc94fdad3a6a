"""The build-time check of the code object (cogni-ml_amd/csrc/check_hazards.py) on hand-written disassembly: it must see a
scalar register written by a vector instruction and read by a memory instruction fewer than five wait states later, and a
write of M0 directly ahead of a load to LDS; it must accept the same sequences with the wait states in place; and the
code object that is built must pass."""
import importlib.util
import os
import shutil

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("check_hazards", os.path.join(ROOT, "cogni-ml_amd", "csrc", "check_hazards.py"))
ch = importlib.util.module_from_spec(spec)
spec.loader.exec_module(ch)


def lines(text):
    return ["0000000000001000 <k>:"] + ["\t" + ln.strip() + "    // 000000001000: 00000000" for ln in text.strip().splitlines()]


def test_scalar_base_written_by_a_vector_instruction():
    bad = lines("""
        v_readfirstlane_b32 s6, v147
        v_readfirstlane_b32 s7, v146
        global_load_dwordx4 v[102:105], v134, s[6:7] offset:1024
    """)
    p = ch.check(bad)
    assert len(p) == 2 and "s[6]" in p[0] + p[1] and "s[7]" in p[0] + p[1]
    for nops, expect in (("s_nop 2", 2), ("s_nop 3", 1), ("s_nop 4", 0)):      # s_nop N is N + 1 wait states
        ok = lines("v_readfirstlane_b32 s6, v147\nv_readfirstlane_b32 s7, v146\n%s\nglobal_load_dwordx4 v[2:5], v1, s[6:7]" % nops)
        assert len(ch.check(ok)) == expect, nops
    # five other instructions do as well as five wait states of s_nop
    ok = lines("v_readfirstlane_b32 s6, v147\n" + "v_mov_b32_e32 v1, v2\n" * 5 + "global_load_dword v3, v1, s[6:7]")
    assert ch.check(ok) == []
    # a carry-out and a compare write scalar registers too; a scalar source of a vector instruction does not
    assert len(ch.check(lines("v_mad_u64_u32 v[2:3], s[8:9], s4, v2, 0\nbuffer_load_dword v1, v2, s[8:11], 0 offen"))) == 1
    assert len(ch.check(lines("v_cmp_gt_u32_e64 s[8:9], 16, v2\nbuffer_load_dword v1, v2, s[8:11], 0 offen"))) == 1
    assert ch.check(lines("v_add_u32_e32 v1, s4, v2\nglobal_load_dword v3, v1, s[4:5]")) == []
    # scalar instructions that write the base are the compiler's business and need no wait states
    assert ch.check(lines("s_add_u32 s6, s6, s10\ns_addc_u32 s7, s7, 0\nglobal_load_dword v3, v1, s[6:7]")) == []


def test_m0_ahead_of_a_load_to_lds():
    assert len(ch.check(lines("s_mov_b32 m0, s3\nglobal_load_lds_dwordx4 v[2:3], off"))) == 1
    assert ch.check(lines("s_mov_b32 m0, s3\ns_nop 0\nglobal_load_lds_dwordx4 v[2:3], off")) == []
    assert ch.check(lines("s_mov_b32 m0, s3\nglobal_load_dwordx4 v[4:7], v[2:3], off")) == []      # not a load to LDS


def test_m0_readers_in_kernels_with_asm_copies():
    """Kernels whose copies set M0 inside asm statements: every reader of M0 sits right behind a write of M0."""
    def mt(text):
        return ["0000000000001000 <q4_k_gemv_mt_f32>:"] + lines(text)[1:]
    assert ch.check(mt("s_mov_b32 m0, s3\ns_nop 0\nglobal_load_lds_dwordx4 v[2:3], off")) == []
    # a reader that relies on an older value of M0: a second copy without its own write, a movrel, a label in between
    assert len(ch.check(mt("s_mov_b32 m0, s3\ns_nop 0\nglobal_load_lds_dwordx4 v[2:3], off\nv_mov_b32_e32 v1, v2\nglobal_load_lds_dwordx4 v[4:5], off"))) == 1
    assert len(ch.check(mt("s_mov_b32 m0, s3\ns_nop 0\nv_mov_b32_e32 v1, v2\nv_mov_b32_e32 v1, v2\nv_movrels_b32_e32 v1, v2"))) == 1
    assert len(ch.check(mt("s_mov_b32 m0, s3\ns_nop 0") + ["0000000000001010 <L1>:", "\tglobal_load_lds_dwordx4 v[2:3], off    // 0: 0"])) == 1
    assert len(ch.check(mt("v_readlane_b32 s4, v1, m0"))) == 1
    # the same sequence in a kernel the compiler alone writes M0 for is its own business
    assert ch.check(lines("s_mov_b32 m0, s3\ns_nop 0\nglobal_load_lds_dwordx4 v[2:3], off\nv_mov_b32_e32 v1, v2\nv_mov_b32_e32 v1, v2\nglobal_load_lds_dwordx4 v[4:5], off")) == []


def test_registers_of_asm_loads_are_left_alone_until_their_wait():
    """Kernels whose loads are written in asm statements: nothing reads or writes a load's destination before the
    s_waitcnt vmcnt(N) that covers it (in-order retirement: all but the last N issued are done)."""
    def mt(text):
        return ["0000000000001000 <q4_k_gemv_mt_f32>:"] + lines(text)[1:]
    load = "global_load_dwordx4 v[4:7], v1, s[2:3]\n"
    assert len(ch.check(mt(load + "v_add_f32_e32 v9, v5, v8"))) == 1                       # read before any wait
    assert len(ch.check(mt(load + "v_mov_b32_e32 v6, v8"))) == 1                           # overwritten before it lands
    assert ch.check(mt(load + "s_waitcnt vmcnt(0)\nv_add_f32_e32 v9, v5, v8")) == []
    assert ch.check(mt(load + "v_add_f32_e32 v9, v10, v8\nv_mov_b32_e32 v3, v40")) == []    # other registers (v40 is not v4)
    # two more memory instructions behind it: vmcnt(2) covers it, vmcnt(3) does not; a wait without a vmcnt field does not
    two = load + "global_load_dwordx4 v[10:13], v1, s[2:3] offset:16\ns_mov_b32 m0, s9\ns_nop 0\nglobal_load_lds_dwordx4 v[20:21], off\n"
    assert ch.check(mt(two + "s_waitcnt vmcnt(2)\nv_add_f32_e32 v9, v5, v8")) == []
    assert len(ch.check(mt(two + "s_waitcnt vmcnt(3)\nv_add_f32_e32 v9, v5, v8"))) == 1
    assert len(ch.check(mt(two + "s_waitcnt lgkmcnt(0)\nv_add_f32_e32 v9, v5, v8"))) == 1
    assert len(ch.check(mt(two + "s_waitcnt vmcnt(2)\nv_add_f32_e32 v9, v11, v8"))) == 1     # the second load is still out
    # a store that takes its data from a pending register, and the code behind an unconditional branch (reached from elsewhere)
    assert len(ch.check(mt(load + "global_store_dword v1, v4, s[2:3]"))) == 1
    assert ch.check(mt(load + "s_branch 12\nv_add_f32_e32 v9, v5, v8")) == []
    # kernels the compiler writes the loads of: its own business
    assert ch.check(lines(load + "v_add_f32_e32 v9, v5, v8")) == []


def test_a_new_kernel_starts_clean():
    two = lines("v_readfirstlane_b32 s6, v147") + ["0000000000002000 <k2>:", "\tglobal_load_dword v3, v1, s[6:7]    // 0: 0"]
    assert ch.check(two) == []


def test_the_built_code_object_passes():
    objdump = "/opt/rocm/lib/llvm/bin/llvm-objdump"
    hsaco = os.path.join(ROOT, "cogni-ml_amd", "lib", "cogni_quant_gfx950.hsaco")
    if not (os.path.exists(objdump) or shutil.which("llvm-objdump")) or not os.path.exists(hsaco):
        pytest.skip("no llvm-objdump or no built code object here")
    assert ch.main(["check_hazards.py", objdump if os.path.exists(objdump) else shutil.which("llvm-objdump"), hsaco]) == 0
