#!/usr/bin/env python3
"""Build-time check of the gfx950 code object for rules that the compiler keeps for the code it emits itself but cannot
keep for instructions written inside asm statements:

  * a vector instruction that writes a scalar register (v_readfirstlane_b32, v_readlane_b32, a compare with a scalar
    destination, a carry-out) must be five wait states ahead of a memory instruction that reads that register as its
    scalar base;
  * a write of M0 must be one wait state ahead of a global load that writes to LDS;
  * in the kernels whose copies to LDS set M0 inside asm statements (names with "_mt_"), the compiler does not know
    that M0 changes, so nothing may read a value of M0 that it assumes to have survived: every instruction that reads
    M0 must have a write of M0 within the two instructions in front of it, with no label in between.

  * in the same kernels the loads into registers are written in asm statements too, so the compiler takes their
    destinations for valid from the load on and does not know about the counted s_waitcnt vmcnt(N) that makes them
    so: no instruction may read or write such a register between its load and the wait that covers it (vector memory
    instructions retire in order: after vmcnt(N) all but the last N issued are done). Followed along the fall-through
    path only: behind an unconditional branch nothing is taken to be pending.

An instruction is one wait state, "s_nop N" is N + 1. The scan is linear over each kernel of the disassembly (this
library's own code object, made by llvm-objdump); labels do not reset it, so a sequence that is only adjacent in the
file, not in execution, can be reported too: better that than the reverse.

usage: check_hazards.py <llvm-objdump> <code object>       exit status 1 and a report when a rule is broken
"""
import re
import subprocess
import sys

VALU_SGPR_TO_VMEM = 5
M0_TO_LDS_DMA = 1
M0_WRITE_WITHIN = 2
# instructions that read M0 without naming it
M0_IMPLICIT = ("s_movrel", "v_movrel", "s_set_gpr_idx", "s_sendmsg", "ds_gws", "v_interp", "ds_read_addtid", "ds_write_addtid")


def reads_m0(mnemonic, operands):
    if "_lds_" in mnemonic or (is_vmem(mnemonic) and operands and operands[-1].strip().endswith("lds")):
        return True
    if mnemonic.startswith(M0_IMPLICIT):
        return True
    return any(o.strip() == "m0" for o in operands[1:])


def asm_m0_kernel(name):
    return "_mt_" in name
# vector instructions whose second operand is a scalar destination (carry or scale flag)
SDST_SECOND = ("v_mad_u64_u32", "v_mad_i64_i32", "v_add_co_u32", "v_sub_co_u32", "v_subrev_co_u32", "v_addc_co_u32",
               "v_subb_co_u32", "v_subbrev_co_u32", "v_div_scale_f32", "v_div_scale_f64")
SREG = re.compile(r"^s(\d+)$|^s\[(\d+):(\d+)\]$")


def sregs(operand):
    """The scalar registers an operand names, as a set of numbers."""
    m = SREG.match(operand.strip())
    if not m:
        return set()
    if m.group(1) is not None:
        return {int(m.group(1))}
    return set(range(int(m.group(2)), int(m.group(3)) + 1))


def written_sgprs(mnemonic, operands):
    if not mnemonic.startswith("v_") or not operands:
        return set()
    out = set(sregs(operands[0]))
    if mnemonic.startswith(SDST_SECOND) and len(operands) > 1:
        out |= sregs(operands[1])
    return out


def is_vmem(mnemonic):
    return mnemonic.startswith(("global_", "buffer_", "flat_", "scratch_"))


def vmem_scalar_base(mnemonic, operands):
    """Scalar registers a memory instruction reads: every scalar operand it has (base pair, resource, offset)."""
    out = set()
    for op in operands:
        out |= sregs(op.split(" ")[0])
    return out


VREG = re.compile(r"(?<![a-z0-9_])v(\d+)(?![0-9\[])|(?<![a-z0-9_])v\[(\d+):(\d+)\]")


def vregs(text):
    """The vector registers a piece of operand text names."""
    out = set()
    for m in VREG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out |= set(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def waited_vmcnt(operands_text):
    """N of an s_waitcnt that has a vmcnt field, else None."""
    m = re.search(r"vmcnt\((\d+)\)", operands_text)
    return int(m.group(1)) if m else None


def check(lines):
    problems = []
    kernel = "?"
    vm_issued = 0    # vector memory instructions issued so far in this kernel
    pending = []     # (issue number, destination vgprs, text) of loads into registers not yet covered by a wait
    recent = []      # (wait states since, written sgprs, text) of recent vector-writes-scalar instructions
    m0_age = None    # wait states since the last write of m0
    m0_dist = None   # instructions since the last write of m0 in this basic block
    for raw in lines:
        line = raw.split("//")[0].strip()
        if not line:
            continue
        lab = re.match(r"^[0-9a-f]+ <([^>]+)>:$", line)
        if lab:
            if not lab.group(1).startswith("L"):
                kernel = lab.group(1)
                recent, m0_age = [], None
                vm_issued, pending = 0, []
            m0_dist = None
            continue
        if line.endswith(":") or line.startswith((".", "Disassembly", "/")) or "file format" in line:
            continue
        parts = line.split(None, 1)
        mnemonic = parts[0]
        operands = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
        if asm_m0_kernel(kernel):
            if mnemonic == "s_waitcnt":
                n = waited_vmcnt(parts[1] if len(parts) > 1 else "")
                if n is not None:
                    pending = [p for p in pending if p[0] > vm_issued - n]
            elif pending:
                touched = vregs(parts[1]) if len(parts) > 1 else set()
                for num, regs, text in pending:
                    if touched & regs:
                        problems.append("%s: '%s' touches v%s, loaded by '%s' %d vector memory instruction(s) ago and not waited for" % (
                            kernel, line, sorted(touched & regs)[:4], text, vm_issued - num))
                        break
            if mnemonic in ("s_branch", "s_endpgm", "s_setpc_b64"):
                pending = []   # what follows is reached from elsewhere, not by falling through
            if is_vmem(mnemonic):
                vm_issued += 1
                to_lds = "_lds_" in mnemonic or (operands and operands[-1].strip().endswith("lds"))
                if "_load_" in mnemonic and not to_lds and operands:
                    pending.append((vm_issued, vregs(operands[0]), line))
        if is_vmem(mnemonic):
            used = vmem_scalar_base(mnemonic, operands)
            for age, regs, text in recent:
                if age < VALU_SGPR_TO_VMEM and used & regs:
                    problems.append("%s: '%s' reads s%s %d wait state(s) after '%s' (needs %d)" % (
                        kernel, line, sorted(used & regs), age, text, VALU_SGPR_TO_VMEM))
            if "_lds_" in mnemonic and m0_age is not None and m0_age < M0_TO_LDS_DMA:
                problems.append("%s: '%s' %d wait state(s) after a write of m0 (needs %d)" % (kernel, line, m0_age, M0_TO_LDS_DMA))
        if asm_m0_kernel(kernel) and reads_m0(mnemonic, operands) and (m0_dist is None or m0_dist > M0_WRITE_WITHIN):
            problems.append("%s: '%s' reads m0 %s" % (kernel, line, "with no write of m0 in its basic block" if m0_dist is None else
                                                      "%d instructions after the last write of m0 (at most %d)" % (m0_dist, M0_WRITE_WITHIN)))
        if m0_dist is not None:
            m0_dist += 1
        states = 1
        if mnemonic == "s_nop" and operands:
            states = int(operands[0], 0) + 1
        recent = [(age + states, regs, text) for age, regs, text in recent if age + states < 8]
        if m0_age is not None:
            m0_age += states
        w = written_sgprs(mnemonic, operands)
        if w:
            recent.append((0, w, line))
        if mnemonic.startswith("s_") and operands and operands[0] == "m0":
            m0_age = 0
            m0_dist = 0
    return problems


def main(argv):
    if len(argv) != 3:
        print(__doc__)
        return 2
    dis = subprocess.run([argv[1], "-d", "--no-show-raw-insn", argv[2]], check=True, capture_output=True, text=True).stdout
    problems = check(dis.splitlines())
    n = dis.count("\n")
    if problems:
        print("check_hazards: %d problem(s) in %s" % (len(problems), argv[2]))
        for p in problems[:40]:
            print("  " + p)
        return 1
    print("check_hazards: %s clean (%d lines of disassembly)" % (argv[2], n))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
