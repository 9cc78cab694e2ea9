"""Static check of the gfx950 machine code in libtriton_int_hip.so for the pipeline hazards that need
software wait states and that the compiler cannot see inside inline-asm blocks.

The library's global -> LDS loads, its sub-dword int8 packing and a few waits are written as inline
assembly.  The compiler inserts the wait states ("s_nop") the hardware needs between instructions it
emits itself, but it treats an asm block as opaque text: a hazard between its own instruction and one
inside the block, or between two instructions of a block, is the source's job.  This module
disassembles the code objects of the built library (this project's own kernels) and walks every
function, following branches, looking for:

  sgpr_vmem     a VMEM instruction reads an SGPR (descriptor, scalar offset, address) fewer than 5 wait
                states after a VALU instruction (v_readfirstlane, v_cmp, carry-outs ...) wrote it: the
                access would use the register's previous contents.  The scalar offset of a buffer
                access is added after the range check, so a stale one addresses outside the buffer.
  m0_lds_dma    a buffer load to LDS follows a write of M0 by fewer than 1 wait state.
  sdwa_forward  a VALU instruction reads a VGPR that the instruction right before it wrote through a
                sub-dword destination select (needs 1 wait state).
  store_data    a VALU instruction overwrites the data registers of a buffer/global store of more than
                8 bytes issued right before it (1 wait state; applied to stores with a register in the
                scalar-offset field too).
  sgpr_lanesel  v_readlane / v_writelane use an SGPR as lane select fewer than 4 wait states after a
                VALU instruction wrote it.

A wait state is one issued instruction of the wave; "s_nop N" counts N + 1.
"""
from __future__ import annotations

import os
import re
import shutil
import subprocess
import tempfile
from dataclasses import dataclass, field

OBJDUMP = "/opt/rocm/llvm/bin/llvm-objdump"

_REG = re.compile(r"\b([sv])(\d+)\b|\b([sv])\[(\d+):(\d+)\]|\b(vcc|exec|m0)(?:_lo|_hi)?\b")
_SECOND_SDST = ("_co_", "v_div_scale", "v_mad_u64_u32", "v_mad_i64_i32")
_VMEM = ("buffer_", "tbuffer_", "global_", "flat_", "scratch_")


@dataclass
class Insn:
    mnem: str
    ops: list
    text: str
    addr: int = 0              # byte address of the instruction
    target: int | None = None  # byte address a branch jumps to


@dataclass
class Finding:
    kind: str
    function: str
    producer: str
    consumer: str
    wait_states: int

    def __str__(self):
        return f"[{self.kind}] {self.function}: `{self.producer}` -> `{self.consumer}` after {self.wait_states} wait state(s)"


def _regs(op: str) -> set:
    out = set()
    for m in _REG.finditer(op):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        elif m.group(3):
            for i in range(int(m.group(4)), int(m.group(5)) + 1):
                out.add((m.group(3), i))
        else:
            out.add(("x", m.group(6)))
    return out


def _sgprs(regs: set) -> set:
    return {r for r in regs if r[0] == "s" or r == ("x", "vcc")}


def _vgprs(regs: set) -> set:
    return {r for r in regs if r[0] == "v"}


def extract_code_objects(lib_path: str, workdir: str) -> list:
    """Copies the library into workdir and unbundles its gfx950 code objects there."""
    local = os.path.join(workdir, os.path.basename(lib_path))
    shutil.copy(lib_path, local)
    subprocess.run([OBJDUMP, "--offloading", local], check=True, capture_output=True, cwd=workdir)
    return sorted(os.path.join(workdir, f) for f in os.listdir(workdir) if f.endswith("gfx950"))


def disassemble(code_object: str) -> dict:
    """{function name: [Insn, ...]} of one code object."""
    txt = subprocess.run([OBJDUMP, "-d", code_object], check=True, capture_output=True, text=True).stdout
    funcs: dict = {}
    cur = None
    start = 0
    for line in txt.splitlines():
        m = re.match(r"^([0-9a-f]+) <([^>]+)>:\s*$", line)
        if m:
            start = int(m.group(1), 16)
            cur = funcs.setdefault(m.group(2), [])
            continue
        if cur is None or not line.startswith("\t"):
            continue
        body, _, comment = line.partition("//")
        body = body.strip()
        if not body:
            continue
        parts = body.split(None, 1)
        mnem = parts[0]
        ops = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
        a = re.match(r"\s*([0-9A-Fa-f]+):", comment)
        ins = Insn(mnem, ops, body, int(a.group(1), 16) if a else 0)
        if mnem.startswith("s_cbranch") or mnem == "s_branch":
            t = re.search(r"<[^>+]+(?:\+0x([0-9a-fA-F]+))?>", comment)
            if t:
                ins.target = start + (int(t.group(1), 16) if t.group(1) else 0)
        cur.append(ins)
    return funcs


def _valu_sgpr_writes(ins: Insn) -> set:
    if not ins.mnem.startswith("v_"):
        return set()
    w = set()
    if ins.ops:
        w |= _sgprs(_regs(ins.ops[0]))
    if len(ins.ops) > 1 and any(t in ins.mnem for t in _SECOND_SDST):
        w |= _sgprs(_regs(ins.ops[1]))
    if ins.mnem.startswith("v_cmp") and ins.mnem.endswith("_e32"):
        w.add(("x", "vcc"))
    return w


def _salu_sgpr_writes(ins: Insn) -> set:
    if ins.mnem.startswith("s_") and ins.ops and not ins.mnem.startswith(("s_cbranch", "s_branch", "s_waitcnt", "s_nop", "s_barrier", "s_cmp", "s_bitcmp")):
        return _sgprs(_regs(ins.ops[0])) | {r for r in _regs(ins.ops[0]) if r == ("x", "m0")}
    return set()


def _wait_states(ins: Insn) -> int:
    if ins.mnem == "s_nop":
        return int(ins.ops[0], 0) + 1
    return 1


def _is_vmem(ins: Insn) -> bool:
    return ins.mnem.startswith(_VMEM)


def _store_data_regs(ins: Insn) -> set:
    m = re.match(r"(buffer|global|flat|scratch)_store_dwordx([34])", ins.mnem)
    if not m:
        return set()
    idx = 1 if m.group(1) in ("global", "flat", "scratch") else 0
    return _vgprs(_regs(ins.ops[idx])) if len(ins.ops) > idx else set()


def _valu_vgpr_writes(ins: Insn) -> set:
    if ins.mnem.startswith("v_") and ins.ops and not ins.mnem.startswith(("v_cmp", "v_readfirstlane", "v_readlane", "v_nop")):
        return _vgprs(_regs(ins.ops[0]))
    return set()


def _valu_vgpr_reads(ins: Insn) -> set:
    if not ins.mnem.startswith("v_"):
        return set()
    r = set()
    for o in ins.ops[1:]:
        r |= _vgprs(_regs(o))
    if "UNUSED_PRESERVE" in ins.text and ins.ops:
        r |= _vgprs(_regs(ins.ops[0]))  # a preserved destination is also read
    return r


def lint_function(name: str, code: list) -> list:
    """Walks the function from every instruction that starts a hazard window, along fall-through and
    taken branches, for as many wait states as the longest window (5)."""
    labels = {ins.addr: i for i, ins in enumerate(code)}
    findings = []

    def walk(start: int, age: int, limit: int, check, seen: set):
        i = start
        while i < len(code) and age < limit:
            if (i, age) in seen:
                return
            seen.add((i, age))
            ins = code[i]
            stop = check(ins, age)
            if stop:
                return
            if ins.target is not None and ins.target in labels:
                walk(labels[ins.target], age + 1, limit, check, seen)
                if ins.mnem == "s_branch":
                    return
            if ins.mnem in ("s_endpgm", "s_setpc_b64"):
                return
            age += _wait_states(ins)
            i += 1

    for i, prod in enumerate(code):
        # (1) VALU-written SGPR read by VMEM (5) / used as lane select (4)
        w = _valu_sgpr_writes(prod)
        if w:
            live = set(w)

            def check(ins, age, live=live, prod=prod):
                if _is_vmem(ins):
                    used = set()
                    for o in ins.ops:
                        used |= _sgprs(_regs(o))
                    if used & live:
                        findings.append(Finding("sgpr_vmem", name, prod.text, ins.text, age))
                if ins.mnem.startswith(("v_readlane", "v_writelane")) and len(ins.ops) >= 3 and age < 4:
                    if _sgprs(_regs(ins.ops[2])) & live:
                        findings.append(Finding("sgpr_lanesel", name, prod.text, ins.text, age))
                live.difference_update(_salu_sgpr_writes(ins))  # a scalar write makes it a SALU-written register
                return not live

            walk(i + 1, 0, 5, check, set())
        # (2) M0 write -> LDS DMA (1)
        if prod.mnem.startswith("s_") and prod.ops and ("x", "m0") in _regs(prod.ops[0]) and not prod.mnem.startswith("s_cmp"):
            def check(ins, age, prod=prod):
                if ins.mnem.startswith("buffer_load") and ins.text.rstrip().endswith("lds"):
                    findings.append(Finding("m0_lds_dma", name, prod.text, ins.text, age))
                return False

            walk(i + 1, 0, 1, check, set())
        # (3) sub-dword destination write -> VALU read of the same VGPR (1)
        if prod.mnem.endswith("_sdwa") and "dst_sel:DWORD" not in prod.text and prod.ops:
            wv = _vgprs(_regs(prod.ops[0]))

            def check(ins, age, wv=wv, prod=prod):
                if _valu_vgpr_reads(ins) & wv:
                    findings.append(Finding("sdwa_forward", name, prod.text, ins.text, age))
                return False

            walk(i + 1, 0, 1, check, set())
        # (4) wide store -> VALU overwrite of its data registers (1)
        data = _store_data_regs(prod)
        if data:
            def check(ins, age, data=data, prod=prod):
                if _valu_vgpr_writes(ins) & data:
                    findings.append(Finding("store_data", name, prod.text, ins.text, age))
                return False

            walk(i + 1, 0, 1, check, set())
    return findings


def lint_library(lib_path: str) -> tuple:
    """(findings, number of functions, number of instructions) over all gfx950 code objects of the library."""
    findings, nfun, nins = [], 0, 0
    with tempfile.TemporaryDirectory() as tmp:
        for co in extract_code_objects(lib_path, tmp):
            for fname, code in disassemble(co).items():
                nfun += 1
                nins += len(code)
                findings += lint_function(fname, code)
    return findings, nfun, nins


if __name__ == "__main__":
    import sys

    here = os.path.dirname(os.path.abspath(__file__))
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(here, "..", "triton_int_amd", "lib", "libtriton_int_hip.so")
    f, nf, ni = lint_library(path)
    for x in f:
        print(x)
    print(f"{len(f)} finding(s) in {nf} functions, {ni} instructions")
