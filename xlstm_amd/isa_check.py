"""Checks on the assembly listing the compiler makes of ``csrc/*.hip``, for two things it cannot know about the
hand-issued memory instructions (inline assembly) in the kernels:

1. A vector-memory instruction that reads a scalar register needs five wait states behind a VECTOR instruction that
   wrote that register (``v_readlane_b32`` reloading a spilled scalar, ``v_readfirstlane_b32``).  The compiler inserts
   them for its own instructions and does not look inside an inline-assembly statement, so the statements that take
   scalar operands start with ``s_nop 4``; ``scalar_read_hazards`` finds the ones that do not.
2. A load issued by inline assembly into a register is invisible to the compiler until the statement that waits for
   it: between the two the compiler may copy or reuse that register (a copy at a loop entry is enough), and what it
   copies is the old content.  ``inflight_register_uses`` finds compiler-generated instructions that touch such a
   register before a wait that covers the load.  (The kernels avoid the pattern where they can: loads in flight across
   a loop go straight into LDS.)

Both scan each kernel's listing in program order: exact in straight-line code, approximate across branches.
``python -m xlstm_amd.isa_check`` compiles the sources to assembly (no GPU needed) and prints what it finds.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile

from .build import HIPCC_FLAGS, ROOT, SOURCES

_VMEM = re.compile(r"^(buffer_|global_|flat_|scratch_)(load|store|atomic)")
_SCALAR_WRITERS = re.compile(r"^(v_readlane_b32|v_readfirstlane_b32|v_cmp\w*|v_add_co\w*|v_mad_u64_u32)\s+(\S+),")


def emit_assembly(out_path: str, extra_flags=()) -> str:
    """``hipcc -S`` of the device code with the flags of the product build."""
    flags = [f for f in HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [os.environ.get("HIPCC", "hipcc"), *flags, *extra_flags, "--cuda-device-only", "-S",
           "-I", os.path.join(ROOT, "include"), "-o", out_path, *SOURCES]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc -S failed ({res.returncode}):\n{res.stdout}")
    with open(out_path) as f:
        return f.read()


def _regs(text: str, kind: str) -> set:
    out = set()
    for m in re.finditer(r"\b%s\[(\d+):(\d+)\]" % kind, text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\b%s(\d+)\b" % kind, text):
        out.add(int(m.group(1)))
    return out


def _is_code(ins: str) -> bool:
    return bool(ins) and not ins.startswith(";") and not ins.startswith(".") and not ins.endswith(":")


def scalar_read_hazards(listing: str) -> list:
    """Inline-assembly statements whose vector-memory instructions read a scalar register fewer than five wait states
    behind the vector instruction that wrote it."""
    lines = listing.split("\n")
    found, kernel, i = [], None, 0
    while i < len(lines):
        line = lines[i]
        if re.match(r"^_Z\w+:", line):
            kernel = line.split(":")[0]
        if "ASMSTART" in line:
            j = i + 1
            block = []
            while "ASMEND" not in lines[j]:
                block.append(lines[j].strip())
                j += 1
            read, states = set(), 0
            for ins in block:
                if not _is_code(ins):
                    continue
                if ins.startswith("s_nop"):
                    states += int(ins.split()[1]) + 1
                    continue
                if states >= 5:
                    break
                if _VMEM.match(ins):
                    read |= _regs(ins.split(None, 1)[1] if " " in ins else "", "s")
                states += 1
            k, back = i - 1, 0
            while read and k >= 0 and back < 5:
                ins = lines[k].strip()
                k -= 1
                if not _is_code(ins) or "ASMEND" in ins or "ASMSTART" in ins:
                    continue
                if ins.startswith("s_nop"):
                    back += int(ins.split()[1]) + 1
                    continue
                back += 1
                m = _SCALAR_WRITERS.match(ins)
                if m and (_regs(m.group(2), "s") & read):
                    found.append(f"{kernel}: line {i + 1}: memory instruction in inline assembly reads "
                                 f"s{sorted(_regs(m.group(2), 's') & read)} {back} wait state(s) behind '{ins}'")
            i = j
        i += 1
    return found


def inflight_register_uses(listing: str) -> list:
    """Compiler-generated instructions that touch a vector register while a load issued by inline assembly into it has
    not been covered by a wait (``s_waitcnt vmcnt(k)`` with no more than k memory instructions issued behind the load)."""
    found, kernel, in_asm, inflight = [], None, False, []
    for i, line in enumerate(listing.split("\n")):
        ins = line.strip()
        if re.match(r"^_Z\w+:", line):
            kernel, inflight = line.split(":")[0], []
            continue
        if "ASMSTART" in ins:
            in_asm = True
            continue
        if "ASMEND" in ins:
            in_asm = False
            continue
        if not _is_code(ins):
            continue
        if not in_asm and (ins.startswith("s_branch") or ins.startswith("s_endpgm")):
            inflight = []  # (what follows in the listing is not what runs next)
            continue
        if ins.startswith("s_waitcnt"):
            m = re.search(r"vmcnt\((\d+)\)", ins)
            if m:
                inflight = [e for e in inflight if e[1] < int(m.group(1))]
            elif "cnt" not in ins.split(None, 1)[-1]:
                inflight = []  # (a wait written as a plain number covers everything)
            continue
        if not in_asm and inflight:
            used = _regs(ins.split(None, 1)[1] if " " in ins else "", "v")
            for e in inflight:
                if used & e[0]:
                    found.append(f"{kernel}: line {i + 1}: '{ins}' touches v{sorted(used & e[0])}, the destination of "
                                 f"the hand-issued load at line {e[2]} that no wait has covered yet")
        if _VMEM.match(ins):
            for e in inflight:
                e[1] += 1
            if in_asm and "_load" in ins and " lds" not in ins:
                inflight.append([_regs(ins.split(None, 1)[1].split(",")[0], "v"), 0, i + 1])
    return found


def check(listing: str) -> list:
    return scalar_read_hazards(listing) + inflight_register_uses(listing)


if __name__ == "__main__":
    with tempfile.TemporaryDirectory() as tmp:
        text = emit_assembly(os.path.join(tmp, "device.s"), tuple(sys.argv[1:]))
    problems = check(text)
    for p in problems:
        print(p)
    print(f"{len(problems)} finding(s)")
    sys.exit(1 if problems else 0)
