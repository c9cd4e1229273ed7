#!/usr/bin/env python3
"""Build-time check of the scalar-load weight pipeline in the xor/popcount kernels.

The kernels issue `s_load_dwordxN` from inline asm and wait for it in a LATER asm statement, so that vector work on the
previous batch covers the latency.  Between the two statements the destination SGPRs hold nothing yet, which an asm
constraint cannot tell the compiler: if its register allocator copied or spilled them there (v_writelane_b32 to a VGPR
lane, s_mov_b32 to another SGPR), it would move garbage and the kernel would count wrong bits with no error.  This
script reads the device assembly the compiler produced (hipcc --save-temps) and fails the build when any instruction
reads an SGPR of a scalar load issued from inline asm before the next `s_waitcnt lgkmcnt(0)`.

A second rule of the same kind: a vector store of more than 8 bytes still reads its data registers for two cycles after
it has issued.  The compiler inserts the wait states behind the stores it emits itself, but not behind one inside an
inline-asm statement, where the next vector instruction may overwrite the data: such a store must be followed, inside
its own statement, by `s_nop 1` or more.

usage: check_sgpr_pipeline.py file.s [file.s ...]
"""
import re
import sys

LOAD = re.compile(r"^\s*s_load_dwordx(\d+)\s+s\[(\d+):(\d+)\]")
LOAD1 = re.compile(r"^\s*s_load_dword\s+s(\d+),")
WAIT0 = re.compile(r"^\s*s_waitcnt\b.*lgkmcnt\(0\)")
WAIT_ALL = re.compile(r"^\s*s_waitcnt\s+(0|0x0+)\s*$")
SREG = re.compile(r"\bs(\d+)\b")
SRANGE = re.compile(r"\bs\[(\d+):(\d+)\]")
LABEL = re.compile(r"^[.\w$]+:")
WIDE_STORE = re.compile(r"^\s*(global|buffer|flat|scratch)_store_dwordx[34]\b")
NOP = re.compile(r"^\s*s_nop\s+(\d+)")


def sregs_read(line):
    """SGPR numbers an instruction names as sources (every operand but the first)."""
    body = line.split(";")[0].strip()
    if not body or " " not in body:
        return set()
    operands = body.split(None, 1)[1]
    parts = operands.split(",")
    srcs = ",".join(parts[1:]) if len(parts) > 1 else ""
    regs = set()
    for lo, hi in SRANGE.findall(srcs):
        regs.update(range(int(lo), int(hi) + 1))
    for n in SREG.findall(SRANGE.sub("", srcs)):
        regs.add(int(n))
    return regs


def check(path):
    problems = []
    kernel = None
    in_asm = False
    in_flight = {}  # sgpr -> line number of the load
    wide_store = None  # line number of a wide store in the current asm statement that still waits for its s_nop
    for no, line in enumerate(open(path), 1):
        text = line.rstrip("\n")
        if LABEL.match(text) and not text.startswith(".L"):
            kernel = text.rstrip(":")
            in_flight.clear()
            continue
        if ";;#ASMSTART" in text:
            in_asm = True
            continue
        if ";;#ASMEND" in text:
            in_asm = False
            if wide_store is not None:
                problems.append("%s:%d: a store of more than 8 bytes in inline asm without s_nop 1 behind it (kernel %s)" % (
                    path, wide_store, kernel))
                wide_store = None
            continue
        if in_asm and wide_store is not None:
            m = NOP.match(text)
            if not (m and int(m.group(1)) >= 1):
                problems.append("%s:%d: a store of more than 8 bytes in inline asm without s_nop 1 behind it (kernel %s)" % (
                    path, wide_store, kernel))
            wide_store = None
            if m:
                continue
        if in_asm and WIDE_STORE.match(text):
            wide_store = no
            continue
        if WAIT0.match(text) or WAIT_ALL.match(text):
            in_flight.clear()
            continue
        m = LOAD.match(text)
        if m and in_asm:
            for r in range(int(m.group(2)), int(m.group(3)) + 1):
                in_flight[r] = no
            continue
        if in_flight:
            stripped = text.strip()
            if not stripped or stripped.startswith((";", ".", "//")):
                continue
            hit = sregs_read(text) & set(in_flight)
            if hit:
                problems.append("%s:%d: %s reads s%s while the scalar load of line %d is in flight (kernel %s)" % (
                    path, no, stripped.split()[0], sorted(hit), in_flight[min(hit)], kernel))
    return problems


def main():
    bad = []
    for path in sys.argv[1:]:
        bad += check(path)
    for p in bad[:40]:
        print(p, file=sys.stderr)
    if bad:
        print("check_sgpr_pipeline: %d instruction(s) touch scalar-load destinations before their wait" % len(bad), file=sys.stderr)
        return 1
    print("check_sgpr_pipeline: ok (%s)" % ", ".join(sys.argv[1:]))
    return 0


if __name__ == "__main__":
    sys.exit(main())
