#!/usr/bin/env python3
"""Looks through the compiler's assembly of the device code (the .s files `make` keeps beside the objects) for registers
that a kernel reads and never writes.

Why: the register allocator of this toolchain has produced such code under heavy register pressure.  A 128-bit matrix
operand was spilled in two parts, three dwords to scratch memory and the fourth to an AGPR; the reload brought the three
dwords back and dropped the fourth, so a matrix instruction read an AGPR that no instruction of the kernel ever wrote
(whatever the previous kernel on that SIMD left there: results that were right or NaN from run to run).  The check is
flow-insensitive on purpose: it only asks, per kernel, that every VGPR / AGPR that appears as a source also appears as
a destination somewhere, which is cheap, has no false positives beyond the registers the hardware initialises (v0 - v2:
work-item ids), and catches exactly that class of miscompile.

usage: check_isa_registers.py file.s [file.s ...]   (exit status 1 and one line per finding if any)
"""
import re
import sys

REG = re.compile(r'\b([av])(\d+)\b|\b([av])\[(\d+):(\d+)\]')
# instructions without a register destination: every operand is a source
STORES = ('scratch_store', 'global_store', 'flat_store', 'buffer_store', 'ds_write', 'ds_store', 's_waitcnt', 's_nop')


def regs(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        else:
            out.update((m.group(3), i) for i in range(int(m.group(4)), int(m.group(5)) + 1))
    return out


def check(path):
    findings = []
    kernel, written, read, first_read = None, set(), set(), {}
    for ln, line in enumerate(open(path, errors='replace'), 1):
        code = line.split(';')[0].strip()
        if not code:
            continue
        if code.endswith(':') and not code.startswith('.'):
            kernel, written, read, first_read = code[:-1], set(), set(), {}
            continue
        if code.startswith('.end_amdhsa_kernel') or code.startswith('.section'):
            continue
        if kernel is None or code.startswith('.'):
            if code.startswith('.amdhsa_kernel') and kernel is not None:
                for r in sorted(read - written):
                    if r[0] == 'v' and r[1] <= 2:
                        continue   # work-item ids
                    findings.append(f"{path}: {kernel}: {r[0]}{r[1]} is read (first at line {first_read[r]}) and never written")
                kernel = None
            continue
        parts = code.split(None, 1)
        op, args = parts[0], parts[1] if len(parts) > 1 else ''
        ops = [a.strip() for a in args.split(',')]
        is_store = op.startswith(STORES)
        dst = set() if is_store else regs(ops[0]) if ops else set()
        src = regs(', '.join(ops if is_store else ops[1:]))
        for r in src:
            if r not in read:
                read.add(r)
                first_read[r] = ln
        written |= dst
    return findings


if __name__ == '__main__':
    bad = []
    for f in sys.argv[1:]:
        bad += check(f)
    for b in bad:
        print(b)
    print(f"{len(sys.argv) - 1} files, {len(bad)} registers read and never written")
    sys.exit(1 if bad else 0)
