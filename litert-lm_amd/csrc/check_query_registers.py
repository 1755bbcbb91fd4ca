#!/usr/bin/env python3
"""Build-time check of prefill_attn16_kernel's query registers.

The kernel loads its query operands with inline assembly and waits for them with its own s_waitcnt, so the
compiler does not know that those registers are pending between the load and the wait. That is only sound if the
generated code never touches them except as MFMA operands: a copy or a spill placed after the loads would read
them before the data has arrived. This script reads the device assembly (hipcc -S) and fails if, in any
instantiation of the kernel, an instruction other than an MFMA names one of those registers after the first load.

It also fails when an instantiation spills vector registers.

    check_query_registers.py prefill_attn.s
"""
import re
import sys


def registers(text):
    regs = set()
    for lo, hi in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(lo), int(hi) + 1))
    regs.update(int(r) for r in re.findall(r"\bv(\d+)\b", text))
    return regs


def main(path):
    asm = open(path).read()
    kernels = re.findall(r"^(_ZN5mi355\w*prefill_attn16_kernel\w+):", asm, re.M)
    if not kernels:
        sys.exit(f"{path}: no prefill_attn16_kernel found")
    bad = 0
    for name in kernels:
        body = re.search(r"^" + re.escape(name) + r":(.*?)\.Lfunc_end", asm, re.S | re.M).group(1).splitlines()
        query, first = set(), None
        for i, line in enumerate(body):
            m = re.search(r"\bglobal_load_dwordx4 v\[(\d+):(\d+)\], v\[\d+:\d+\], off", line)
            if m:
                query.update(range(int(m.group(1)), int(m.group(2)) + 1))
                first = i if first is None else first
        if len(query) != 64:
            print(f"{name}: expected 64 query registers, found {len(query)}")
            bad += 1
            continue
        for i, line in enumerate(body[first:], first):
            m = re.match(r"\s+([a-z_0-9]+)\s+(.*?)(;.*)?$", line)
            if not m or m.group(1).startswith("v_mfma") or m.group(1) == "global_load_dwordx4":
                continue
            if registers(m.group(2)) & query:
                print(f"{name}: line {i}: `{line.strip()}` touches a query register")
                bad += 1
    # No instantiation may spill vector registers: the loop is laid out for exactly 256 of them, and a spill is
    # scratch traffic plus a wait inside every key block (it has happened after changes that looked harmless).
    for name, count in re.findall(r"\.name:\s+(_ZN5mi355\w*prefill_attn16_kernel\w+)\s.*?\.vgpr_spill_count:\s+(\d+)", asm, re.S):
        if int(count):
            print(f"{name}: {count} vector registers spilled")
            bad += 1
    if bad:
        sys.exit(1)
    print(f"{path}: query registers of {len(kernels)} kernel instantiations are touched by MFMAs only, no vector register spills")


if __name__ == "__main__":
    main(sys.argv[1])
