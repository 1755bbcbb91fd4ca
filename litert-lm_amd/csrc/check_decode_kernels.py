#!/usr/bin/env python3
"""Build-time check of the decode kernels' device assembly.

The decode kernels keep up to 128 registers of K / V buffer loads in flight while they set up the query
operands (and, in the fused step, norm and rotate the new token's rows). That is laid out for straight-line
code: a function call inside a kernel (s_swappc_b64 / s_setpc_b64 to a callee) would have to save those
registers around the call, and scratch memory (register spills, a stack) would put memory traffic and waits
into the block loop. This script reads the device assembly (hipcc -S) and fails if any instantiation of
decode_attn_kernel or decode_merge_kernel contains a call, uses scratch memory or spills registers.

It also looks for one miscompilation that this compiler has produced in these kernels: the register allocator
handing registers of a loaded V operand group (four registers, one matrix-instruction operand) to the softmax as
temporaries between the place where the fused step patches the new token's row into that group and the matrix
instruction that reads it, so that a sixteenth of the outputs came out wrong (seen when the patch wrote single
elements of the four-element vector; written as whole-vector operations it compiles correctly). The four
registers of a matrix-instruction operand are always produced together - one 16-byte load, one LDS read, four
conversions, four selects of a patch - so the check walks each kernel in program order and fails when the last
instructions that wrote the registers of an operand group are of different kinds.

    check_decode_kernels.py decode_attn.s
"""
import re
import sys


def registers(text):
    regs = set()
    for lo, hi in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(lo), int(hi) + 1))
    regs.update(int(r) for r in re.findall(r"\bv(\d+)\b", text))
    return regs


def torn_operands(body):
    """(line, operand, writers) of every matrix instruction one of whose source operand groups was last
    written, register by register, by instructions of different kinds."""
    found = []
    last = {}
    for i, line in enumerate(body.splitlines()):
        m = re.match(r"\s+([a-z_0-9]+)\s+(.*?)(;.*)?$", line)
        if not m:
            continue
        op, args = m.group(1), m.group(2)
        if op.startswith("v_mfma"):
            for lo, hi in re.findall(r"v\[(\d+):(\d+)\]", args)[1:3]:
                kinds = {last.get(r, (0, "?"))[1] for r in range(int(lo), int(hi) + 1)}
                if len(kinds) > 1:
                    found.append((i, f"v[{lo}:{hi}]", sorted(kinds)))
        writes = op.startswith(("v_", "buffer_load", "ds_read", "ds_bpermute", "global_load", "flat_load")) and not op.startswith("v_cmp")
        if writes:
            for r in registers(args.split(",")[0]):
                last[r] = (i, op)
    return found


def main(path):
    asm = open(path).read()
    names = re.findall(r"^(_ZN5mi355\w*decode_(?:attn|merge)_kernel\w+):", asm, re.M)
    if not names:
        sys.exit(f"{path}: no decode kernel found")
    bad = 0
    for name in names:
        body = re.search(r"^" + re.escape(name) + r":(.*?)\.Lfunc_end", asm, re.S | re.M).group(1)
        for op in ("s_swappc_b64", "s_call_b64", "scratch_load", "scratch_store", "buffer_store_dword v[0-9]+, off, s\\[0:3\\]"):
            hits = re.findall(r"^\s+" + op + r"\b.*$", body, re.M)
            if hits:
                print(f"{name}: {len(hits)} x `{hits[0].strip()}`")
                bad += 1
        for line, operand, kinds in torn_operands(body):
            print(f"{name}: line {line}: matrix-instruction operand {operand} last written by {kinds}: live registers reused?")
            bad += 1
    meta = re.findall(r"\.name:\s+(_ZN5mi355\w*decode_(?:attn|merge)_kernel\w+)\n(.*?)\.wavefront_size", asm, re.S)
    if len(meta) != len(names):
        print(f"{path}: {len(names)} kernels but {len(meta)} metadata records")
        bad += 1
    for name, rec in meta:
        for key in ("private_segment_fixed_size", "vgpr_spill_count", "sgpr_spill_count"):
            m = re.search(r"\." + key + r":\s+(\d+)", rec)
            if not m:
                print(f"{name}: no {key} in the metadata")
                bad += 1
            elif int(m.group(1)) and key != "sgpr_spill_count":  # (scalar registers spill into vector lanes, not memory)
                print(f"{name}: {key} = {m.group(1)}")
                bad += 1
        if re.search(r"\.uses_dynamic_stack:\s+true", rec):
            print(f"{name}: uses a dynamic stack")
            bad += 1
    if bad:
        sys.exit(1)
    print(f"{path}: {len(names)} decode kernel instantiations: no calls, no scratch memory, no vector register spills, no torn matrix operands")


if __name__ == "__main__":
    main(sys.argv[1])
