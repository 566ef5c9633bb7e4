#!/usr/bin/env python3
"""List the MFMA loops of the kernels in a gfx950 assembly listing and the forward branches inside them.

The K-step schedule of the GEMM kernels is fixed by hand between scheduling barriers; a branch that the compiler puts
inside the K loop (for instance around a group of conditional scalar updates) cuts a K step's schedule in two and costs
a few percent without changing any instruction count.  Expected: no forward branch in the main loop of the plain SGEMM
kernels (the first loop listed for each), exactly one in the ABFT kernels (the flush of the FP32 checksum partials).

    hipcc -O3 -std=c++17 --offload-arch=gfx950 -I../../include -I. -Xclang -target-feature -Xclang -packed-fp32-ops \\
          -S --cuda-device-only sgemm.hip -o /tmp/sgemm.s && python3 check_mfma_loops.py /tmp/sgemm.s [--strict]

With --strict the exit status is 1 when a plain SGEMM kernel's main loop holds a forward branch or an ABFT kernel's
main loop holds more than one (`make check-loops` runs it over all four kernel translation units).
"""
import re
import sys


def loops_of(lines):
    label_at = {}
    for i, line in enumerate(lines):
        m = re.match(r"^(\.LBB\d+_\d+):", line)
        if m:
            label_at[m.group(1)] = i
    out = []
    for i, line in enumerate(lines):
        m = re.search(r"s_c?branch\w* (\.LBB\d+_\d+)", line)
        if not (m and m.group(1) in label_at and label_at[m.group(1)] < i):
            continue  # not a backward branch
        head = label_at[m.group(1)]
        body = lines[head:i]
        mfma = sum("v_mfma" in x for x in body)
        if not mfma:
            continue
        forward = 0
        for x in body:
            b = re.search(r"s_cbranch\w* (\.LBB\d+_\d+)", x)
            if b and b.group(1) in label_at and head < label_at[b.group(1)] <= i:
                forward += 1
        out.append((mfma, forward))
    return out


def main():
    args = [a for a in sys.argv[1:] if not a.startswith("--")]
    strict = "--strict" in sys.argv[1:]
    if len(args) != 1:
        print(__doc__)
        return 2
    text = open(args[0]).read()
    bad = 0
    for name in re.findall(r"^(_ZN6hpcdnn\d+sgemm\w*kernelI\w+):", text, re.M):
        start = text.index("\n" + name + ":")
        lines = text[start:text.index(".end_amdhsa_kernel", start)].split("\n")
        loops = loops_of(lines)
        # template arguments after the tile and wave layout: EDGE flag, then FT (0 plain, 1 or 2 ABFT)
        m = re.match(r"_ZN6hpcdnn12sgemm_kernelILi\d+ELi\d+ELi\d+ELi\d+ELb[01]ELi(\d)E", name)
        allowed = None if m is None else (0 if m.group(1) == "0" else 1)
        flag = ""
        if allowed is not None and loops and loops[0][1] > allowed:
            flag = "   <-- branch inside the main loop"
            bad += 1
        print(f"{name[10:86]:78s} {loops}{flag}")
    return 1 if (strict and bad) else 0


if __name__ == "__main__":
    sys.exit(main())
