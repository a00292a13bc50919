#!/usr/bin/env python3
"""Build-time check of the device assembly of kernels that move tiles with `buffer_load ... lds`.

Those loads take their LDS base address from M0.  The GEMM kernels write M0 in one inline-assembly
statement (set_lds_dma_base) and consume it in up to four later ones (load16_to_lds_at), with
compiler-scheduled code in between; the compiler is not told that M0 stays live.  It has no use
for M0 of its own in these kernels (no indirect register indexing, messages or GWS), but nothing
in the language guarantees that, so the build verifies it: inside every kernel that contains an
inline-assembly LDS-DMA load, no instruction OUTSIDE the inline-assembly blocks may write M0, and
none may be of a kind that implies an M0 use the compiler chose (s_movrel*, v_movrel*, s_sendmsg,
ds_gws_*).  A violation would send tiles to the wrong LDS address without any other symptom.

A file in which the scan recognises no kernel with such loads fails too (every GEMM unit has
several): kernels are found by their mangled label and the loads by the inline-assembly markers,
and a compiler that changed either would otherwise make the check pass without checking anything.

usage: check_m0.py file.s [minimum kernels, default 1]     (exit status 1 on a violation)
"""
import re
import sys

WRITES_M0 = re.compile(r"^(s_|v_readfirstlane_b32|v_readlane_b32)\S*\s+m0\b")
USES_M0 = re.compile(r"^(s_movrel|v_movrel|s_sendmsg|ds_gws_)")
LDS_DMA = re.compile(r"^buffer_load_\S+\s.*\blds\b")


def check(path, minimum=1):
    lines = open(path).read().split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_Z\w+:", l)]
    failures = 0
    checked = 0
    for k, begin in enumerate(starts):
        end = starts[k + 1] if k + 1 < len(starts) else len(lines)
        name = lines[begin].split(":")[0]
        in_asm = False
        has_dma = False
        bad = []
        for n in range(begin + 1, end):
            raw = lines[n].strip()
            if raw.startswith(";;#ASMSTART") or raw.startswith(";#ASMSTART"):
                in_asm = True
                continue
            if raw.startswith(";;#ASMEND") or raw.startswith(";#ASMEND"):
                in_asm = False
                continue
            text = raw.split(";")[0].strip()
            if not text or text.startswith(".") or text.endswith(":"):
                continue
            if in_asm:
                has_dma = has_dma or bool(LDS_DMA.match(text))
            elif WRITES_M0.match(text) or USES_M0.match(text):
                bad.append((n + 1, text))
        if has_dma:
            checked += 1
            for line_no, text in bad:
                print(f"{path}:{line_no}: {name}: compiler-generated use of M0 in a kernel with LDS-DMA loads: {text}")
                failures += 1
    print(f"check_m0: {checked} kernels with LDS-DMA loads checked in {path}, {failures} violation(s)")
    if checked < minimum:
        print(f"{path}: expected at least {minimum} kernel(s) with LDS-DMA loads, recognised {checked}: "
              "the scan no longer matches the assembly, nothing was verified")
        failures += 1
    return failures


if __name__ == "__main__":
    sys.exit(1 if check(sys.argv[1], int(sys.argv[2]) if len(sys.argv) > 2 else 1) else 0)
