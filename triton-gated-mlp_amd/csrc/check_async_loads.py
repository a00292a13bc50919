#!/usr/bin/env python3
"""Build-time check of the device assembly of kernels that issue loads as inline assembly.

Such a load fills its destination VGPRs some time after the instruction: the kernel orders the
uses with explicit `s_waitcnt vmcnt(N)`.  The compiler does not know that; when it runs short of
VGPRs it may copy a destination register elsewhere (an AGPR, another VGPR) right behind the load
instruction, i.e. copy what the register held before the data arrived.  Nothing warns of that and
the kernel then computes on stale values.

Model: vector-memory loads retire in issue order.  Walking each kernel's instructions in program
order, the loads in flight are a FIFO; `s_waitcnt vmcnt(N)` retires all but the youngest N.  Any
other instruction that names a VGPR an in-flight load will still write is an error.

usage: check_async_loads.py file.s      (exit status 1 on a violation)
"""
import re
import sys


def vgprs(operand):
    m = re.match(r"v\[(\d+):(\d+)\]$", operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", operand)
    return {int(m.group(1))} if m else set()


def check(path):
    lines = open(path).read().split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_Z\w+:", l)]
    failures = 0
    for k, begin in enumerate(starts):
        end = starts[k + 1] if k + 1 < len(starts) else len(lines)
        name = lines[begin].split(":")[0]
        in_flight = []  # destination VGPRs per load, oldest first (empty set: a load into LDS)
        bad = []
        for n in range(begin + 1, end):
            text = lines[n].split(";")[0].strip()
            if not text or text.startswith(".") or text.endswith(":"):
                continue
            if text.startswith("s_endpgm"):
                break
            wait = re.search(r"vmcnt\((\d+)\)", text)
            if text.startswith("s_waitcnt") and wait:
                keep = int(wait.group(1))
                in_flight = in_flight[len(in_flight) - keep:] if keep < len(in_flight) else in_flight
                if keep == 0:
                    in_flight = []
                continue
            operands = [o for o in re.split(r"[ ,]+", text)[1:] if o]
            if re.match(r"(buffer|global|flat)_load", text):
                in_flight.append(set() if re.search(r"\blds\b", text) else vgprs(operands[0]))
                continue
            pending = set().union(*in_flight) if in_flight else set()
            used = set()
            for o in operands:
                used |= vgprs(o)
            if used & pending:
                bad.append((n + 1, text))
        if bad:
            failures += 1
            print(f"{path}: {name}: {len(bad)} instruction(s) touch a register that a load in flight has yet to fill, e.g.")
            for n, text in bad[:4]:
                print(f"    line {n}: {text}")
    return failures


if __name__ == "__main__":
    sys.exit(1 if check(sys.argv[1]) else 0)
