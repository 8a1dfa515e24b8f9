"""Hazard check of the generated gfx950 assembly for the hazards the compiler cannot resolve inside inline assembly.

The hand-written kernels issue memory instructions from inline assembly.  LLVM inserts the wait states the hardware
needs between dependent instructions for the instructions it generates itself, but it does not look inside an
assembly statement.  Two of those rules can be broken by code the compiler places *in front of* such a statement:

* a scalar register written by the vector ALU (``v_readlane_b32`` / ``v_readfirstlane_b32``: this is how spilled
  scalar registers come back) needs five wait states before a vector-memory instruction reads it as descriptor or
  offset -- otherwise the load goes out with the register's old value, i.e. to a wild address;
* ``M0`` written by the scalar ALU needs one wait state before a direct-to-LDS load uses it.

``lint(path)`` returns the violations found in an assembly file (``hipcc -S --cuda-device-only``); the build fails
on any.
"""

from __future__ import annotations

import re
import sys

_VMEM = ("buffer_", "global_", "scratch_", "flat_", "tbuffer_")


def _instructions(path: str):
    out = []
    with open(path) as f:
        for n, line in enumerate(f, 1):
            t = line.strip()
            if not t or t[0] in ";." or t.endswith(":") or t.startswith(";;#"):
                continue
            out.append((n, t))
    return out


def _sregs(operands: str) -> set[int]:
    regs: set[int] = set()
    for m in re.finditer(r"\bs\[(\d+):(\d+)\]", operands):
        regs.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bs(\d+)\b", operands):
        regs.add(int(m.group(1)))
    return regs


def _wait_states(text: str) -> int:
    m = re.match(r"s_nop (\d+)", text)
    return int(m.group(1)) + 1 if m else 1


def lint(path: str) -> list[str]:
    ins = _instructions(path)
    found = []
    for idx, (n, t) in enumerate(ins):
        if not t.startswith(_VMEM):
            continue
        used = _sregs(t.split(None, 1)[1] if " " in t else "")
        waited = 0
        for k in range(idx - 1, max(idx - 8, -1), -1):
            pn, pt = ins[k]
            if waited >= 5:
                break
            d = re.match(r"v_read(?:first)?lane_b32 s(\d+)", pt)
            if d and int(d.group(1)) in used:
                found.append(f"{path}:{n}: `{t}` reads s{d.group(1)} {waited} wait states after `{pt}` (line {pn}); needs 5")
            waited += _wait_states(pt)
        if t.endswith(" lds") and idx > 0 and re.match(r"s_\w+ m0\b", ins[idx - 1][1]):
            found.append(f"{path}:{n}: `{t}` directly behind `{ins[idx - 1][1]}`; M0 needs one wait state")
    return found


if __name__ == "__main__":
    bad = [v for p in sys.argv[1:] for v in lint(p)]
    print("\n".join(bad) if bad else "no hazards found")
    sys.exit(1 if bad else 0)
