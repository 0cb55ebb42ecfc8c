#!/usr/bin/env python3
"""Build-time check of the device assembly of a source file that holds hand-written DPP instructions.

The compiler's hazard recogniser does not look into inline asm, and on this target a DPP operand must not be read
sooner than two wait states after a vector instruction wrote that register, nor sooner than five after a vector
instruction wrote EXEC.  This script walks the assembly (`hipcc -S --cuda-device-only`) and fails if any DPP
instruction, hand-written or not, comes too early.  Usage: check_dpp_hazards.py file.s [minimum count of
v_fmac_f32_dpp expected]."""
import re
import sys


def instructions(path):
    for raw in open(path):
        line = raw.split(";")[0].split("//")[0].strip()
        if not line or line.startswith(".") or line.endswith(":"):
            continue
        yield line


def written_vgprs(ins):
    """VGPRs a vector ALU instruction writes (its first operand)."""
    m = re.match(r"v_\w+\s+(?:v\[(\d+):(\d+)\]|v(\d+))", ins)
    if not m or ins.startswith(("v_cmp_", "v_cmpx_", "v_nop")):
        return set()
    if m.group(1):
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    return {int(m.group(3))}


def writes_exec(ins):
    return ins.startswith("v_cmpx_") or bool(re.match(r"v_\w+\s+exec", ins))


def dpp_source(ins):
    """The register a DPP instruction reads through the DPP path: its first source operand."""
    m = re.match(r"v_\w+_dpp\s+\S+,\s*v(\d+)", ins)
    return int(m.group(1)) if m else None


def wait_states(ins):
    m = re.match(r"s_nop\s+(\d+)", ins)
    return int(m.group(1)) + 1 if m else 1


def main():
    path = sys.argv[1]
    want = int(sys.argv[2]) if len(sys.argv) > 2 else 0
    window, bad, n_dpp, n_fmac = [], [], 0, 0
    for ins in instructions(path):
        src = dpp_source(ins)
        if src is not None:
            n_dpp += 1
            n_fmac += ins.startswith("v_fmac_f32_dpp")
            between = 0  # wait states between an earlier instruction and this one
            for prev in reversed(window):
                if between < 2 and src in written_vgprs(prev):
                    bad.append((prev, ins, between))
                if between < 5 and writes_exec(prev):
                    bad.append((prev, ins, between))
                between += wait_states(prev)
                if between >= 5:
                    break
        window.append(ins)
        if len(window) > 8:
            window.pop(0)
    for prev, ins, between in bad[:20]:
        print("hazard: %d wait state(s) between\n    %s\nand\n    %s" % (between, prev, ins))
    print("%s: %d DPP instructions (%d v_fmac_f32_dpp), %d hazards" % (path, n_dpp, n_fmac, len(bad)))
    if bad or n_fmac < want:
        sys.exit(1)


if __name__ == "__main__":
    main()
