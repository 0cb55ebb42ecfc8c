#!/usr/bin/env python3
"""Build-time check of the device assembly of a source file that holds hand-written DPP instructions.

The compiler's hazard recogniser does not look into inline asm, and on this target a DPP operand must not be read
sooner than two wait states after a vector instruction wrote that register, nor sooner than five after a vector
instruction wrote EXEC.  This script walks the assembly (`hipcc -S --cuda-device-only`) and fails if any DPP
instruction, hand-written or not, comes too early: along the text order (the fall-through path; after an
unconditional branch this is stricter than needed, never laxer) and along every branch, i.e. from the instructions
in front of each `s_branch` / `s_cbranch_*` to those behind its target label.  Indirect jumps (`s_setpc_b64`,
`s_swappc_b64`) are refused: their targets are not in the text.

A third rule is for hand-written READERS: a vector instruction may not read the result registers of a
v_mfma_*_4x4x4_* (two passes) sooner than five wait states after it.  The compiler keeps that distance for the
instructions it emits itself, but an asm statement that takes the result as an operand is opaque to it.  Other
matrix-core shapes have other distances: the script refuses a file that holds them until their rule is added.

These rules are the hazards of what this build writes by hand: vector instructions with a DPP source, in asm
statements next to matrix-core instructions.
Whoever adds another hand-written class (an `s_waitcnt`-sensitive memory instruction, an MFMA with its own
dependency wait states, writes of M0 or VCC in front of their readers, ...) has to add that class's rules here:
the script knows nothing of hazards it was not told about.

A compile that silently dropped the hand-written instructions must not pass either: the optional second argument
is a regular expression, and every function of the file whose symbol matches it (the set of instantiations is the
build's own, not a number kept by hand) has to hold at least one v_fmac_f32_dpp, and at least one function has to
match.  A plain number is taken as the minimum count over the whole file.

Usage: check_dpp_hazards.py file.s [regular expression of the symbols that must hold v_fmac_f32_dpp | minimum count]."""
import re
import sys


def instructions(path):
    """The instructions in text order; a label is yielded as ("label", name)."""
    for raw in open(path):
        line = raw.split(";")[0].split("//")[0].strip()
        if line.endswith(":"):  # labels first: local ones start with a dot, as directives do
            yield ("label", line[:-1])
            continue
        if not line or line.startswith("."):
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


def read_vgprs(ins):
    """VGPRs a vector instruction reads: every register operand behind the first, and the first as well where the
    instruction accumulates into its destination."""
    if not ins.startswith("v_"):
        return set()
    ops = ins.split(None, 1)[1] if " " in ins else ""
    first, _, rest = ops.partition(",")
    if "UNUSED_PRESERVE" in ins or ins.startswith(("v_fmac", "v_mac", "v_dot4c")):
        rest = first + "," + rest  # the destination is a source, too
    regs = set()
    for a, b in re.findall(r"v\[(\d+):(\d+)\]", rest):
        regs.update(range(int(a), int(b) + 1))
    regs.update(int(r) for r in re.findall(r"\bv(\d+)\b", rest))
    return regs


MFMA_4X4_WAIT = 5  # wait states between a two-pass matrix-core instruction and a vector read of its result


def mfma_result(ins):
    """The result registers of a 4x4x4 matrix-core instruction, or None."""
    m = re.match(r"v_mfma_\w+_4x4x4\w*\s+v\[(\d+):(\d+)\]", ins)
    return set(range(int(m.group(1)), int(m.group(2)) + 1)) if m else None


def wait_states(ins):
    m = re.match(r"s_nop\s+(\d+)", ins)
    return int(m.group(1)) + 1 if m else 1


REACH = 8  # instructions looked at on either side of a point: more than five wait states in any case


def hazards(seq, first_checked=0):
    """(earlier instruction, DPP instruction, wait states between) for every DPP instruction of seq from index
    first_checked on that reads its operand too early after an instruction of seq in front of it."""
    bad = []
    for k in range(first_checked, len(seq)):
        reads = read_vgprs(seq[k])
        if not reads:
            continue
        between = 0
        for prev in reversed(seq[max(0, k - REACH):k]):
            res = mfma_result(prev)
            if res and between < MFMA_4X4_WAIT and res & reads:
                bad.append((prev, seq[k], between))
            if written_vgprs(prev) & reads and not res:
                reads = reads - written_vgprs(prev)  # a later writer in between: the read is of that value
            between += wait_states(prev)
            if between >= MFMA_4X4_WAIT:
                break
    for k in range(first_checked, len(seq)):
        src = dpp_source(seq[k])
        if src is None:
            continue
        between = 0  # wait states between an earlier instruction and this one
        for prev in reversed(seq[max(0, k - REACH):k]):
            if between < 2 and src in written_vgprs(prev):
                bad.append((prev, seq[k], between))
            if between < 5 and writes_exec(prev):
                bad.append((prev, seq[k], between))
            between += wait_states(prev)
            if between >= 5:
                break
    return bad


def branch_target(ins):
    m = re.match(r"s_c?branch\w*\s+(\S+)", ins)
    return m.group(1) if m else None


def main():
    path = sys.argv[1]
    want = sys.argv[2] if len(sys.argv) > 2 else "0"
    code, labels = [], {}
    for item in instructions(path):
        if isinstance(item, tuple):
            labels[item[1]] = len(code)  # index of the first instruction behind the label
        else:
            code.append(item)
    n_dpp = sum(dpp_source(ins) is not None for ins in code)
    n_fmac = sum(ins.startswith("v_fmac_f32_dpp") for ins in code)
    bad = hazards(code)
    unknown = [ins for ins in code if ins.startswith(("s_setpc_b64", "s_swappc_b64"))]
    unknown += [ins for ins in code if ins.startswith("v_mfma") and mfma_result(ins) is None]  # a shape without a rule
    for k, ins in enumerate(code):
        target = branch_target(ins)
        if target is None:
            continue
        if target not in labels:
            unknown.append(ins)
            continue
        head = code[max(0, k + 1 - REACH):k + 1]  # up to and including the branch, which is a wait state itself
        tail = code[labels[target]:labels[target] + REACH]
        bad += hazards(head + tail, first_checked=len(head))
    bad = sorted(set(bad))
    for prev, ins, between in bad[:20]:
        print("hazard: %d wait state(s) between\n    %s\nand\n    %s" % (between, prev, ins))
    for ins in unknown[:20]:
        print("cannot follow: %s" % ins)
    missing = []
    if want.isdigit():
        if n_fmac < int(want):
            missing.append("the file: %d v_fmac_f32_dpp, %s expected" % (n_fmac, want))
    else:
        starts = sorted((at, name) for name, at in labels.items() if not name.startswith("."))  # function symbols
        matched = 0
        for i, (at, name) in enumerate(starts):
            if not re.search(want, name):
                continue
            matched += 1
            end = starts[i + 1][0] if i + 1 < len(starts) else len(code)
            if not any(ins.startswith("v_fmac_f32_dpp") for ins in code[at:end]):
                missing.append(name)
        if not matched:
            missing.append("no function symbol matches %r" % want)
    for name in missing[:20]:
        print("no v_fmac_f32_dpp: %s" % name)
    print("%s: %d DPP instructions (%d v_fmac_f32_dpp), %d hazards" % (path, n_dpp, n_fmac, len(bad)))
    if bad or unknown or missing:
        sys.exit(1)


if __name__ == "__main__":
    main()
