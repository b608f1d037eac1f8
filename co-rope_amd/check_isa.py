"""Build-time check of the one place where the kernels rely on something the compiler does not know.

``mfma32_from`` (csrc/common.hpp) issues a matrix-core instruction from an asm statement so that its result lands in
registers of its own.  The compiler inserts the wait states that a vector instruction needs before it may touch the
result of a matrix-core instruction only for instructions it selected itself: to it the asm statement is opaque.  The
kernels are written so that the next instruction that touches those registers is another matrix-core instruction that
accumulates into them in place, which needs no wait states; ``check_asm_mfma`` verifies on the generated assembly, for
every such statement of every kernel, that nothing else touches them (and no branch is taken) within the wait states
the instruction set asks for, and the build fails if a register copy, a spill or anything else
has come between them (a different compiler version, more register pressure, accumulators moved to the other half of
the register file)."""
from __future__ import annotations

import re

_RANGE = re.compile(r"\bv\[(\d+):(\d+)\]")
_SINGLE = re.compile(r"\bv(\d+)\b")
# Wait states after which any instruction may touch the result of a matrix-core instruction: the CDNA3/4 instruction set
# manuals ask for 11 after one of 8 passes (32x32x16 with 16-bit operands on gfx950: 32 cycles) and 18 or 19 after one of
# 16 passes, before a vector instruction reads or overwrites the result.  One more than that here.
_WINDOW_8_PASSES = 12
_WINDOW_ANY = 20
_MFMA = re.compile(r"^\s*v_mfma_\w+\s+v\[(\d+):(\d+)\]\s*,\s*[^,]+,\s*[^,]+,\s*(\S+)")


def _vgprs(text):
    """VGPR numbers an instruction line names."""
    regs = set()
    for lo, hi in _RANGE.findall(text):
        regs.update(range(int(lo), int(hi) + 1))
    for r in _SINGLE.findall(text):
        regs.add(int(r))
    return regs


def _is_instruction(line):
    s = line.strip()
    return bool(s) and not s.startswith((";", ".", "//")) and not s.endswith(":")


def _first_touch(lines, labels, start, dst, window):
    """Follows every path from line `start` for `window` wait states (one per instruction issued, N + 1 for s_nop N).
    Returns None if on every path the first instruction that names a register of `dst` within the window is a
    matrix-core instruction accumulating into exactly `dst` in place; otherwise a description of the offender."""
    todo = [(start, 0)]
    seen = set()
    while todo:
        j, waited = todo.pop()
        while waited < window:
            if j >= len(lines):
                break
            if (j, waited) in seen:
                break
            seen.add((j, waited))
            nxt = lines[j]
            s = nxt.strip()
            j += 1
            if not _is_instruction(nxt) or "#ASM" in nxt:
                continue   # labels, comments, directives: fall through
            if s.startswith("s_endpgm"):
                break
            if s.startswith(("s_setpc", "s_swappc", "s_call")):
                return f"indirect control flow ({s}) {waited} wait states after it"
            if s.startswith(("s_branch", "s_cbranch")):
                target = s.split()[-1]
                if target not in labels:
                    return f"branch to an unknown label ({s})"
                if s.startswith("s_cbranch"):
                    todo.append((j, waited + 1))          # not taken
                j, waited = labels[target], waited + 1     # taken
                continue
            if _vgprs(nxt) & dst:
                mm = _MFMA.match(nxt)
                same = mm is not None and set(range(int(mm.group(1)), int(mm.group(2)) + 1)) == dst \
                    and _vgprs(mm.group(3)) == dst
                if not same:
                    return f"touched {waited} wait states after it by: {s}"
                break
            nop = re.match(r"s_nop\s+(\d+)", s)
            waited += int(nop.group(1)) + 1 if nop else 1
    return None


def check_asm_mfma(asm_text, name="<asm>"):
    """Returns a list of problems (empty: every asm-issued matrix-core result is first touched by an in-place accumulate,
    or by nothing within the wait states it needs)."""
    lines = asm_text.split("\n")
    labels = {m.group(1): n for n, l in enumerate(lines) for m in [re.match(r"^([.\w$]+):", l)] if m}
    problems = []
    kernel = "?"
    for i, line in enumerate(lines):
        if re.match(r"^[A-Za-z_]\w*:", line):
            kernel = line.split(":")[0]
        if "#ASMSTART" in line and i + 1 < len(lines) and "v_mfma" in lines[i + 1]:
            m = _MFMA.match(lines[i + 1])
            where = f"{name}: {kernel}: line {i + 2}"
            if m is None:
                problems.append(f"{where}: asm matrix-core instruction whose result is not a VGPR range: {lines[i + 1].strip()}")
                continue
            dst = set(range(int(m.group(1)), int(m.group(2)) + 1))
            window = _WINDOW_8_PASSES if re.search(r"v_mfma_f32_32x32x16_(bf16|f16)\b", lines[i + 1]) else _WINDOW_ANY
            verdict = _first_touch(lines, labels, i + 2, dst, window)
            if verdict:
                problems.append(f"{where}: v[{m.group(1)}:{m.group(2)}] {verdict}")
    return problems
