"""Build-time check of the places where the kernels rely on something the compiler does not know.

Some matrix-core instructions are issued from asm statements (``mfma32_from`` in csrc/common.hpp: a result in registers of
its own; the score products of csrc/rope_attn_fwd_pipe_acc.hip: an operand in the accumulation half of the register file).
The compiler inserts the wait states the instruction set asks for around a matrix-core instruction only for instructions
it selected itself: to it an asm statement is opaque.  ``check_asm_mfma`` verifies on the generated assembly, for every
such statement of every kernel:

* result: the next instruction that touches its result registers is a matrix-core instruction accumulating into them in
  place (which needs no wait states), or nothing touches them (and no indirect branch is taken) within the wait states a
  vector instruction needs before it may read or overwrite them -- every path from the statement is followed;
* addend: when the result lands in other registers than the addend (C), nothing but a matrix-core instruction writes
  the addend's registers while the instruction may still be reading them;
* operands: no vector instruction wrote one of its operand registers in the two wait states before it (looked for in the
  straight-line code in front of the statement; a label ends the search).

The build fails if a register copy, a spill or anything else has come between (a different compiler version, more
register pressure, accumulators moved to the other half of the register file)."""
from __future__ import annotations

import re

_RANGE = re.compile(r"\b([va])\[(\d+):(\d+)\]")
_SINGLE = re.compile(r"\b([va])(\d+)\b")
# Wait states after which any instruction may touch the result of a matrix-core instruction: the CDNA3/4 instruction set
# manuals ask for 11 after one of 8 passes (32x32x16 with 16-bit operands on gfx950: 32 cycles) and 18 or 19 after one of
# 16 passes, before a vector instruction reads or overwrites the result.  One more than that here.
_WINDOW_8_PASSES = 12
_WINDOW_ANY = 20
# ... during which a vector instruction must not overwrite the addend of an instruction that is still reading it (7 after
# one of 8 passes, 15 after one of 16; one more here)
_ADDEND_8_PASSES = 8
_ADDEND_ANY = 16
# ... and between a vector instruction's write of a register and a matrix-core instruction's read of it (the compiler
# itself puts two there)
_OPERAND_WAIT = 2
_MFMA = re.compile(r"^\s*v_mfma_\w+\s+([va]\[\d+:\d+\])\s*,\s*([^,]+),\s*([^,]+),\s*(\S+)")
#: source text that issues a matrix-core instruction from an asm statement, or calls a helper that does
ASM_MFMA_IN_SOURCE = re.compile(r"\bmfma32_(from|acc|zero)\w*\s*\(|asm[^;]*\"v_mfma")


def _regs(text):
    """Registers ('v' | 'a', number) an instruction line (or operand) names."""
    regs = set()
    for f, lo, hi in _RANGE.findall(text):
        regs.update((f, n) for n in range(int(lo), int(hi) + 1))
    for f, r in _SINGLE.findall(text):
        regs.add((f, int(r)))
    return regs


def _written(line):
    """Registers an instruction writes: those of its first operand (stores and compares write none that matter here)."""
    s = line.strip()
    op = s.split()[0]
    if op.startswith(("ds_write", "global_store", "scratch_store", "buffer_store", "v_cmp", "s_", "flat_store")):
        return set()
    rest = s[len(op):]
    first = rest.split(",")[0]
    return _regs(first)


def _is_instruction(line):
    s = line.strip()
    return bool(s) and not s.startswith((";", ".", "//")) and not s.endswith(":")


def _walk(lines, labels, start, window, visit):
    """Follows every path from line `start` for `window` wait states (one per instruction issued, N + 1 for s_nop N).
    visit(line, waited) -> None: go on; "stop": this path is settled; any other string: a problem, returned."""
    todo = [(start, 0)]
    seen = set()
    while todo:
        j, waited = todo.pop()
        while waited < window:
            if j >= len(lines) or (j, waited) in seen:
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
            verdict = visit(nxt, waited)
            if verdict == "stop":
                break
            if verdict:
                return verdict
            nop = re.match(r"s_nop\s+(\d+)", s)
            waited += int(nop.group(1)) + 1 if nop else 1
    return None


def _first_touch(lines, labels, start, dst, window):
    """None if on every path the first instruction that names a register of `dst` within the window is a matrix-core
    instruction accumulating into exactly `dst` in place; otherwise a description of the offender."""
    def visit(line, waited):
        if _regs(line) & dst:
            mm = _MFMA.match(line)
            same = mm is not None and _regs(mm.group(1)) == dst and _regs(mm.group(4)) == dst
            return "stop" if same else f"touched {waited} wait states after it by: {line.strip()}"
        return None
    return _walk(lines, labels, start, window, visit)


def _addend_overwritten(lines, labels, start, addend, window):
    def visit(line, waited):
        if line.strip().startswith("v_mfma"):
            return None        # matrix-core instructions queue up behind each other
        if _written(line) & addend:
            return f"addend overwritten {waited} wait states after it by: {line.strip()}"
        return None
    return _walk(lines, labels, start, window, visit)


def _operand_written_just_before(lines, at, operands):
    """Looks back from line `at` (the asm instruction) over straight-line code for a vector write of an operand register."""
    waited, j = 0, at - 1
    while j >= 0 and waited < _OPERAND_WAIT:
        line = lines[j]
        j -= 1
        s = line.strip()
        if re.match(r"^[.\w$]+:", line):
            return None                     # a label: other paths lead here, not looked into
        if not _is_instruction(line) or "#ASM" in line:
            continue
        if s.startswith(("s_branch", "s_cbranch")):
            return None
        if s.startswith("v_") and not s.startswith("v_mfma") and _written(line) & operands:
            return f"operand written {waited} wait states before it by: {s}"
        nop = re.match(r"s_nop\s+(\d+)", s)
        waited += int(nop.group(1)) + 1 if nop else 1
    return None


def check_asm_mfma(asm_text, name="<asm>"):
    """Returns a list of problems (empty: every asm-issued matrix-core instruction is safe in the sense of the module text)."""
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
                problems.append(f"{where}: asm matrix-core instruction not understood: {lines[i + 1].strip()}")
                continue
            dst, addend = _regs(m.group(1)), _regs(m.group(4))
            eight = re.search(r"v_mfma_f32_32x32x16_(bf16|f16)\b", lines[i + 1]) is not None
            verdict = _first_touch(lines, labels, i + 2, dst, _WINDOW_8_PASSES if eight else _WINDOW_ANY)
            if verdict:
                problems.append(f"{where}: {m.group(1)} {verdict}")
            if addend and addend != dst:
                verdict = _addend_overwritten(lines, labels, i + 2, addend, _ADDEND_8_PASSES if eight else _ADDEND_ANY)
                if verdict:
                    problems.append(f"{where}: {m.group(4)} {verdict}")
            verdict = _operand_written_just_before(lines, i + 1, _regs(m.group(2)) | _regs(m.group(3)) | addend)
            if verdict:
                problems.append(f"{where}: {verdict}")
    return problems
