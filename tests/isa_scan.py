"""Scans gfx950 assembly text for a hazard the compiler cannot see: a VALU instruction (v_accvgpr_write
included) that writes a source register of an inline-assembly MFMA fewer than `min_wait` wait states
before it.  For its own MFMA instructions the compiler inserts the wait states; an MFMA inside an asm
statement is opaque to it, and on the GPU such an MFMA was observed to read the old register content.
"""
import re

_RANGE = re.compile(r"\b([va])\[(\d+):(\d+)\]")
_SINGLE = re.compile(r"\b([va])(\d+)\b")


def registers(text):
    out = set()
    for kind, lo, hi in _RANGE.findall(text):
        out.update("%s%d" % (kind, i) for i in range(int(lo), int(hi) + 1))
    for kind, idx in _SINGLE.findall(_RANGE.sub(" ", text)):
        out.add(kind + idx)
    return out


def instructions(asm_text):
    """(line number, instruction text, inside an asm statement) for every instruction line."""
    inside = False
    for n, raw in enumerate(asm_text.split("\n"), 1):
        s = raw.strip()
        if s.startswith(";;#ASMSTART"):
            inside = True
            continue
        if s.startswith(";;#ASMEND"):
            inside = False
            continue
        s = s.split(";")[0].strip()
        if not s or s.startswith(".") or s.endswith(":"):
            continue
        yield n, s, inside


def asm_mfma_hazards(asm_text, min_wait=3, lookback=8):
    """List of (mfma line, writer line, wait states between, writer text)."""
    ins = list(instructions(asm_text))
    found = []
    for i, (n, s, inside) in enumerate(ins):
        if not (inside and s.startswith("v_mfma")):
            continue
        operands = s.split(None, 1)[1].split(",")
        pending = registers(",".join(operands[1:]))   # sources whose most recent writer has not been seen yet
        wait = 0
        for n2, s2, _ in reversed(ins[max(0, i - lookback):i]):
            if wait >= min_wait or not pending:
                break
            m = re.match(r"s_nop (\d+)", s2)
            if m:
                wait += int(m.group(1)) + 1
                continue
            parts = s2.split(None, 1)
            written = registers(parts[1].split(",")[0]) & pending if len(parts) > 1 and not parts[0].startswith("s_") else set()
            if written:
                is_valu = parts[0].startswith("v_") and not parts[0].startswith("v_mfma")
                if is_valu:
                    found.append((n, n2, wait, s2))
                    break
                pending -= written      # a load wrote them last: ordered by s_waitcnt
            wait += 1
    return found
