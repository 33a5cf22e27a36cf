"""Check the generated gfx950 assembly for a hazard the compiler cannot see.

The MFMAs of the hand-scheduled kernels are inline asm, which the compiler's hazard recogniser treats as
opaque.  The hardware wants two wait states between a vector-ALU write of a register and an MFMA that reads
it; when the register allocator moves an operand (v_mov, v_accvgpr_*) right in front of such an asm MFMA, the
matrix pipe reads the old value and the kernel computes garbage without any error.  `scan` reports every
v_mfma whose source registers were written by one of the two instructions before it; the build runs it over
the device assembly of every source that holds asm MFMAs and fails on a hit.
"""
import re

_RANGE = re.compile(r"([va])\[(\d+):(\d+)\]$")
_ONE = re.compile(r"([va])(\d+)$")
WAIT_STATES = 2


def _regs(tok):
    tok = tok.strip().rstrip(",")
    m = _RANGE.match(tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = _ONE.match(tok)
    if m:
        return {(m.group(1), int(m.group(2)))}
    return set()


def scan(lines):
    """Hazards in an assembly listing: a list of (line number, kernel, writer, mfma)."""
    hits, kernel, window = [], None, []
    for ln, line in enumerate(lines, 1):
        s = line.split(";")[0].strip()
        if not s:
            continue
        if s.endswith(":"):
            if not s.startswith(".L"):
                kernel, window = s[:-1], []
            continue
        if s.startswith("."):
            continue
        parts = s.split(None, 1)
        op = parts[0]
        args = [a.strip().split(" ")[0] for a in parts[1].split(",")] if len(parts) > 1 else []
        if op.startswith("v_mfma"):
            src = set()
            for a in args[1:]:
                src |= _regs(a)
            for writer, written in window[-WAIT_STATES:]:
                if written & src:
                    hits.append((ln, kernel, writer, s))
            window.append((s, set()))
        elif op == "s_nop":
            window.extend([("s_nop", set())] * (int(args[0], 0) + 1 if args else 1))
        elif op.startswith("v_") and not op.startswith("v_cmp"):
            window.append((s, _regs(args[0]) if args else set()))
        else:
            window.append((s, set()))
        del window[:-WAIT_STATES]
    return hits


def scan_file(path):
    with open(path) as f:
        return scan(f)
