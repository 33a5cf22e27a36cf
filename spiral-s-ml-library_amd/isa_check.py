"""Check the generated gfx950 assembly for hazards the compiler cannot see.

Instructions inside inline asm are opaque to the compiler's hazard recogniser.  Two of the hardware's rules
bite the hand-scheduled kernels, both silently (wrong numbers, no error):

* two wait states between a vector-ALU write of a register and an MFMA that reads it: when the register
  allocator moves an operand (v_mov, v_accvgpr_*) right in front of an asm MFMA, the matrix pipe reads the old
  value;
* two wait states between a memory store of more than 8 bytes and a vector-ALU write of its data registers:
  when the next instruction's result lands in a register an asm store has not read yet, that result goes to
  memory instead.

`scan` reports every v_mfma whose source registers were written by one of the two instructions before it and
every wide store whose data registers are written by one of the two instructions behind it; the build runs it
over the device assembly of every source with such asm and fails on a hit.
"""
import re

_RANGE = re.compile(r"([va])\[(\d+):(\d+)\]$")
_ONE = re.compile(r"([va])(\d+)$")
_WIDE_STORE = re.compile(r"(global|flat|scratch|buffer)_store_dwordx[34]$")
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
    """Hazards in an assembly listing: a list of (line number, kernel, writer, mfma) and, for stores, of
    (line number, kernel, writer, store)."""
    hits, kernel, window, stores = [], None, [], []       # stores: [wait states since, data registers, text]
    for ln, line in enumerate(lines, 1):
        s = line.split(";")[0].strip()
        if not s:
            continue
        if s.endswith(":"):
            if not s.startswith(".L"):
                kernel, window, stores = s[:-1], [], []
            continue
        if s.startswith("."):
            continue
        parts = s.split(None, 1)
        op = parts[0]
        args = [a.strip().split(" ")[0] for a in parts[1].split(",")] if len(parts) > 1 else []
        is_valu = op.startswith("v_") and not op.startswith("v_cmp")
        if is_valu and args:
            written = _regs(args[0])
            for st in stores:
                if st[1] & written:
                    hits.append((ln, kernel, s, st[2]))
        for st in stores:
            st[0] += int(args[0], 0) + 1 if op == "s_nop" and args else 1
        stores = [st for st in stores if st[0] < WAIT_STATES]
        if _WIDE_STORE.match(op) and len(args) > 1:
            stores.append([0, _regs(args[0] if op.startswith("buffer_") else args[1]), s])
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
