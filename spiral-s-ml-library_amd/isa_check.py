"""Check the generated gfx950 assembly for hazards the compiler cannot see.

Instructions inside inline asm are opaque to the compiler's hazard recogniser.  Two of the hardware's rules
bite the hand-scheduled kernels, both silently (wrong numbers, no error):

* two wait states between a vector-ALU write of a register and an MFMA that reads it: when the register
  allocator moves an operand (v_mov, v_accvgpr_*) right in front of an asm MFMA, the matrix pipe reads the old
  value;
* two wait states between a memory store of more than 8 bytes and a vector-ALU write of its data registers:
  when the next instruction's result lands in a register an asm store has not read yet, that result goes to
  memory instead;
* eight wait states (a 16x16x32 MFMA is four passes on gfx950) between an MFMA and any other kind of
  instruction that reads or overwrites its result; an MFMA in between counts as four, since it waits for the
  matrix pipe.

`scan` reports every v_mfma whose source registers were written by one of the two instructions before it,
every wide store whose data registers are written by one of the two instructions behind it, and every
instruction that touches an MFMA's result too early; the build runs it
over the device assembly of every source with such asm and fails on a hit.  The scan follows the listing, not
the control flow: it forgets what it has seen at an unconditional branch (the next line is reached through its
label only) and treats every other label as fall-through.
"""
import re

_RANGE = re.compile(r"([va])\[(\d+):(\d+)\]$")
_ONE = re.compile(r"([va])(\d+)$")
_WIDE_STORE = re.compile(r"(global|flat|scratch|buffer)_store_dwordx[34]$")
WAIT_STATES = 2
MFMA_RESULT_WAIT_STATES = 8


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
    """Hazards in an assembly listing: a list of (line number, kernel, writer, mfma); for stores, of
    (line number, kernel, writer, store); for early uses of an MFMA's result, of (line number, kernel, user, mfma)."""
    hits, kernel, window, stores, results = [], None, [], [], []   # stores, results: [wait states since, registers, text]
    for ln, line in enumerate(lines, 1):
        s = line.split(";")[0].strip()
        if not s:
            continue
        if s.endswith(":"):
            if not s.startswith(".L"):
                kernel, window, stores, results = s[:-1], [], [], []
            continue
        if s.startswith("."):
            continue
        parts = s.split(None, 1)
        op = parts[0]
        args = [a.strip().split(" ")[0] for a in parts[1].split(",")] if len(parts) > 1 else []
        if not op.startswith("v_mfma") and not op.startswith("s_"):
            touched = set()
            for a in args:
                touched |= _regs(a)
            for r in results:
                if r[1] & touched:
                    hits.append((ln, kernel, s, r[2]))
        for r in results:
            r[0] += int(args[0], 0) + 1 if op == "s_nop" and args else 4 if op.startswith("v_mfma") else 1
        results = [r for r in results if r[0] < MFMA_RESULT_WAIT_STATES]
        if op.startswith("v_mfma") and args:
            dst = _regs(args[0])
            results = [r for r in results if not (r[1] & dst)] + [[0, dst, s]]
        if op in ("s_branch", "s_endpgm", "s_setpc_b64"):
            # what follows in the listing is not what runs next: it is reached through its label only
            window, stores, results = [], [], []
            continue
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
