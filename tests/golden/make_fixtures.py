#!/usr/bin/env python3
"""Convert the reference's golden stdout captures into small .npz fixtures.

The reference's tests print tensors into `test_text_outputs/` (writer:
coreext/testing.spi:6-15, tensor printer: coreext/console/tensor.spi:4-45).  The
format is nested `[` `]` lists, leaves separated by "; ", tuple components by
", ", floats printed with %f (6 decimals) and the whole print cut with " ..."
after a leaf limit.  A file may start with a "DEBUG MODE. ..." banner line
(corecuda/base.spi:104-105).

This script only reads those *data* files (no reference code is imported or run)
and writes one compressed .npz per reference test case next to itself:

    python tests/golden/make_fixtures.py [/root/reference]

Every array is stored flat-complete when the print was complete, or as the
leading complete rows when the print was truncated; `<name>__truncated` tells
which.
"""
import os
import re
import sys

import numpy as np

_TOKEN = re.compile(r"\[|\]|;|,|\.\.\.|[-+]?(?:\d+\.\d*|\.\d+|\d+)(?:[eE][-+]?\d+)?|[-+]?inf|nan")


def parse_tensor_text(text):
    """Parse one printed tensor.  Returns (nested python lists, truncated flag).

    A leaf is a number or a tuple of numbers (printed `a, b`)."""
    lines = [ln for ln in text.splitlines() if ln.strip() and not ln.startswith("DEBUG MODE")]
    toks = _TOKEN.findall(" ".join(lines))
    pos = 0
    truncated = False

    def number(tok):
        return float(tok) if any(c in tok for c in ".einf") else int(tok)

    def parse_list():
        nonlocal pos, truncated
        assert toks[pos] == "["
        pos += 1
        items = []
        cur = []  # components of the current leaf tuple
        while pos < len(toks):
            t = toks[pos]
            if t == "[":
                items.append(parse_list())
            elif t == "]":
                pos += 1
                if cur:
                    items.append(cur[0] if len(cur) == 1 else tuple(cur))
                return items
            elif t == ";":
                pos += 1
                if cur:
                    items.append(cur[0] if len(cur) == 1 else tuple(cur))
                    cur = []
            elif t == ",":
                pos += 1
            elif t == "...":
                truncated = True
                pos += 1
            else:
                cur.append(number(t))
                pos += 1
        return items

    if toks and toks[0] != "[":  # a bare scalar
        return number(toks[0]), False
    return parse_list(), truncated


def to_array(nested, truncated):
    """Nested lists -> ndarray.  For truncated prints keep only the complete leading rows."""
    if not isinstance(nested, list):
        return np.asarray(nested)
    if truncated:
        # drop ragged tails: keep rows whose length equals the first row's length
        def fix(x):
            if x and isinstance(x[0], list):
                rows = [fix(r) for r in x]
                n0 = len(rows[0])
                rows = [r for r in rows if len(r) == n0]
                return rows
            return x
        nested = fix(nested)
    arr = np.asarray(nested)
    return arr


def load(path):
    with open(path) as f:
        text = f.read()
    # test5 prints input and output tensors one after another, separated by the banner line
    return text


def convert_case(src_dir, names):
    out = {}
    for name in names:
        p = os.path.join(src_dir, name + ".txt")
        if not os.path.exists(p):
            continue
        nested, trunc = parse_tensor_text(load(p))
        arr = to_array(nested, trunc)
        key = name.replace("''", "_pp").replace("'", "_p")
        if arr.dtype.kind == "f":
            arr = arr.astype(np.float32) if key != "output_reduce" else arr.astype(np.float64)
        elif arr.dtype.kind in "iu":
            arr = arr.astype(np.int64)
        out[key] = arr
        out[key + "__truncated"] = np.asarray(trunc)
    return out


ROW_NAMES = ["input", "input_identity", "output_reduce", "output_identity", "output_softmax",
             "output_masked_softmax", "output_softmax_scan", "output_ln", "output_argmax",
             "output_indices_map", "output_indices_reduction", "output_sum_exclusive",
             "output_softmax'", "output_softmax''", "output_sampling", "output_sampling'"]
GATHER_NAMES = ["zip_input_output_identity_map", "input_identity", "output_indices_map", "output_op_map",
                "output_sample_reduce", "output_indices_reduce"]
REDUCE_NAMES = ["input_identity", "output_reduce_block", "output_reduce_grid"]


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    root = os.path.join(ref, "test_text_outputs", "primitives")
    here = os.path.dirname(os.path.abspath(__file__))
    for test, names in (("test2", ROW_NAMES), ("test4", ROW_NAMES), ("test3", GATHER_NAMES)):
        for sub in ("a", "b"):
            d = convert_case(os.path.join(root, test, sub), names)
            np.savez_compressed(os.path.join(here, f"primitives_{test}_{sub}.npz"), **d)
            print(test, sub, {k: v.shape for k, v in d.items() if not k.endswith("__truncated")})
    d = convert_case(os.path.join(root, "test6", "a"), REDUCE_NAMES)
    np.savez_compressed(os.path.join(here, "primitives_test6_a.npz"), **d)
    # test5: two tensors (input, transposed output) in one file
    for sub in ("a", "b"):
        text = load(os.path.join(root, "test5", sub, "transpose.txt"))
        parts = [ln for ln in text.splitlines() if ln.startswith("[")]
        assert len(parts) == 2
        a = to_array(*parse_tensor_text(parts[0])).astype(np.int64)
        b = to_array(*parse_tensor_text(parts[1])).astype(np.int64)
        np.savez_compressed(os.path.join(here, f"primitives_test5_{sub}.npz"), input=a, output=b)
        print("test5", sub, a.shape, b.shape)


if __name__ == "__main__":
    main()
