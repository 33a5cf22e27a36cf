"""Tensor printer in the reference's golden-file format (coreext/console/tensor.spi:4-45):
nested `[` `]`, leaves separated by "; ", tuple components by ", ", floats as %f, and the print
cut with " ..." once `limit` leaves were written."""
import numpy as np


def _leaf(v):
    if isinstance(v, tuple):
        return ", ".join(_leaf(x) for x in v)
    if isinstance(v, (float, np.floating)):
        return "%f" % v
    return str(int(v))


def format_tensor(limit, *arrays):
    """Zip `arrays` (same shape) into tuple leaves and print up to `limit` leaves."""
    arrays = [np.asarray(a) for a in arrays]
    shape = arrays[0].shape
    count = [0]

    def leaf(idx):
        vals = tuple(a[idx].item() for a in arrays)
        return _leaf(vals if len(vals) > 1 else vals[0])

    def rec(prefix, depth):
        if depth == len(shape):
            count[0] += 1
            return leaf(prefix)
        parts = []
        for i in range(shape[depth]):
            if count[0] >= limit:
                return "[" + "; ".join(parts) + " ...]"
            parts.append(rec(prefix + (i,), depth + 1))
        return "[" + "; ".join(parts) + "]"

    return rec((), 0) if shape else leaf(())


def write_ln(path, limit, *arrays):
    with open(path, "w") as f:
        f.write(format_tensor(limit, *arrays) + "\n")
