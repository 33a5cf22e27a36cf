"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def dev(x, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return t if dtype is None else t.to(dtype)


def host(t):
    if t.dtype == torch.bfloat16:
        return t.float().cpu().numpy()
    return t.cpu().numpy()


def announce(msg):
    """Name the case before each GPU step, flushed, so a lost box still tells which case ran."""
    print("[gpu-case] " + msg, flush=True)
