"""Host surface of the dense layers (reference: ml/layers.spi, generated ml/layers.py).

The reference builds a static graph (`matmul`, `relu`, `softmax`, ... ml/layers.spi:353-484) and
interprets it inside one kernel with every node's output going through a global-memory workspace
(graph_extract_, :181-252).  Here a dense stack with ReLU between layers and a row head is ONE
fused kernel (sp_mlp_forward): activations never leave the compute unit.
"""
import ctypes as C

import torch

from . import _lib
from ._lib import check, lib, ptr, stream_ptr

HEADS = {None: _lib.HEAD_NONE, "none": _lib.HEAD_NONE, "softmax": _lib.HEAD_SOFTMAX,
         "regret_matching": _lib.HEAD_REGRET_MATCHING, "softmax_regret_matching": _lib.HEAD_SOFTMAX_RM}


def weight_init(out_features, in_features, std=0.1, dtype=torch.float16, generator=None, device="cuda"):
    """`weight_init` (ml/layers.spi:460-463): N(0, std), std = 0.1 in the reference; stored
    (out_features, in_features) like `weight (a, b)` (:467)."""
    w = torch.randn((out_features, in_features), generator=generator, device=device, dtype=torch.float32) * std
    return w.to(dtype)


def mlp_forward(x, weights, biases=None, head="softmax_regret_matching", u=None, mask_size=0, want_logits=False):
    """policy, action[, logits] = fused forward of relu-MLP + head + discrete sampling.

    x: (batch, in) f16/bf16; weights[i]: (out_i, in_i) of the same dtype (the B operand of A.B^T,
    ml/layers.spi:227-240,467); biases: optional list of f32 (out_i,) or None entries (build
    extension, the reference has no bias); u: (batch,) f32 uniforms in (0, 1] or None (no action).
    head: None | "softmax" | "regret_matching" | "softmax_regret_matching"; mask_size > 0 restricts
    the head to columns j < mask_size (masked_* layers, ml/layers.spi:408-432)."""
    n = len(weights)
    dims = [x.shape[1]] + [w.shape[0] for w in weights]
    for i, w in enumerate(weights):
        if w.dtype != x.dtype:
            raise TypeError("weights[%d] must have the dtype of x" % i)
        assert w.shape[1] == dims[i], "The K dimension of the A and B tensors must match."
    batch = x.shape[0]
    policy = torch.empty((batch, dims[-1]), dtype=torch.float32, device=x.device)
    action = torch.empty((batch,), dtype=torch.int32, device=x.device) if u is not None else None
    logits = torch.empty((batch, dims[-1]), dtype=torch.float32, device=x.device) if want_logits else None
    wp = (C.c_void_p * n)(*[ptr(w, name="weights[%d]" % i) for i, w in enumerate(weights)])
    bp = None
    if biases is not None:
        bp = (C.c_void_p * n)(*[ptr(b, torch.float32, "biases[%d]" % i) if b is not None else None
                                for i, b in enumerate(biases)])
    dp = (C.c_int32 * (n + 1))(*dims)
    check(lib.sp_mlp_forward(_lib.DTYPES[x.dtype], ptr(x, name="x"), n, wp, bp, dp, ptr(u, torch.float32, "u"),
                             ptr(policy), ptr(action), ptr(logits), batch, HEADS[head], mask_size, stream_ptr()))
    out = (policy, action)
    return out + (logits,) if want_logits else out
