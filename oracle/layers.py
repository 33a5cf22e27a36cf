"""Dense-layer forward pass restated in NumPy.  TEST INFRASTRUCTURE ONLY.

Follows the graph interpreter of ml/layers.spi:194-240: `BlockMatmul(x, w)` is
`matmul_tf32' false true 1 x w 0 out`, i.e. out = x . w^T with the weight stored
(out_features, in_features) row-major (`matmul (b,a) x = BlockMatmul(x, weight (a,b))`, :467);
`relu = max 0` (:355); the heads are the row primitives (:367-432).  There is no bias in the
reference; `bias` here is this build's extension.

PARITY UNPINNED end to end against the reference: its layer goldens
(test_text_outputs/layers/test3..5) hold weights and inputs truncated to 100 values, so no
forward output can be recomputed from them.  The function is a composition of gemm_abt
(pinned mathematically) and the golden-pinned row primitives.
"""
import numpy as np

from . import gemm, row_ops

HEAD_NONE = 0               # raw last-layer outputs
HEAD_SOFTMAX = 1            # softmax (ml/layers.spi:370-375)
HEAD_REGRET_MATCHING = 2    # regret_matching (:377-382)
HEAD_SOFTMAX_RM = 3         # softmax, then regret matching of the probabilities


def mlp_forward(x, weights, biases=None, head=HEAD_SOFTMAX_RM, u=None, act_dtype=None, mask_size=None):
    """x: (batch, in) f32 values; weights[i]: (out_i, in_i) f32 values (already rounded to their
    storage dtype).  ReLU after every layer but the last.  `act_dtype` ("f16"/"bf16"/None) rounds
    the hidden activations to the dtype the fused kernel feeds to the next layer's MFMA.

    Returns (policy, action, logits): policy = head(logits) (masked to `j < mask_size` if given),
    action = discrete sample from policy with the per-row uniform `u` (None if u is None)."""
    h = np.ascontiguousarray(x, dtype=np.float32)
    n = len(weights)
    for i, w in enumerate(weights):
        b = None if biases is None else biases[i]
        h = gemm.gemm_abt(h, w, bias=b, relu=(i + 1 < n))
        if i + 1 < n and act_dtype is not None:
            h = gemm.round_to(h, act_dtype)
    logits = h
    if head == HEAD_NONE:
        policy = logits
    elif head == HEAD_SOFTMAX:
        policy = row_ops.softmax(logits) if mask_size is None else row_ops.masked_softmax(logits, mask_size)
    elif head == HEAD_REGRET_MATCHING:
        policy = row_ops.regret_matching(logits) if mask_size is None else \
            row_ops.masked_regret_matching(logits, mask_size)
    elif head == HEAD_SOFTMAX_RM:
        sm = row_ops.softmax(logits) if mask_size is None else row_ops.masked_softmax(logits, mask_size)
        policy = row_ops.regret_matching(sm) if mask_size is None else \
            row_ops.masked_regret_matching(sm, mask_size)
    else:
        raise ValueError(head)
    action = None if u is None else row_ops.discrete_sampling(policy, u)
    return policy, action, logits


def weight_init(rng, out_features, in_features, std=None):
    """`weight_init` (ml/layers.spi:460-463) draws N(0, 0.1); the benchmark configs override the
    standard deviation with 1/sqrt(fan_in)."""
    std = (1.0 / np.sqrt(in_features)) if std is None else std
    return (rng.standard_normal((out_features, in_features), dtype=np.float32) * np.float32(std)).astype(np.float32)
