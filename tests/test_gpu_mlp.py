"""Fused dense-stack forward on the GPU (through the C ABI) against the NumPy oracle.
Bar: policy within a relative Frobenius error of 3e-3 of the f32 oracle evaluated on the rounded
inputs; sampled actions bit-exact given the kernel's own policy and the same uniforms."""
import numpy as np
import pytest
import torch

from oracle import gemm as ogemm, layers as olayers, row_ops as orow
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu

TORCH = {"f16": torch.float16, "bf16": torch.bfloat16}
HEAD_CODE = {"softmax": olayers.HEAD_SOFTMAX, "regret_matching": olayers.HEAD_REGRET_MATCHING,
             "softmax_regret_matching": olayers.HEAD_SOFTMAX_RM, None: olayers.HEAD_NONE}


@pytest.fixture(scope="module")
def LY():
    from ml import layers
    return layers


def make_problem(rng, batch, dims, dtype):
    x = (rng.random((batch, dims[0])) < 0.2).astype(np.float32)
    ws = [ogemm.round_to(olayers.weight_init(rng, o, i), dtype) for i, o in zip(dims[:-1], dims[1:])]
    u = (1 - rng.random(batch, dtype=np.float32)).astype(np.float32)
    return x, ws, u


def check(LY, x, ws, u, dtype, head="softmax_regret_matching", mask=0, biases=None, packed=False):
    t = TORCH[dtype]
    bd = None if biases is None else [dev(b) if b is not None else None for b in biases]
    wd = [dev(w, t) for w in ws]
    pk = None
    if packed:
        pk = LY.pack_weights(wd)
        assert pk is not None and pk.buffer.numel() == LY.packed_bytes([x.shape[1]] + [w.shape[0] for w in ws])
    policy, action, logits = LY.mlp_forward(dev(x, t), wd, bd, head, dev(u), mask, True, packed=pk)
    policy, action, logits = host(policy), host(action), host(logits)
    want_p, _, want_l = olayers.mlp_forward(x, ws, biases, HEAD_CODE[head], u, None, mask or None)
    # hidden activations are rounded to the storage dtype before they feed the next MFMA: f16 keeps
    # 11 significant bits, bf16 only 8 (2^-9 relative rounding per activation and layer), so the raw
    # last-layer outputs of a bf16 stack get a looser bound; the policy keeps the 3e-3 contract
    assert ogemm.rel_frobenius(logits, want_l) < (3e-3 if dtype == "f16" else 1e-2)
    assert ogemm.rel_frobenius(policy, want_p) < 3e-3
    # against the oracle that rounds hidden activations to the storage dtype like the kernel does:
    # only summation order differs, which now and then flips a rounded activation by one ulp
    tight_p, _, tight_l = olayers.mlp_forward(x, ws, biases, HEAD_CODE[head], u, dtype, mask or None)
    assert ogemm.rel_frobenius(logits, tight_l) < 2e-4
    assert ogemm.rel_frobenius(policy, tight_p) < 2e-4
    # bit-exact action given the kernel's policy and the same uniforms
    if head is not None:
        assert (action == orow.discrete_sampling(policy, u)).all()
        assert (np.take_along_axis(policy, action[:, None].astype(np.int64), 1) > 0).all()
        if mask:
            assert (action < mask).all() and (policy[:, mask:] == 0).all()
        assert np.abs(policy.sum(axis=1) - 1).max() < 1e-5
    return policy, action


def test_config3_leduc_policy(LY):
    """The benchmark's policy-network workload: batch 16384, 32 -> 256 -> 256 -> 256 -> 3, f16, softmax head, regret-matching sampling."""
    announce("mlp config 3")
    rng = np.random.default_rng(3)
    x, ws, u = make_problem(rng, 16384, [32, 256, 256, 256, 3], "f16")
    policy, action = check(LY, x, ws, u, "f16")
    counts = np.bincount(action, minlength=3) / len(action)
    assert np.abs(counts - policy.mean(axis=0)).max() < 0.02   # sampled frequencies follow the policy


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("batch", [1, 100, 640])
def test_ragged_batches_and_dtypes(LY, dtype, batch):
    announce("mlp ragged batch=%d %s" % (batch, dtype))
    rng = np.random.default_rng(batch)
    x, ws, u = make_problem(rng, batch, [32, 256, 256, 256, 3], dtype)
    check(LY, x, ws, u, dtype)


@pytest.mark.parametrize("dims,head,mask", [([128, 64, 64], "regret_matching", 3), ([64, 64, 64], "softmax", 3),
                                            ([16, 32, 8], "softmax", 0), ([256, 256, 64], None, 0),
                                            ([32, 96, 160, 5], "softmax_regret_matching", 0), ([48, 3], "softmax", 0)])
def test_other_stacks(LY, dims, head, mask):
    """Shapes of the reference's real models: Leduc input(128) -> 64 -> 64 (3 valid) with a masked
    regret-matching head (game/leduc/model_cem.spi:47-63)."""
    announce("mlp stack %s head=%s mask=%d" % (dims, head, mask))
    rng = np.random.default_rng(len(dims) * 100 + dims[0])
    x, ws, u = make_problem(rng, 300, dims, "f16")
    if head is None:
        t = TORCH["f16"]
        policy, _, logits = LY.mlp_forward(dev(x, t), [dev(w, t) for w in ws], None, None, None, 0, True)
        want = olayers.mlp_forward(x, ws, head=olayers.HEAD_NONE, act_dtype="f16")[2]
        assert ogemm.rel_frobenius(host(policy), want) < 2e-4 and (host(policy) == host(logits)).all()
    else:
        check(LY, x, ws, u, "f16", head, mask)


@pytest.mark.parametrize("dims,head,mask,batch,dtype,with_bias", [
    ([48, 256, 256, 17], "softmax", 0, 300, "f16", True),                 # K0 not a multiple of 64, ragged head
    ([128, 256, 256, 256, 64], "softmax_regret_matching", 40, 200, "bf16", True),   # four first-layer chunks, widest head
    ([256, 256, 8], "regret_matching", 5, 130, "f16", False),             # no hidden 256 -> 256 layer at all
    ([64, 256, 256, 3], "softmax_regret_matching", 0, 20000, "f16", False),  # more rows than 4-wave workgroups cover: 8 waves
    ([16, 256, 256, 256, 256, 256, 256, 256, 4], "softmax", 0, 64, "f16", True),  # the deepest stack
    # up to one 64-row workgroup per compute unit and at most 16 outputs: hidden layers split by output features
    ([128, 256, 256, 256, 10], "softmax", 7, 300, "f16", True),           # four first-layer chunks, head staged in LDS
    ([48, 256, 256, 16], "regret_matching", 0, 130, "bf16", False),       # K0 in (32, 64], not a multiple of 32; 16 outputs
    ([32, 256, 256, 256, 256, 5], "softmax_regret_matching", 0, 16384, "bf16", True),   # every compute unit busy
])
def test_stacks_with_256_wide_hidden_layers(LY, dims, head, mask, batch, dtype, with_bias):
    """The shapes served by the two kernels for stacks whose hidden layers are all 256 wide."""
    announce("mlp h256 %s head=%s mask=%d batch=%d %s bias=%s" % (dims, head, mask, batch, dtype, with_bias))
    rng = np.random.default_rng(sum(dims) + batch)
    x, ws, u = make_problem(rng, batch, dims, dtype)
    biases = None
    if with_bias:
        biases = [rng.standard_normal(d, dtype=np.float32) * np.float32(0.1) for d in dims[1:]]
        biases[0] = None
    check(LY, x, ws, u, dtype, head, mask, biases)


def test_bias_extension(LY):
    announce("mlp biases")
    rng = np.random.default_rng(9)
    dims = [32, 64, 64, 3]
    x, ws, u = make_problem(rng, 200, dims, "bf16")
    biases = [rng.standard_normal(d, dtype=np.float32) * np.float32(0.1) for d in dims[1:]]
    biases[1] = None
    check(LY, x, ws, u, "bf16", biases=biases)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("batch,dims,head,mask", [(16384, [32, 256, 256, 256, 64], "softmax", 3),
                                                  (1000, [128, 256, 256, 64], "regret_matching", 3),
                                                  (333, [32, 256, 256, 256, 64], "softmax_regret_matching", 11),
                                                  (40000, [32, 256, 256, 32], "softmax", 16),
                                                  (257, [64, 256, 256, 6], "softmax", 5)])
def test_masked_head_without_logits(LY, dtype, batch, dims, head, mask):
    """Without the logits output a masked head is computed for its valid columns only and the rest of every policy
    row is written as zeros (a 64-wide layer with 3 valid columns is the reference's shape for a 3-action game).
    The policy must match the oracle and the run that does write the logits, the masked columns must be exact zeros
    inside a buffer of sentinels, and the action must be the one the kernel's own policy and the uniforms give."""
    announce("mlp masked head, no logits: %s %s batch=%d mask=%d %s" % (dims, head, batch, mask, dtype))
    rng = np.random.default_rng(batch + mask)
    x, ws, u = make_problem(rng, batch, dims, dtype)
    t = TORCH[dtype]
    xd, wd, ud = dev(x, t), [dev(w, t) for w in ws], dev(u)
    n = dims[-1]
    buf = torch.full((64 + batch * n + 64,), -9.0, dtype=torch.float32, device="cuda")
    policy_t = buf[64:64 + batch * n].view(batch, n)
    action_t = torch.full((batch,), -1, dtype=torch.int32, device="cuda")
    LY.mlp_forward(xd, wd, None, head, ud, mask, False, policy_out=policy_t, action_out=action_t)
    raw = host(buf)
    assert (raw[:64] == -9).all() and (raw[-64:] == -9).all()
    policy, action = raw[64:-64].reshape(batch, n), host(action_t)
    full_p, full_a, _ = LY.mlp_forward(xd, wd, None, head, ud, mask, True)
    want_p, _, _ = olayers.mlp_forward(x, ws, None, HEAD_CODE[head], u, dtype, mask)
    assert (policy[:, mask:] == 0).all() and np.abs(policy.sum(axis=1) - 1).max() < 1e-5
    assert ogemm.rel_frobenius(policy, want_p) < 2e-4 and ogemm.rel_frobenius(policy, host(full_p)) < 2e-4
    assert (action == orow.discrete_sampling(policy, u)).all() and (action < mask).all() and (action >= 0).all()


@pytest.mark.parametrize("dims,head,mask,batch,dtype,with_bias", [
    ([32, 256, 256, 256, 3], "softmax_regret_matching", 0, 16384, "f16", False),     # the benchmark's policy network
    ([32, 256, 256, 256, 3], "softmax", 0, 1, "bf16", False),                        # a single row
    ([32, 256, 256, 3], "softmax_regret_matching", 0, 100, "f16", True),             # three layers
    ([32, 256, 256, 256, 256, 5], "softmax_regret_matching", 0, 333, "bf16", True),  # five layers: refills into both register sets
    ([48, 256, 256, 16], "regret_matching", 0, 130, "bf16", False),                  # two first-layer k-steps, K0 not a multiple of 32
    ([64, 256, 256, 256, 256, 9], "softmax", 7, 640, "f16", True),                   # two first-layer k-steps, five layers, masked head with logits
    ([128, 256, 256, 256, 10], "softmax", 7, 300, "f16", True),                      # eight first-layer k-steps (zero-padded K0)
    ([256, 256, 256, 8], "regret_matching", 5, 130, "f16", False),                   # a full-width first layer, three layers
    ([256, 256, 256, 256, 256, 16], "softmax", 0, 64, "bf16", True),                 # full-width first layer, five layers, widest head
    ([32, 256, 256, 256, 3], "softmax_regret_matching", 0, 20000, "f16", False),     # more workgroups than compute units
    ([32, 256, 256, 256, 3], "softmax", 0, 200, "f16", "all"),                        # a bias on every layer
    ([256, 256, 256, 256, 256, 12], "softmax", 0, 200, "bf16", "all"),
    ([64, 256, 256, 256, 4], "regret_matching", 0, 77, "f16", "only1"),               # a bias on the second layer alone
])
def test_packed_weights_kernel(LY, dims, head, mask, batch, dtype, with_bias):
    """The kernel that streams pre-packed weights straight into registers (sp_mlp_pack_weights +
    sp_mlp_forward_packed) against the oracle, and against sp_mlp_forward on the row-major weights."""
    announce("mlp packed %s head=%s mask=%d batch=%d %s bias=%s" % (dims, head, mask, batch, dtype, with_bias))
    rng = np.random.default_rng(sum(dims) + batch + 1)
    x, ws, u = make_problem(rng, batch, dims, dtype)
    biases = None
    if with_bias:
        biases = [rng.standard_normal(d, dtype=np.float32) * np.float32(0.1) for d in dims[1:]]
        if with_bias == "only1":
            biases = [b if l == 1 else None for l, b in enumerate(biases)]
        elif with_bias != "all":
            biases[1] = None
    policy, action = check(LY, x, ws, u, dtype, head, mask, biases, packed=True)
    t = TORCH[dtype]
    bd = None if biases is None else [dev(b) if b is not None else None for b in biases]
    plain_p, plain_a = LY.mlp_forward(dev(x, t), [dev(w, t) for w in ws], bd, head, dev(u), mask)
    assert ogemm.rel_frobenius(policy, host(plain_p)) < 2e-4
    assert (action != host(plain_a)).mean() < 1e-3      # same uniforms, policies equal to rounding


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_packed_masked_head_without_logits(LY, dtype):
    """A 64-wide output layer under a 3-column mask (the reference's shape for a 3-action game) on the packed
    kernel: only the valid columns are computed, the rest of each policy row is exact zeros inside sentinels."""
    announce("mlp packed masked head, no logits " + dtype)
    batch, dims, mask = 4100, [32, 256, 256, 256, 64], 3
    rng = np.random.default_rng(77)
    x, ws, u = make_problem(rng, batch, dims, dtype)
    t = TORCH[dtype]
    xd, wd, ud = dev(x, t), [dev(w, t) for w in ws], dev(u)
    pk = LY.pack_weights(wd)
    buf = torch.full((64 + batch * 64 + 64,), -9.0, dtype=torch.float32, device="cuda")
    policy_t = buf[64:64 + batch * 64].view(batch, 64)
    action_t = torch.full((batch,), -1, dtype=torch.int32, device="cuda")
    LY.mlp_forward(xd, None, None, "softmax", ud, mask, False, policy_out=policy_t, action_out=action_t, packed=pk)
    raw = host(buf)
    assert (raw[:64] == -9).all() and (raw[-64:] == -9).all()
    policy, action = raw[64:-64].reshape(batch, 64), host(action_t)
    want_p, _, _ = olayers.mlp_forward(x, ws, None, HEAD_CODE["softmax"], u, dtype, mask)
    assert (policy[:, mask:] == 0).all() and np.abs(policy.sum(axis=1) - 1).max() < 1e-5
    assert ogemm.rel_frobenius(policy, want_p) < 2e-4
    assert (action == orow.discrete_sampling(policy, u)).all() and (action < mask).all() and (action >= 0).all()
    # the logits of a wide masked layer are more than the packed kernel computes: the call says so
    from ml import _lib
    with pytest.raises(_lib.SpiralError, match="UNSUPPORTED"):
        LY.mlp_forward(xd, None, None, "softmax", ud, mask, True, packed=pk)


def test_packing_is_refused_for_other_stacks(LY):
    announce("mlp packed: unsupported stacks")
    t = torch.float16
    mk = lambda dims: [torch.zeros((o, i), dtype=t, device="cuda") for i, o in zip(dims[:-1], dims[1:])]
    assert LY.pack_weights(mk([32, 64, 64, 3])) is None                  # hidden width other than 256
    assert LY.pack_weights(mk([32, 256, 3])) is None                     # two layers
    assert LY.pack_weights(mk([32] + [256] * 6 + [3])) is None           # deeper than the packed kernel goes
    assert LY.packed_bytes([32, 256, 256, 256, 3]) == 4 * 4096 + 2 * 131072 + 8192


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("dims,mask,with_bias", [([32, 256, 256, 256, 3], 0, False), ([32, 256, 256, 256, 64], 3, False),
                                                 ([256, 256, 256, 16], 0, True), ([64, 128, 96, 8], 0, False)])
def test_results_do_not_change_from_run_to_run(LY, dims, mask, with_bias, packed):
    """Three launches on the same inputs give the same bits, for every fused kernel (hand-issued MFMAs and loads
    counted by hand: a wait that is one short, or a register overwritten too early, shows up as results that
    differ between launches)."""
    announce("mlp run-to-run dims=%s packed=%s" % (dims, packed))
    rng = np.random.default_rng(23)
    x, ws, u = make_problem(rng, 16384, dims, "f16")
    wd = [dev(w, torch.float16) for w in ws]
    bd = [dev(rng.standard_normal(w.shape[0], dtype=np.float32)) for w in ws] if with_bias else None
    pk = LY.pack_weights(wd) if packed else None
    if packed and pk is None:
        pytest.skip("this stack has no packed form")
    xd, ud = dev(x, torch.float16), dev(u)
    logits = not (packed and mask)        # the packed kernel computes a masked head for its valid columns only
    first = [t.clone() for t in LY.mlp_forward(xd, wd, bd, "softmax_regret_matching", ud, mask, logits, packed=pk) if t is not None]
    for _ in range(2):
        again = [t for t in LY.mlp_forward(xd, wd, bd, "softmax_regret_matching", ud, mask, logits, packed=pk) if t is not None]
        assert len(first) == len(again)
        for a, b in zip(first, again):
            assert torch.equal(a, b)



@pytest.mark.parametrize("dims,mask,batch,want_logits,packed,mode", [
    ([32, 96, 160, 8], 0, 24 * 13, False, False, "layer"),               # the general kernel
    ([128, 256, 256, 64], 40, 24 * 9, True, False, "layer"),             # 256-wide hidden layers, wide head
    ([32, 256, 256, 256, 64], 3, 16384, False, False, "layer"),          # feature-split kernel, head of 3 valid columns of 64
    ([32, 256, 256, 256, 64], 3, 16384, False, True, "layer"),           # the same on packed weights
    ([32, 256, 256, 256, 4], 0, 1000, False, True, "block"),             # packed, plain head, the block-level stream
    ([64, 256, 256, 16], 0, 40000, False, False, "grid"),                # more rows than one round of workgroups
])
def test_head_draws_its_own_uniforms(LY, dims, mask, batch, want_logits, packed, mode):
    """A head given a Philox stream instead of a tensor of uniforms (the reference seeds one generator per thread
    and the sampling node draws in the kernel, ml/layers.spi:339-344): every row must use exactly the uniform
    sp_philox_uniforms hands out for it -- same policy bits, same actions as the run that reads those uniforms
    from a tensor -- and those uniforms are the stream the golden sampled indices pin."""
    from ml import _lib, primitives
    from oracle import philox as ophilox
    announce("mlp philox head dims=%s mask=%d batch=%d packed=%s mode=%s" % (dims, mask, batch, packed, mode))
    rng = np.random.default_rng(sum(dims) + batch)
    x, ws, _ = make_problem(rng, batch, dims, "f16")
    xd, wd = dev(x, torch.float16), [dev(w, torch.float16) for w in ws]
    pk = LY.pack_weights(wd) if packed else None
    cols = dims[-1]
    if mode == "layer":
        q = 24 if batch % 24 == 0 else 32
        cfg = primitives.philox(_lib.PHILOX_LAYER, blocks_per_grid=q, rows_per_block=batch // q, offset=8)
        want_u = ophilox.row_uniforms_layer(q, batch // q, cols, offset=8)
    elif mode == "block":
        cfg = primitives.philox(_lib.PHILOX_BLOCK)
        want_u = ophilox.row_uniforms_block(batch, cols)
    else:
        cfg = primitives.philox(_lib.PHILOX_GRID, blocks_per_grid=24)
        want_u = ophilox.row_uniforms_grid(batch, cols, blocks=24)
    u = primitives.philox_uniforms(cfg, batch, cols)
    assert (host(u) == np.asarray(want_u, dtype=np.float32).reshape(-1)).all()
    head = "softmax_regret_matching"
    with_u = LY.mlp_forward(xd, wd, None, head, u, mask, want_logits, packed=pk)
    with_rng = LY.mlp_forward(xd, wd, None, head, None, mask, want_logits, packed=pk, rng=cfg)
    for a, b in zip(with_u, with_rng):
        assert torch.equal(a, b)
    assert (host(with_rng[1]) == orow.discrete_sampling(host(with_rng[0]), host(u))).all()


@pytest.mark.parametrize("dims,head,mask,batch,dtype,with_bias,packed", [
    ([32, 256, 256, 256, 3], "softmax_regret_matching", 0, 100000, "f16", False, True),   # the benchmark's network, ragged last pair
    ([32, 256, 256, 256, 3], "softmax_regret_matching", 0, 133000, "f16", False, False),  # ... from the row-major weights
    ([32, 256, 256, 256, 3], "softmax", 0, 300000, "bf16", "all", True),                  # 18 tiles per compute unit
    ([16, 256, 256, 4], "softmax_regret_matching", 0, 132000, "f16", True, False),        # three layers, a 16-wide first layer
    ([48, 256, 256, 256, 16], "softmax", 0, 131100, "bf16", True, False),                 # two first-layer k-steps, K0 not a multiple of 32, 16 outputs
    ([64, 256, 256, 12], "softmax", 7, 98400, "f16", "only1", True),                      # masked head with logits, head staged in LDS
    ([32, 256, 256, 256, 2], "softmax_regret_matching", 0, 98304 + 65, "bf16", False, True),   # one row in the second tile of the last pair
    ([64, 256, 256, 256, 4], "softmax_regret_matching", 0, 131072 + 31, "f16", "all", False),  # pipelined form: two first-layer k-steps, every bias, row-major
    ([48, 256, 256, 256, 8], "softmax", 3, 99000, "bf16", True, True),                          # pipelined form: 3 of 8 columns valid, zeros behind them
    ([32, 256, 256, 256, 3], "softmax_regret_matching", 0, 98304 + 32 * 256 * 9 + 5, "f16", False, True),  # a last head pass of one tile on some units
    ([32, 256, 256, 256, 3], "softmax_regret_matching", 0, 65536 + 7, "f16", False, True),      # the smallest batch the pipelined form takes, packed
    ([32, 256, 256, 256, 3], "softmax_regret_matching", 0, 81920 + 33, "f16", False, False),    # ... and from row-major weights
])
def test_weights_resident_in_registers(LY, dims, head, mask, batch, dtype, with_bias, packed):
    """Batches of several 64-row tiles per compute unit run on the kernels that load the weights once and keep them in
    registers while they walk over their tiles (from six tiles per unit with packed weights, from eight with row-major
    ones; the pipelined form of four-layer stacks from four and five): against the oracle like every other kernel, and against the per-tile packed kernel run on the same rows in
    slices small enough to stay on that kernel (same operand layout; the same order of the sums except in the output
    layer of the pipelined form)."""
    announce("mlp resident %s head=%s mask=%d batch=%d %s bias=%s packed=%s" % (dims, head, mask, batch, dtype, with_bias, packed))
    rng = np.random.default_rng(sum(dims) + batch + 7)
    x, ws, u = make_problem(rng, batch, dims, dtype)
    biases = None
    if with_bias:
        biases = [rng.standard_normal(d, dtype=np.float32) * np.float32(0.1) for d in dims[1:]]
        if with_bias == "only1":
            biases = [b if l == 1 else None for l, b in enumerate(biases)]
        elif with_bias != "all":
            biases[1] = None
    policy, action = check(LY, x, ws, u, dtype, head, mask, biases, packed=packed)
    t = TORCH[dtype]
    wd = [dev(w, t) for w in ws]
    bd = None if biases is None else [dev(b) if b is not None else None for b in biases]
    pk = LY.pack_weights(wd)
    # four-layer stacks with at most 4 outputs take the pipelined form, whose output layer adds its k-steps slice by
    # slice: equal to the per-tile kernel to rounding; the others add in the per-tile kernel's order: equal bit for bit
    pipelined = len(dims) == 5 and (mask or dims[-1]) <= 4
    # the call that asks for no logits is another instance of the kernel: the same bits -- unless only that call can
    # leave the masked columns out of the output layer and so comes to run on the pipelined form
    p, a = LY.mlp_forward(dev(x, t), wd, bd, head, dev(u), mask, packed=pk if packed else None)
    if pipelined and mask:
        assert ogemm.rel_frobenius(policy, host(p)) < 2e-5 and (host(a) != action).mean() < 1e-3
        assert (host(a) == orow.discrete_sampling(host(p), u)).all() and (host(p)[:, mask:] == 0).all()
    else:
        assert (host(p) == policy).all() and (host(a) == action).all()
    step = 16384
    for lo in range(0, batch, step):
        hi = min(batch, lo + step)
        p, a = LY.mlp_forward(dev(x[lo:hi], t), None, bd, head, dev(u[lo:hi]), mask, packed=pk)
        if pipelined:
            assert ogemm.rel_frobenius(policy[lo:hi], host(p)) < 2e-5, lo
            assert (host(a) != action[lo:hi]).mean() < 1e-3, lo
        else:
            assert (host(p) == policy[lo:hi]).all() and (host(a) == action[lo:hi]).all(), lo


def test_resident_kernel_run_to_run_and_philox(LY):
    """The resident kernel gives the same bits on every launch, and with a Philox stream in place of the uniforms tensor
    it draws for every tile of its walk what sp_philox_uniforms hands out for those rows."""
    from ml import _lib, primitives
    announce("mlp resident run-to-run + philox")
    rng = np.random.default_rng(41)
    batch, dims = 24 * 5632, [32, 256, 256, 256, 64]
    x, ws, _ = make_problem(rng, batch, dims, "f16")
    xd, wd = dev(x, torch.float16), [dev(w, torch.float16) for w in ws]
    pk = LY.pack_weights(wd)
    cfg = primitives.philox(_lib.PHILOX_LAYER, blocks_per_grid=24, rows_per_block=5632)
    u = primitives.philox_uniforms(cfg, batch, 64)
    for packed in (pk, None):
        first = [t.clone() for t in LY.mlp_forward(xd, wd, None, "softmax", u, 3, packed=packed)]
        for _ in range(2):
            again = LY.mlp_forward(xd, wd, None, "softmax", u, 3, packed=packed)
            assert all(torch.equal(a, b) for a, b in zip(first, again))
        drawn = LY.mlp_forward(xd, wd, None, "softmax", None, 3, packed=packed, rng=cfg)
        assert all(torch.equal(a, b) for a, b in zip(first, drawn))
        assert (host(first[1]) == orow.discrete_sampling(host(first[0]), host(u))).all()


@pytest.mark.parametrize("members,batch,dims,head,mask,sample", [
    (32, 6144, [128, 64, 64], "regret_matching", 3, None),      # the reference's Leduc policy: 3 valid of 64 columns, no sampling
    (5, 1000, [128, 64, 64], "softmax", 3, "u"),                 # ragged last tile, uniforms from a tensor
    (3, 4100, [64, 64, 4], "softmax_regret_matching", 0, "u"),   # a head 4 wide, no mask: dense rows
    (7, 777, [24, 64, 6], "regret_matching", 2, "philox"),       # K0 not a multiple of 32, row width not a multiple of 4
    (300, 64, [8, 64, 64], "softmax", 4, "philox"),              # more members than compute units
])
def test_ensemble_forward(LY, members, batch, dims, head, mask, sample):
    """sp_mlp_forward_ensemble -- every member's relu(x.W1^T).W2^T + head in one launch -- against the oracle's
    forward of each member on its own (f32: relative Frobenius error below 1e-5, the f32 bar), zeros behind the
    mask, and actions bit-exact given the kernel's own policy and the member's uniforms."""
    from ml import _lib, primitives
    from oracle import philox as ophilox
    announce("mlp ensemble members=%d batch=%d dims=%s head=%s mask=%d sample=%s" % (members, batch, dims, head, mask, sample))
    rng = np.random.default_rng(members * 1000 + batch)
    x = rng.standard_normal((batch, dims[0]), dtype=np.float32)
    w1 = rng.standard_normal((members, dims[1], dims[0]), dtype=np.float32) * np.float32(1 / np.sqrt(dims[0]))
    w2 = rng.standard_normal((members, dims[2], dims[1]), dtype=np.float32) * np.float32(1 / np.sqrt(dims[1]))
    u, cfg = None, None
    if sample == "u":
        u = (1 - rng.random((members, batch), dtype=np.float32)).astype(np.float32)
    elif sample == "philox":
        # the stacked rows of the members, each member a run of its own `member_draws` further into every thread's stream
        cols = dims[2] if dims[2] % 4 == 0 else 8
        cfg = primitives.philox(_lib.PHILOX_LAYER, blocks_per_grid=1, rows_per_block=batch, member_rows=batch, member_draws=12)
        u = host(primitives.philox_uniforms(cfg, members * batch, cols)).reshape(members, batch)
        if dims[2] % 4 != 0:
            sample = "u"          # (a Philox stream needs 16-byte rows: such a head takes the same numbers as a tensor)
    out = LY.mlp_forward_ensemble(dev(x), (dev(w1), dev(w2)), head, dev(u) if sample == "u" else None, mask,
                                  rng=cfg if sample == "philox" else None)
    policy, action = (host(out[0]), host(out[1])) if sample else (host(out), None)
    assert policy.shape == (members, batch, dims[2])
    for e in range(members):
        want, _, _ = olayers.mlp_forward(x, [w1[e], w2[e]], None, HEAD_CODE[head], None, None, mask or None)
        assert ogemm.rel_frobenius(policy[e], want) < 1e-5, e
        if mask:
            assert (policy[e][:, mask:] == 0).all()
        assert np.abs(policy[e].sum(axis=1) - 1).max() < 1e-5
        if sample:
            assert (action[e] == orow.discrete_sampling(policy[e], u[e])).all(), e
    if sample:
        assert len(np.unique(action)) > 1


def test_ensemble_rejects_what_it_does_not_take(LY):
    from ml import _lib
    x = torch.zeros((64, 128), dtype=torch.float32, device="cuda")
    w1 = torch.zeros((2, 64, 128), dtype=torch.float32, device="cuda")
    with pytest.raises(_lib.SpiralError) as err:      # 64 computed outputs: left to the node-by-node pass
        LY.mlp_forward_ensemble(x, (w1, torch.zeros((2, 64, 64), dtype=torch.float32, device="cuda")), "softmax")
    assert err.value.code == -2
    with pytest.raises(_lib.SpiralError) as err:      # a hidden layer of another width
        LY.mlp_forward_ensemble(x, (torch.zeros((2, 32, 128), dtype=torch.float32, device="cuda"),
                                    torch.zeros((2, 4, 32), dtype=torch.float32, device="cuda")), "softmax")
    assert err.value.code == -2


@pytest.mark.parametrize("members,batch,k0,n,head,mask,sample", [
    (4, 6144, 128, 64, "regret_matching", 3, None),     # the reference's hold'em CEM policy: one layer, 3 valid of 64 columns
    (6, 1000, 256, 64, "softmax", 4, "u"),              # the widest input, a ragged last tile, sampling
    (3, 333, 40, 3, "softmax_regret_matching", 0, "u"),  # input width not a multiple of 32, a dense 3-wide head
])
def test_single_layer_ensemble_forward(LY, members, batch, k0, n, head, mask, sample):
    """sp_mlp_forward_ensemble with ONE layer per member (policy[e] = head(x . W[e]^T), only the head's valid columns
    computed) against the oracle's forward of each member (f32 bar 1e-5), zeros behind the mask, actions exact given
    the kernel's policy."""
    announce("ensemble single layer members=%d batch=%d k0=%d n=%d head=%s mask=%d" % (members, batch, k0, n, head, mask))
    rng = np.random.default_rng(members + batch + k0)
    x = rng.standard_normal((batch, k0), dtype=np.float32)
    w = rng.standard_normal((members, n, k0), dtype=np.float32) * np.float32(1 / np.sqrt(k0))
    u = (1 - rng.random((members, batch), dtype=np.float32)).astype(np.float32) if sample else None
    out = LY.mlp_forward_ensemble(dev(x), (dev(w),), head, dev(u) if sample else None, mask)
    policy, action = (host(out[0]), host(out[1])) if sample else (host(out), None)
    for e in range(members):
        want, _, _ = olayers.mlp_forward(x, [w[e]], None, HEAD_CODE[head], None, None, mask or None)
        assert ogemm.rel_frobenius(policy[e], want) < 1e-5, e
        if mask:
            assert (policy[e][:, mask:] == 0).all()
        if sample:
            assert (action[e] == orow.discrete_sampling(policy[e], u[e])).all(), e


@pytest.mark.parametrize("members,batch,k0,n,modulo", [
    (4, 6144, 128, 128, 1 << 12),     # the reference's CFR models: 128 outputs hashed into 4096 worlds
    (5, 1001, 256, 20, 1000003),      # fewer than 32 columns, a modulus that is not a power of two, a ragged last tile
    (3, 64, 24, 40, 1 << 31),         # every one of the 32 counted bits kept
])
def test_ensemble_binarize(LY, members, batch, k0, n, modulo):
    """sp_ensemble_binarize (one ensemble layer + the hash head, the product never written) against the oracle's
    binarize of the oracle's product.  A bit can only differ where an output is so close to zero that the order of the
    sum decides its sign: such entries are left out of the comparison (and are counted: there must be next to none)."""
    from ml import primitives
    announce("ensemble binarize members=%d batch=%d k0=%d n=%d modulo=%d" % (members, batch, k0, n, modulo))
    rng = np.random.default_rng(members * 7 + batch + n)
    x = rng.standard_normal((batch, k0), dtype=np.float32)
    w = rng.standard_normal((members, n, k0), dtype=np.float32)
    got = host(LY.ensemble_binarize(dev(x), dev(w), modulo)).view(np.uint32)
    assert got.shape == (members, batch)
    close = 0
    for e in range(members):
        y = ogemm.gemm_abt(x, w[e])
        want = orow.binarize(y, modulo)
        sure = (np.abs(y[:, :32]) > 1e-4).all(axis=1)       # rows whose counted outputs are all clear of zero
        close += int((~sure).sum())
        assert (got[e][sure] == want[sure]).all(), e
        # and exactly the node-by-node result on the same product computed by the library's own GEMM
    assert close < 0.02 * members * batch
    # the row kernel on the library's own product gives the same words wherever the signs are not in question
    from ml import matmul
    y0 = matmul.matmul_abt(dev(x), dev(w[0]))
    node = host(primitives.binarize(y0, modulo)).view(np.uint32)
    sure0 = (np.abs(host(y0)[:, :32]) > 1e-4).all(axis=1)
    assert (node[sure0] == got[0][sure0]).all()
