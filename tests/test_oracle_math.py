"""Checks that pin the oracle where the reference holds no vectors: known-answer vectors of the
published algorithm, closed forms, brute force on tiny inputs and invariants."""
import numpy as np
import pytest

from oracle import gemm, layers, philox, row_ops


def test_philox_known_answers():
    # Random123 kat_vectors, philox4x32 with 10 rounds
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
        ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
        ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
         (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
    ]
    for ctr, key, want in kat:
        got = philox.philox4x32_10(np.array(ctr, dtype=np.uint32), np.array(key, dtype=np.uint32))
        assert tuple(int(v) for v in got) == want


def test_curand_uniform_range():
    u = philox.curand_uniform(np.array([0, 1, 0x7fffffff, 0xffffffff], dtype=np.uint32))
    assert u[0] > 0 and u[-1] == 1.0 and (np.diff(u) >= 0).all()


def test_gemm_bruteforce_and_algebra():
    rng = np.random.default_rng(0)
    a = rng.standard_normal((16, 8), dtype=np.float32)
    b = rng.standard_normal((16, 8), dtype=np.float32)
    c = rng.standard_normal((16, 16), dtype=np.float32)
    for alpha, beta in ((1.0, 0.0), (1.0, 1.0), (0.5, -2.0)):
        want = gemm.gemm_abt_bruteforce(a, b, c, alpha, beta)
        got = gemm.gemm_abt(a, b, c, alpha, beta)
        assert gemm.rel_frobenius(got, want) < 1e-6
    # a transposed operand or a swapped A/B must fail: B = identity gives C = A, not A^T
    a2 = rng.standard_normal((8, 8), dtype=np.float32)
    assert (gemm.gemm_abt(a2, np.eye(8, dtype=np.float32)) == a2).all()
    # non-square: C[i, j] = <A_i, B_j>
    a3 = np.arange(6, dtype=np.float32).reshape(2, 3)
    b3 = np.arange(12, dtype=np.float32).reshape(4, 3)
    assert (gemm.gemm_abt(a3, b3) == np.array([[5, 14, 23, 32], [14, 50, 86, 122]], dtype=np.float32)).all()
    # NaNs in C do not propagate when beta == 0 (ml/matmul/kernel.spi:152-154)
    assert np.isfinite(gemm.gemm_abt(a, b, np.full((16, 16), np.nan, dtype=np.float32), 1.0, 0.0)).all()
    with pytest.raises(AssertionError):
        gemm.gemm_abt(a, b, alpha=0.0)


def test_gemm_integer_inputs_exact():
    # the reference's commented `arange` alternative (ml/matmul/run.spi:52): integer results are exact
    a = (np.arange(32 * 16) % 7).astype(np.float32).reshape(32, 16)
    b = (np.arange(24 * 16) % 5).astype(np.float32).reshape(24, 16)
    want = (a.astype(np.int64) @ b.astype(np.int64).T)
    assert (gemm.gemm_abt(a, b).astype(np.int64) == want).all()


def test_bf16_rounding():
    x = np.array([1.0, 1.00390625, 1.01171875, -2.5, 3.0e38, 1e-40, np.inf], dtype=np.float32)
    bits = gemm.f32_to_bf16_bits(x)
    back = gemm.bf16_bits_to_f32(bits)
    assert back[0] == 1.0 and back[3] == -2.5 and np.isinf(back[-1])
    # 1 + 2^-8 is a tie between 1.0 and 1 + 2^-7: RNE picks the even mantissa (1.0)
    assert back[1] == 1.0
    # 1 + 3*2^-8 is a tie between 1+2^-7 (odd) and 1+2^-6 (even)
    assert back[2] == np.float32(1.015625)
    import torch
    t = torch.from_numpy(np.random.default_rng(1).standard_normal(4096).astype(np.float32))
    want = t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (gemm.f32_to_bf16_bits(t.numpy()) == want).all()
    assert np.isnan(gemm.bf16_bits_to_f32(gemm.f32_to_bf16_bits(np.array([np.nan], dtype=np.float32)))).all()


def test_tile_heuristic_matches_generated_code():
    # ml/matmul/run.py (96 KB build): 128x128x64 tiles (ldm 136 = 128 + 8); 224 KB: 128x256x64
    assert gemm.matmul_tile_config(8192, 8192, 4096, 96 * 1024) == (128, 128, 64)
    assert gemm.matmul_tile_config(8192, 8192, 4096, 224 * 1024) == (128, 256, 64)
    assert gemm.matmul_tile_config(16, 16, 8) == (16, 16, 8)
    with pytest.raises(AssertionError):
        gemm.matmul_tile_config(16384, 3, 256)


def test_softmax_invariants():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((64, 256)) * 2).astype(np.float32)
    p = row_ops.softmax(x)
    assert np.abs(p.sum(axis=1) - 1).max() < 1e-5
    assert np.abs(row_ops.softmax(x + 3.0) - p).max() < 1e-6
    assert np.abs(row_ops.softmax(x, "mean") - p).max() < 1e-6
    assert (row_ops.masked_softmax(x, 256) == p).all()
    m, s = row_ops.softmax_stats(x)
    assert (m == x.max(axis=1)).all() and np.allclose(np.exp(x - m[:, None]) / s[:, None], p, rtol=1e-6)


def test_regret_matching_closed_forms():
    x = np.array([[1, -1, 3, 0], [-1, -2, -3, -4], [0, 0, 0, 0], [2, 2, 0, -5]], dtype=np.float32)
    want = np.array([[.25, 0, .75, 0], [.25] * 4, [.25] * 4, [.5, .5, 0, 0]], dtype=np.float32)
    assert (row_ops.regret_matching(x) == want).all()
    assert (row_ops.masked_regret_matching(x, 4) == want).all()
    m = row_ops.masked_regret_matching(x, 2)
    assert (m == np.array([[1, 0, 0, 0], [.5, .5, 0, 0], [.5, .5, 0, 0], [.5, .5, 0, 0]], dtype=np.float32)).all()


def test_scan_orders():
    rng = np.random.default_rng(3)
    for cols in (4, 12, 16, 64, 128, 256, 260, 512, 1024):
        xi = rng.integers(-1000, 1000, size=(7, cols)).astype(np.int32)
        assert (row_ops._wave_scan(xi, True) == np.cumsum(xi, axis=1)).all()
        assert (row_ops._wave_scan(xi, False) == np.cumsum(xi, axis=1) - xi).all()
        xf = rng.random((7, cols), dtype=np.float32)
        seq = row_ops.inclusive_scan_sum(xf, "sequential")
        wav = row_ops.inclusive_scan_sum(xf, "wave")
        assert np.abs(seq - wav).max() <= 1e-6 * cols
        # brute-force sequential reading
        acc = np.float32(0)
        for j in range(cols):
            acc = np.float32(acc + xf[0, j])
            assert acc == seq[0, j]


def test_discrete_sampling_invariants():
    rng = np.random.default_rng(4)
    p = row_ops.softmax((rng.standard_normal((200, 64)) * 2).astype(np.float32))
    p[:, ::3] = 0  # zero-probability entries must never be selected
    u = (1 - rng.random(200, dtype=np.float32)).astype(np.float32)
    idx = row_ops.discrete_sampling(p, u)
    assert (np.take_along_axis(p, idx[:, None].astype(np.int64), 1) > 0).all()
    tiny = np.full(200, np.float32(1e-30))
    first = np.argmax(p > 0, axis=1)
    last = p.shape[1] - 1 - np.argmax(p[:, ::-1] > 0, axis=1)
    assert (row_ops.discrete_sampling(p, tiny) == first).all()
    assert (row_ops.discrete_sampling(p, np.ones(200, dtype=np.float32)) == last).all()
    # monotone in u
    us = np.sort(rng.random(50, dtype=np.float32))[::-1].copy()
    one = np.repeat(p[:1], 50, axis=0)
    assert (np.diff(row_ops.discrete_sampling(one, 1 - us)) >= 0).all()
    # brute force
    for r in range(20):
        cdf = np.cumsum(p[r], dtype=np.float32)
        m = max(cdf[j] for j in range(64) if p[r, j] > 0)
        thr = np.float32(u[r] * m)
        want = min(j for j in range(64) if p[r, j] > 0 and np.float32(cdf[j] - thr) >= 0)
        assert idx[r] == want
    assert row_ops.discrete_sampling(np.zeros((1, 8), np.float32), np.ones(1, np.float32))[0] == row_ops.INT_MAX


def test_mlp_forward_composition():
    rng = np.random.default_rng(5)
    x = (rng.random((32, 32)) < 0.2).astype(np.float32)
    ws = [gemm.round_to(layers.weight_init(rng, o, i), "f16") for o, i in ((256, 32), (256, 256), (256, 256), (3, 256))]
    u = (1 - rng.random(32, dtype=np.float32)).astype(np.float32)
    policy, action, logits = layers.mlp_forward(x, ws, u=u)
    h = x
    for w in ws[:-1]:
        h = np.maximum(h.astype(np.float64) @ w.astype(np.float64).T, 0)
    want_logits = h @ ws[-1].astype(np.float64).T
    assert gemm.rel_frobenius(logits, want_logits) < 1e-5
    e = np.exp(want_logits - want_logits.max(axis=1, keepdims=True))
    assert np.abs(policy - e / e.sum(axis=1, keepdims=True)).max() < 1e-5
    assert ((action >= 0) & (action < 3)).all()
    pol16, _, _ = layers.mlp_forward(x, ws, u=u, act_dtype="f16")
    assert gemm.rel_frobenius(pol16, policy) < 3e-3


def test_binarize_and_get_prob_by_hand():
    x = np.array([[0.5, -1.0, 0.0, 2.0], [-1, -1, -1, -1], [1, 1, 1, 1]], dtype=np.float32)
    assert row_ops.binarize(x, 100).tolist() == [0b1001, 0, 0b1111]
    assert row_ops.binarize(x, 4).tolist() == [0b1001 % 4, 0, 0b1111 % 4]
    wide = np.ones((1, 40), dtype=np.float32)          # columns 32.. are shifted out
    assert row_ops.binarize(wide, 2 ** 32 - 1).tolist() == [0]   # 0xFFFFFFFF mod 0xFFFFFFFF
    assert row_ops.binarize(wide, 2 ** 31).tolist() == [2 ** 31 - 1]
    # the reference's bit test is `not (x <= 0)`: a NaN sets its bit, -0.0 and -inf do not
    odd = np.array([[np.nan, -0.0, np.inf, -np.inf]], dtype=np.float32)
    assert row_ops.binarize(odd, 100).tolist() == [0b0101]
    p = np.array([[0.1, 0.2, 0.7], [0.3, 0.3, 0.4]], dtype=np.float32)
    assert row_ops.get_prob(p, [2, 0]).tolist() == [np.float32(0.7), np.float32(0.3)]


def test_chosen_edge_semantics_of_argmax_and_softmax():
    """Where this build fixes what the reference leaves open (or does differently), the choice is pinned here:
    argmax ties go to the LOWEST index (the reference's `if a > b then a else b` keeps the later operand inside a
    thread and is order-dependent across threads), a row of NaNs gives index 0, and softmax shifts by the row max,
    so it stays finite where the reference's shift by the mean overflows."""
    x = np.array([[1, 3, 3, 2], [5, 5, 5, 5], [-1, -7, -1, -1]], dtype=np.float32)
    assert row_ops.argmax(x).tolist() == [1, 0, 0]
    assert row_ops.argmax(np.full((1, 8), np.nan, dtype=np.float32)).tolist() == [0]
    big = np.array([[0, 0, 0, 200.0]], dtype=np.float32)      # exp(200 - mean 50) overflows f32, exp(200 - 200) does not
    with np.errstate(over="ignore", invalid="ignore"):
        assert not np.isfinite(row_ops.softmax(big, shift="mean")).all()
    assert np.isfinite(row_ops.softmax(big)).all() and row_ops.softmax(big)[0, 3] == 1.0
    small = np.array([[0.5, -1.0, 2.0, 0.0]], dtype=np.float32)
    assert np.allclose(row_ops.softmax(small), row_ops.softmax(small, shift="mean"), rtol=1e-6)


def test_layer_stream_reduces_to_block_stream_and_shifts_by_offset():
    one_block = philox.row_uniforms_layer(1, 96, 64)
    assert (one_block == philox.row_uniforms_block(96, 64)).all()
    # every block restarts the row walk and uses its own 256 subsequences
    u = philox.row_uniforms_layer(3, 32, 64)
    want = philox.curand_uniform(philox.curand_words(philox.CONSTANT_SEED,
                                                     np.repeat(np.arange(3), 32) * 256 + (np.tile(np.arange(32), 3) % 16) * 16,
                                                     4 * (np.tile(np.arange(32), 3) // 16)))
    assert (u == want).all()
    # a node that starts 8 draws in sees what a fresh node sees two row-iterations later
    fresh = philox.row_uniforms_layer(2, 64, 64)
    later = philox.row_uniforms_layer(2, 32, 64, offset=philox.draws_per_sampling_node(32, 64))
    assert (later.reshape(2, 32) == fresh.reshape(2, 64)[:, 32:]).all()


def test_cem_resample_closed_forms():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((5, 8)).astype(np.float32)
    z = rng.standard_normal((5, 8)).astype(np.float32)
    everyone = np.ones(8, dtype=np.int32)
    assert (row_ops.cem_resample(x, everyone, z) == x).all()                 # winners are never touched
    one = np.zeros(8, dtype=np.int32); one[3] = 1                            # one winner: std 0 -> the noise floor
    got = row_ops.cem_resample(x, one, z, noise=0.1)
    assert (got[:, 3] == x[:, 3]).all()
    others = np.delete(got, 3, axis=1)
    assert np.allclose(others, np.delete(z, 3, axis=1) * np.float32(0.1) + x[:, 3:4], rtol=1e-6, atol=1e-7)
    two = np.zeros(8, dtype=np.int32); two[[1, 6]] = 1                       # two winners a, b: mean (a+b)/2,
    got = row_ops.cem_resample(x, two, z, noise=0.0, decay=0.5)              # std = |a-b|/2 * 2/(2-1) = |a-b|
    a, b = x[:, 1], x[:, 6]
    want = (z[:, 0] * np.abs(a - b) + (a + b) / 2) * 0.5
    assert np.allclose(got[:, 0], want, rtol=1e-5, atol=1e-6)
    assert (got[:, [1, 6]] == x[:, [1, 6]]).all()


def test_cem_rewards_mask_by_hand():
    rewards = np.array([[2.0, 1.0], [0.0, 0.0], [9.0, 3.0], [1.0, 2.0]], dtype=np.float32)   # averages 2, 0, 3, 0.5
    assert row_ops.cem_update_rewards_mask(rewards).tolist() == [1, 0, 1, 0]                 # mean 1.375


def test_curand_normal_rows_is_box_muller_on_the_pinned_words():
    """The normals are a fixed function of Philox words that the known-answer vectors pin: for every pair,
    n0^2 + n1^2 = -2 ln u and atan2(n0, n1) = v (mod 2 pi) with u, v from words 2 i, 2 i + 1 of the row's stream;
    the sample moments are a standard normal's; `offset` shifts the sequence."""
    rows, cols = 300, 64
    z = philox.curand_normal_rows(rows, cols, 99, 0).astype(np.float64)
    r = np.repeat(np.arange(rows), cols // 2)
    i = np.tile(np.arange(cols // 2), rows)
    x = philox.curand_words(99, r, 2 * i).astype(np.float64)
    y = philox.curand_words(99, r, 2 * i + 1).astype(np.float64)
    u = x * 2.0 ** -32 + 2.0 ** -33
    v = 2 * np.pi * (y * 2.0 ** -32 + 2.0 ** -33)
    n0, n1 = z[:, 0::2].reshape(-1), z[:, 1::2].reshape(-1)
    assert np.allclose(n0 * n0 + n1 * n1, -2 * np.log(u), rtol=1e-5, atol=1e-6)
    assert np.allclose(n0, np.sqrt(-2 * np.log(u)) * np.sin(v), atol=3e-6)
    assert np.allclose(n1, np.sqrt(-2 * np.log(u)) * np.cos(v), atol=3e-6)
    assert abs(z.mean()) < 5 / np.sqrt(z.size) and abs(z.std() - 1) < 0.02
    assert abs((np.abs(z) < 1).mean() - 0.6827) < 0.01
    shifted = philox.curand_normal_rows(rows, cols, 99, 8)
    assert (shifted[:, :cols - 8] == philox.curand_normal_rows(rows, cols, 99, 0)[:, 8:]).all()


def test_row_reduce_by_hand():
    x = np.array([[1, -2, 3, 0.5], [2, 2, 2, 2]], dtype=np.float32)
    assert row_ops.row_reduce(x, "sum").tolist() == [2.5, 8.0]
    assert row_ops.row_reduce(x, "prod").tolist() == [-3.0, 16.0]
    assert row_ops.row_reduce(x, "max").tolist() == [3.0, 2.0] and row_ops.row_reduce(x, "min").tolist() == [-2.0, 2.0]
    assert row_ops.row_reduce(x, "average").tolist() == [0.625, 2.0]
    assert row_ops.row_reduce(x, "sum", "square", "sqrt").tolist() == [np.float32(np.sqrt(14.25)), 4.0]
    assert row_ops.row_reduce(x, "max", "abs").tolist() == [3.0, 2.0]


def test_l1_normalize_by_hand():
    # (ml/primitives.spi:725-729) rows 0 and 1: l1 norm 8 > 4 -> halved, signs dropped; row 2: norm 2 <= 4 -> |x| as is;
    # row 3: norm exactly at the threshold is not scaled; an l2 clamp would leave row 0 (l2 norm 4) untouched
    x = np.array([[2, -2, 2, -2], [8, 0, 0, 0], [-1, 0.5, 0, -0.5], [1, -1, 1, -1]], dtype=np.float32)
    want = np.array([[1, 1, 1, 1], [4, 0, 0, 0], [1, 0.5, 0, 0.5], [1, 1, 1, 1]], dtype=np.float32)
    assert (row_ops.l1_normalize(x, 4.0) == want).all()
    rng = np.random.default_rng(5)
    y = rng.standard_normal((64, 32)).astype(np.float32) * 3
    out = row_ops.l1_normalize(y, 10.0)
    norms = np.abs(y).sum(axis=1)
    assert (out >= 0).all()
    assert np.allclose(out.sum(axis=1), np.minimum(norms, 10.0), rtol=1e-5)
    assert np.allclose(out * norms[:, None], np.abs(y) * out.sum(axis=1)[:, None], rtol=1e-4)   # proportions kept
    assert (row_ops.l1_normalize(np.zeros((2, 4), np.float32), 1.0) == 0).all()                 # no 0 / 0


def test_regret_matching_of_a_subnormal_sum_is_a_distribution():
    # the positive parts add up to a subnormal number: r / s is still an ordinary quotient
    tiny = np.float32(2.0 ** -140)
    x = np.array([[tiny, -1, 3 * tiny, 0]], dtype=np.float32)
    p = row_ops.regret_matching(x)
    assert np.isfinite(p).all() and (p == np.array([[.25, 0, .75, 0]], dtype=np.float32)).all()


def test_reduce_all_by_hand():
    x = np.array([[3, -7, 2, 5], [1, 4, -2, 6]], dtype=np.int32)
    assert row_ops.reduce_all(x, "+") == 12 and row_ops.reduce_all(x, "max") == 6 and row_ops.reduce_all(x, "min") == -7
    assert row_ops.reduce_all(x, "*") == 3 * -7 * 2 * 5 * 1 * 4 * -2 * 6
    assert row_ops.reduce_all(np.arange(16384, dtype=np.uint64), "+") == 134209536      # the reference's test6
