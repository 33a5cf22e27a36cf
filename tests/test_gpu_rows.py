"""Row primitives on the GPU (through the C ABI) against the reference's golden vectors and the
NumPy oracle.  Bar: indices, integer scans and the f32 prefix sums bit-exact; other floats within
a relative Frobenius error of 1e-5."""
import numpy as np
import pytest
import torch

from oracle import gemm as ogemm, philox as ophilox, row_ops as orow
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu

FLOAT_TOL = 1e-5          # relative Frobenius, f32 outputs
PRINT_TOL = 1.5e-6        # golden files carry 6 decimals
ROW_CASES = ["primitives_test2_a", "primitives_test2_b", "primitives_test4_a", "primitives_test4_b"]


@pytest.fixture(scope="module")
def P():
    from ml import primitives
    return primitives


@pytest.mark.parametrize("case", ROW_CASES)
def test_golden_row_maps(P, golden, case):
    announce("golden row maps " + case)
    g = golden(case)
    x = dev(g["input"])
    assert np.abs(host(P.softmax(x)) - g["output_softmax"]).max() < PRINT_TOL
    assert np.abs(host(P.masked_softmax(x, 4)) - g["output_masked_softmax"]).max() < PRINT_TOL
    assert np.abs(host(P.ln_l2(x)) - g["output_ln"]).max() < PRINT_TOL
    assert (host(P.argmax(x)) == g["output_argmax"][: x.shape[0]]).all()
    key = "output_softmax_pp" if "output_softmax_pp" in g else "output_softmax_p"
    assert np.abs(host(P.masked_softmax(x, 11)) - g[key]).max() < PRINT_TOL
    ident = dev(g["output_identity"].astype(np.int32))
    assert (host(P.exclusive_scan_sum(ident)) == g["output_sum_exclusive"]).all()
    assert (host(P.identity(ident)) == g["output_identity"]).all()
    p = dev(g["output_softmax_scan"][..., 0].copy())
    cdf = host(P.inclusive_scan_sum(p))
    assert np.abs(cdf - g["output_softmax_scan"][..., 1]).max() < p.shape[1] * 5e-7 + PRINT_TOL


@pytest.mark.parametrize("case", ROW_CASES)
def test_golden_sampling_with_device_philox(P, golden, case):
    """The stored sampled indices are reproduced from the stored probabilities with the uniforms
    generated on the device exactly as the reference does (Philox4_32_10, seed 12344321)."""
    from ml import _lib
    announce("golden philox sampling " + case)
    g = golden(case)
    mode = _lib.PHILOX_BLOCK if "test2" in case else _lib.PHILOX_GRID
    p = dev(g["output_softmax_scan"][..., 0].copy())
    probs, sample, u = P.discrete_sampling(p, rng=P.philox(mode), want_u=True)
    rows, cols = p.shape
    want_u = ophilox.row_uniforms_block(rows, cols) if "test2" in case else ophilox.row_uniforms_grid(rows, cols)
    assert (host(u) == want_u).all()
    assert (host(probs) == host(p)).all()
    assert (host(sample) == g["output_sampling"]).all()
    # masked (j < 11) variant from the first rows of the input
    x = dev(g["input"])
    _, sample_m, u_m = P.masked_softmax_and_discrete_sampling(x, 11, rng=P.philox(mode), want_u=True)
    assert (host(u_m) == want_u[: x.shape[0]]).all()
    assert (host(sample_m) == g["output_sampling_p"][: x.shape[0]]).all()


@pytest.mark.parametrize("case", ["primitives_test3_a", "primitives_test3_b"])
def test_golden_gather_rows(P, golden, case):
    from ml import _lib
    announce("golden gather rows " + case)
    g = golden(case)
    x = dev(g["zip_input_output_identity_map"][..., 0].copy())
    assert np.abs(host(P.masked_regret_matching(x, 3)) - g["output_op_map"]).max() < PRINT_TOL
    _, sample = P.masked_softmax_and_discrete_sampling(x, 3, rng=P.philox(_lib.PHILOX_GATHER))
    assert (host(sample) == g["output_sample_reduce"][: x.shape[0]]).all()


def test_golden_reduce_and_transpose(P, golden):
    announce("golden reduce / transpose")
    g = golden("primitives_test6_a")
    x = torch.arange(128 * 128, dtype=torch.int64, device="cuda")
    assert int(P.reduce_sum(x)) == int(g["output_reduce_grid"]) == 134209536
    xi = torch.arange(1 << 20, dtype=torch.int32, device="cuda") % 1000
    assert int(P.reduce_sum(xi)) == int(host(xi).sum())
    xf = dev(np.random.default_rng(0).standard_normal(1 << 20).astype(np.float32))
    assert abs(float(P.reduce_sum(xf)) - float(host(xf).astype(np.float64).sum())) < 1e-2
    for case in ("primitives_test5_a", "primitives_test5_b"):
        t = golden(case)
        assert (host(P.transpose_snd(dev(t["input"].astype(np.int32)))) == t["output"]).all()
    y = dev(np.arange(3 * 70 * 130, dtype=np.int32).reshape(3, 70, 130))
    assert (host(P.transpose_snd(y)) == orow.transpose_inner(host(y))).all()


@pytest.mark.parametrize("shape", [(1, 4, 4), (2, 64, 64), (3, 68, 132), (1, 100, 8), (2, 4, 260), (5, 7, 9),
                                   (1, 1, 257), (1, 1024, 256), (2, 6, 64)])
def test_transpose_shapes(P, shape):
    """Whole and partial 64x64 tiles, through the 16-byte kernel (both dimensions multiples of 4) and the 4-byte one."""
    announce("transpose %s" % (shape,))
    y = dev(np.random.default_rng(1).integers(-2 ** 31, 2 ** 31 - 1, size=shape, dtype=np.int64).astype(np.int32))
    assert (host(P.transpose_snd(y)) == orow.transpose_inner(host(y))).all()
    f = dev(np.random.default_rng(2).standard_normal(shape[1:], dtype=np.float32))
    back = P.grid_transpose(P.grid_transpose(f))
    assert (host(back) == host(f)).all()


@pytest.mark.parametrize("rows,cols", [(1, 4), (5, 16), (130, 64), (257, 256), (33, 260), (1000, 1024), (7, 1000),
                                       (4099, 256)])
def test_fused_and_general_kernels_agree(P, rows, cols):
    """The fused kernel (softmax and regret matching, masked or not, with sampling) against the general kernel (the
    row map alone, then sampling from its output): probabilities, samples, running sums, uniforms and the sampled
    column's probability must agree bit for bit, with given and with device uniforms."""
    announce("fused vs general %dx%d" % (rows, cols))
    rng = np.random.default_rng(rows * 1000 + cols)
    x = dev((rng.standard_normal((rows, cols), dtype=np.float32) * 2).astype(np.float32))
    u = dev((1 - rng.random(rows, dtype=np.float32)).astype(np.float32))
    def general(op_map, t, size, kw):
        """The same results from the general kernel: the row map on its own, then sampling from those probabilities."""
        probs = op_map(t, size)
        return (probs,) + tuple(P.discrete_sampling(probs, want_cdf=True, want_u=True, want_prob=True, **kw)[1:])

    def same(got, want):
        for fa, fb in zip(got, want):
            assert torch.equal(fa, fb)

    for kw in (dict(u=u), dict(rng=P.philox())):
        if "rng" in kw and (256 % (cols // 4) != 0):
            continue   # the reference's generator needs threads_per_block to be a multiple of cols/4
        full = dict(want_cdf=True, want_u=True, want_prob=True, **kw)
        same(P.softmax_and_discrete_sampling(x, **full), general(P.masked_softmax, x, cols, kw))
        same(P.regret_matching_and_discrete_sampling(x, **full), general(P.masked_regret_matching, x, cols, kw))
        for size in sorted({1, 3, cols // 2 + 1, cols - 1} - {0}):
            got = P.masked_softmax_and_discrete_sampling(x, size, **full)
            same(got, general(P.masked_softmax, x, size, kw))
            assert (got[1] < size).all() and (got[0][:, size:] == 0).all()
            same(P.masked_regret_matching_and_discrete_sampling(x, size, **full),
                 general(P.masked_regret_matching, x, size, kw))
        neg = x.clone()
        neg[::3] = -neg[::3].abs()       # rows without a positive entry: the uniform branch of regret matching
        same(P.regret_matching_and_discrete_sampling(neg, **full), general(P.masked_regret_matching, neg, cols, kw))
    assert torch.equal(P.softmax(x), P.masked_softmax(x, cols))     # the map alone: fused kernel vs general kernel


@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 4096, 262144 + 3, (1 << 22) + 1, 65536 * 256])
def test_reduce_sizes(P, n):
    """Exact for integers at every size (vector body, scalar tail, one block to the full grid); f32 against a
    float64 sum, tolerance = a few ulps of the sum of magnitudes."""
    announce("reduce n=%d" % n)
    rng = np.random.default_rng(n)
    xi = rng.integers(-1000, 1000, size=n, dtype=np.int32)
    assert int(P.reduce_sum(dev(xi))) == int(xi.sum(dtype=np.int64))
    xu = rng.integers(0, 2 ** 40, size=min(n, 1 << 20), dtype=np.int64)
    assert int(P.reduce_sum(dev(xu))) == int(xu.sum())
    xf = rng.standard_normal(n, dtype=np.float32)
    want = float(xf.astype(np.float64).sum())
    assert abs(float(P.reduce_sum(dev(xf))) - want) <= 1e-6 * float(np.abs(xf).sum(dtype=np.float64)) + 1e-6


SHAPES = [(1, 4), (3, 12), (5, 16), (130, 64), (64, 128), (257, 256), (33, 260), (9, 512), (1000, 1024), (7, 1000)]


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_row_ops_against_oracle(P, rows, cols):
    announce("row_ops oracle rows=%d cols=%d" % (rows, cols))
    rng = np.random.default_rng(rows * 10007 + cols)
    x = (rng.standard_normal((rows, cols)) * 2).astype(np.float32)
    u = (1 - rng.random(rows, dtype=np.float32)).astype(np.float32)
    out = {k: host(v) for k, v in P.row_ops(dev(x), dev(u)).items()}
    assert (out["argmax"] == orow.argmax(x)).all()
    assert (out["rowmax"] == x.max(axis=1)).all()
    assert ogemm.rel_frobenius(out["probs"], orow.softmax(x)) < FLOAT_TOL
    assert ogemm.rel_frobenius(out["rowsum"], orow.softmax_stats(x)[1]) < FLOAT_TOL
    # the prefix sums and the sampled index are bit-exact given the kernel's own probabilities
    assert (out["cdf"] == orow.inclusive_scan_sum(out["probs"], order="wave")).all()
    assert (out["sample"] == orow.discrete_sampling(out["probs"], u, order="wave")).all()
    assert ogemm.rel_frobenius(out["cdf"], orow.inclusive_scan_sum(orow.softmax(x))) < FLOAT_TOL
    # sequential-order cdf: same index on all but boundary rows
    seq = orow.discrete_sampling(out["probs"], u, order="sequential")
    assert (seq != out["sample"]).mean() < 0.01


@pytest.mark.parametrize("rows,cols", [(3, 12), (130, 64), (257, 256), (9, 512), (7, 1000)])
def test_row_maps_against_oracle(P, rows, cols):
    announce("row maps oracle rows=%d cols=%d" % (rows, cols))
    rng = np.random.default_rng(rows * 31 + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    x[0] = -np.abs(x[0])  # a row with no positive entry: regret matching falls back to uniform
    xd = dev(x)
    size = max(1, cols // 3)
    assert ogemm.rel_frobenius(host(P.softmax(xd)), orow.softmax(x)) < FLOAT_TOL
    assert ogemm.rel_frobenius(host(P.masked_softmax(xd, size)), orow.masked_softmax(x, size)) < FLOAT_TOL
    assert ogemm.rel_frobenius(host(P.ln_l2(xd)), orow.ln_l2(x)) < FLOAT_TOL
    rm = host(P.regret_matching(xd))
    assert ogemm.rel_frobenius(rm, orow.regret_matching(x)) < FLOAT_TOL
    assert (rm[0] == np.float32(1) / np.float32(cols)).all()
    mrm = host(P.masked_regret_matching(xd, size))
    assert ogemm.rel_frobenius(mrm, orow.masked_regret_matching(x, size)) < FLOAT_TOL
    assert (mrm[:, size:] == 0).all()
    assert (host(P.inclusive_scan_sum(xd)) == orow.inclusive_scan_sum(x, order="wave")).all()
    assert (host(P.exclusive_scan_sum(xd)) == orow.exclusive_scan(x, order="wave")).all()
    xi = rng.integers(-2 ** 20, 2 ** 20, size=(rows, cols)).astype(np.int32)
    assert (host(P.inclusive_scan_sum(dev(xi))) == orow.inclusive_scan_sum(xi)).all()
    assert (host(P.exclusive_scan_sum(dev(xi))) == orow.exclusive_scan(xi)).all()
    assert (host(P.map("relu", xd)) == orow.relu(x)).all()
    assert np.abs(host(P.map("tanh", xd)) - np.tanh(x)).max() < 1e-6
    assert np.abs(host(P.map("sigmoid", xd)) - 1 / (1 + np.exp(-x))).max() < 1e-6
    # sampling heads given the same uniforms
    u = (1 - rng.random(rows, dtype=np.float32)).astype(np.float32)
    for fn, args in ((P.softmax_and_discrete_sampling, ()), (P.masked_softmax_and_discrete_sampling, (size,)),
                     (P.regret_matching_and_discrete_sampling, ()),
                     (P.masked_regret_matching_and_discrete_sampling, (size,))):
        probs, sample, cdf = fn(xd, *args, u=dev(u), want_cdf=True)
        probs, sample, cdf = host(probs), host(sample), host(cdf)
        assert (cdf == orow.inclusive_scan_sum(probs, order="wave")).all()
        assert (sample == orow.discrete_sampling(probs, u, cdf=cdf)).all()
        assert (np.take_along_axis(probs, sample[:, None].astype(np.int64), 1) > 0).all()


@pytest.mark.parametrize("cols", [8, 64, 100, 256, 768])
def test_row_ops_zero_probabilities_and_extreme_uniforms(P, cols):
    """Rows whose softmax underflows to exact zeros (also in whole lanes and chunks), with u = 1, tiny u and
    u = 0: the index must still be the first one with p > 0 whose running sum reaches u * max."""
    announce("row_ops zeros/extreme u cols=%d" % cols)
    rng = np.random.default_rng(cols)
    rows = 67
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    x[::3, : cols // 2] -= 300                      # leading zeros
    x[1::3, cols // 4:] -= 300                      # trailing zeros
    x[5, :] = -300; x[5, cols - 1] = 0              # a single atom at the end
    x[6, :] = -300; x[6, 0] = 0                     # ... and at the start
    u = (1 - rng.random(rows, dtype=np.float32)).astype(np.float32)
    u[::4] = 1.0
    u[1::4] = 1e-30
    u[2::8] = 0.0
    out = {k: host(v) for k, v in P.row_ops(dev(x), dev(u)).items()}
    assert (out["probs"] == 0).any()
    assert (out["cdf"] == orow.inclusive_scan_sum(out["probs"], order="wave")).all()
    expect = orow.discrete_sampling(out["probs"], u, cdf=out["cdf"])
    assert (out["sample"] == expect).all()
    assert (np.take_along_axis(out["probs"], out["sample"][:, None].astype(np.int64), 1) > 0).all()
    assert out["sample"][5] == cols - 1 and out["sample"][6] == 0
    assert (out["argmax"] == orow.argmax(x)).all()


@pytest.mark.parametrize("cols", [4, 12, 64, 256])
def test_get_prob_get_action_binarize(P, cols):
    """row_gather_reduce users (ml/cem.spi:152-164, ml/cfr.spi:97-129) and the binarize head."""
    announce("get_prob / get_action / binarize cols=%d" % cols)
    rng = np.random.default_rng(cols + 77)
    rows = 301
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    ids = rng.integers(0, cols, size=rows).astype(np.int32)
    size = max(1, cols // 2)
    assert (host(P.get_prob(dev(x), dev(ids))) == orow.get_prob(x, ids)).all()
    mrm = host(P.masked_regret_matching(dev(x), size))
    assert (host(P.get_prob(dev(x), dev(ids), op="masked_regret_matching", size=size)) == orow.get_prob(mrm, ids)).all()
    sm = host(P.softmax(dev(x)))
    assert (host(P.get_prob(dev(x), dev(ids), op="softmax")) == orow.get_prob(sm, ids)).all()
    bad = ids.copy(); bad[::2] = cols + 3; bad[1::4] = -1
    got = host(P.get_prob(dev(x), dev(bad)))
    assert (got[::2] == 0).all() and (got[1::4] == 0).all()
    # sample + probability of the sample, from given uniforms and from the device stream
    u = (1 - rng.random(rows, dtype=np.float32)).astype(np.float32)
    prob, action = P.get_action(dev(x), u=dev(u), op="masked_softmax", size=size)
    msm = host(P.masked_softmax(dev(x), size))
    assert (host(action) == orow.discrete_sampling(msm, u, order="wave")).all()
    assert (host(prob) == orow.get_prob(msm, host(action))).all() and (host(prob) > 0).all()
    if cols >= 4 and 256 % (cols // 4) == 0:
        prob2, action2 = P.get_action(dev(x), op="masked_softmax", size=size)
        u2 = ophilox.row_uniforms_gather(rows, cols)
        assert (host(action2) == orow.discrete_sampling(msm, u2, order="wave")).all()
        assert (host(prob2) == orow.get_prob(msm, host(action2))).all()
    for modulo in (1, 7, 2 ** 31 - 1, 2 ** 32 - 1):
        assert (host(P.binarize(dev(x), modulo)).view(np.uint32) == orow.binarize(x, modulo)).all()


def test_layer_stream_uniforms(P):
    """The uniforms a sampling node of a layer graph sees (ml/layers.spi:339-344), with a draw offset."""
    from ml import _lib
    announce("philox layer stream")
    blocks, m, n = 6, 64, 64
    x = dev(np.random.default_rng(3).standard_normal((blocks * m, n)).astype(np.float32))
    for offset in (0, 16, 6):
        rng = P.philox(_lib.PHILOX_LAYER, blocks_per_grid=blocks, rows_per_block=m, offset=offset)
        _, _, u = P.softmax_and_discrete_sampling(x, rng=rng, want_u=True)
        assert (host(u) == ophilox.row_uniforms_layer(blocks, m, n, offset=offset)).all()
    # one block: the layer stream is the block-level stream
    rng = P.philox(_lib.PHILOX_LAYER, blocks_per_grid=1, rows_per_block=blocks * m)
    _, _, u = P.softmax_and_discrete_sampling(x, rng=rng, want_u=True)
    assert (host(u) == ophilox.row_uniforms_block(blocks * m, n)).all()


@pytest.mark.parametrize("dim,ensemble", [(77, 16), (1000, 64), (33, 256), (5, 1024), (19, 12)])
def test_cem_update(P, dim, ensemble):
    """Cross-entropy-method weight update (ml/cem.spi:92-146): rewards -> mask, transpose, resample, transpose."""
    announce("cem dim=%d ensemble=%d" % (dim, ensemble))
    rng = np.random.default_rng(dim * 7 + ensemble)
    rewards = np.stack([rng.standard_normal(ensemble) * 3, rng.integers(0, 4, ensemble)], axis=1).astype(np.float32)
    rd = dev(rewards)
    mask = P.cem_update_rewards_mask(rd)
    want_mask = orow.cem_update_rewards_mask(rewards)
    assert (host(mask) == want_mask).all() and (host(rd) == 0).all()
    if want_mask.sum() == 0:
        want_mask[0] = 1
        mask = dev(want_mask)
    weights = rng.standard_normal((ensemble, dim)).astype(np.float32)        # (ensemble, dim) as the layers hold them
    z = rng.standard_normal((dim, ensemble)).astype(np.float32)
    wt = P.grid_transpose(dev(weights))
    assert (host(wt) == weights.T).all()
    out = P.cem(wt, mask, normals=dev(z))
    assert out.data_ptr() == wt.data_ptr()                                    # in place, like the reference
    want = orow.cem_resample(weights.T, want_mask, z)
    assert ogemm.rel_frobenius(host(out), want) < FLOAT_TOL
    winners = want_mask.astype(bool)
    assert (host(out)[:, winners] == weights.T[:, winners]).all()           # winners bit for bit
    back = host(P.grid_transpose(out))
    assert back.shape == (ensemble, dim) and (back[winners] == weights[winners]).all()
    # one winner: every other member becomes z * noise + winner
    single = np.zeros(ensemble, dtype=np.int32); single[ensemble // 2] = 1
    got = host(P.cem(dev(weights.T.copy()), dev(single), normals=dev(z), noise=0.25, decay=1.0))
    want1 = z * np.float32(0.25) + weights.T[:, ensemble // 2: ensemble // 2 + 1]
    want1[:, ensemble // 2] = weights.T[:, ensemble // 2]
    assert np.abs(got - want1).max() < 1e-6


@pytest.mark.parametrize("rows,cols", [(1, 4), (5, 16), (130, 64), (257, 256), (33, 260), (7, 1000), (1, 4096), (3, 5000),
                                       (70000, 8)])
def test_row_reduce(P, rows, cols):
    """`row_reduce` of local_sum / prod / max / min / average and `map_reduce_map_2d` (square -> sum -> sqrt: the
    weight norms of the CEM update) at widths from one lane per row to rows longer than a wave's chunk."""
    announce("row reduce %dx%d" % (rows, cols))
    rng = np.random.default_rng(rows * 7 + cols)
    x = rng.standard_normal((rows, cols), dtype=np.float32)
    xd = dev(x)
    assert (host(P.local_max(xd)) == x.max(axis=1)).all() and (host(P.local_min(xd)) == x.min(axis=1)).all()
    scale = np.abs(x).sum(axis=1) + 1e-30
    assert (np.abs(host(P.local_sum(xd)) - orow.row_reduce(x, "sum")) <= 2e-6 * scale).all()
    assert (np.abs(host(P.local_average(xd)) - orow.row_reduce(x, "average")) <= 2e-6 * scale / cols).all()
    assert P.local_length(xd) == cols
    near_one = (1 + 0.01 * x).astype(np.float32)
    got = host(P.local_prod(dev(near_one)))
    assert np.allclose(got, orow.row_reduce(near_one, "prod"), rtol=1e-4 + 2e-7 * cols)
    norms = host(P.map_reduce_map_2d("sqr", 0, "+", "sqrt", xd))
    assert np.allclose(norms, orow.row_reduce(x, "sum", "square", "sqrt"), rtol=1e-5)
    assert np.allclose(host(P.row_reduce(xd, "max", "abs")), np.abs(x).max(axis=1), rtol=0, atol=0)
    assert float(P.reduce_max(dev(norms.copy())) if rows % 4 == 0 else P.reduce_max(xd)) == \
        (norms.max() if rows % 4 == 0 else x.max())
    into = torch.full((rows,), -5.0, dtype=torch.float32, device="cuda")
    assert P.reduce_2d(0, "+", xd, into) is into and (host(into) == host(P.local_sum(xd))).all()
    with pytest.raises(ValueError, match="neutral element"):
        P.map_reduce_map_2d("id", 1, "+", "id", xd)


@pytest.mark.parametrize("rows,cols", [(64, 16), (1000, 64), (513, 256), (40, 1024)])
def test_cem_with_device_normals(P, rows, cols):
    """sp_cem_resample_philox: the normals are curand_normal's Box-Muller pairs of the Philox stream (seed,
    subsequence = row), restated in oracle.philox.curand_normal_rows; `offset` continues the stream."""
    announce("cem device normals %dx%d" % (rows, cols))
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols), dtype=np.float32)
    mask = (rng.random(cols) < 0.4).astype(np.int32)
    mask[1] = 1
    z = ophilox.curand_normal_rows(rows, cols, 777, 0)
    got = host(P.cem(dev(x), dev(mask), rng=(777, 0), noise=0.1, decay=0.5, out=torch.empty((rows, cols), device="cuda")))
    want = orow.cem_resample(x, mask, z, 0.1, 0.5)
    assert (got[:, mask != 0] == x[:, mask != 0]).all()
    assert np.abs(got - want).max() < 2e-5 * max(1.0, np.abs(want).max())
    # one winner of value 0, noise 1: the redrawn members ARE the normals
    one = np.zeros(cols, dtype=np.int32); one[0] = 1
    x0 = x.copy(); x0[:, 0] = 0
    n0 = host(P.cem(dev(x0), dev(one), rng=(777, 0), noise=1.0, out=torch.empty((rows, cols), device="cuda")))[:, 1:]
    assert np.abs(n0 - z[:, 1:]).max() < 2e-5
    assert abs(n0.mean()) < 5 / np.sqrt(n0.size) and abs(n0.std() - 1) < 0.05
    n8 = host(P.cem(dev(x0), dev(one), rng=(777, 8), noise=1.0, out=torch.empty((rows, cols), device="cuda")))
    assert (n8[:, 1:cols - 8] == n0[:, 8:cols - 1]).all()     # eight draws in: the same sequence, shifted by eight
    from ml import _lib
    with pytest.raises(_lib.SpiralError, match="multiple of 4"):
        P.cem(dev(x0), dev(one), rng=(777, 6))


def test_sampling_edge_cases(P):
    announce("sampling edge cases")
    p = np.zeros((4, 8), dtype=np.float32)
    p[0, 3] = 1.0                      # a single atom
    p[1, [1, 6]] = 0.5                 # zeros around the atoms
    p[2, :] = 0.125
    u = np.array([1.0, 1.0, 1e-30, 0.5], dtype=np.float32)
    _, sample = P.discrete_sampling(dev(p), u=dev(u))
    s = host(sample)
    assert s[0] == 3 and s[1] == 6 and s[2] == 0
    assert s[3] == 2147483647           # no p > 0: the reduction's neutral element (limit.max)


def test_row_ops_full_size(P):
    """The benchmark's row-primitive workload: 65536 x 256 f32 logits ~ N(0, sigma=2), one uniform per row."""
    announce("row_ops full size 65536x256")
    rng = np.random.default_rng(5)
    rows, cols = 65536, 256
    x = (rng.standard_normal((rows, cols), dtype=np.float32) * np.float32(2)).astype(np.float32)
    u = (1 - rng.random(rows, dtype=np.float32)).astype(np.float32)
    out = {k: host(v) for k, v in P.row_ops(dev(x), dev(u)).items()}
    assert (out["argmax"] == orow.argmax(x)).all()
    assert (out["rowmax"] == x.max(axis=1)).all()
    assert ogemm.rel_frobenius(out["probs"], orow.softmax(x)) < FLOAT_TOL
    assert (out["cdf"] == orow.inclusive_scan_sum(out["probs"], order="wave")).all()
    assert (out["sample"] == orow.discrete_sampling(out["probs"], u, cdf=out["cdf"])).all()
    # size-independent properties
    assert np.abs(out["cdf"][:, -1] - 1).max() < 1e-5
    # a parallel prefix sum is monotone only up to rounding where two lanes' partial sums meet
    assert (np.diff(out["cdf"], axis=1) >= -2.5e-7).all()
    assert ((out["sample"] >= 0) & (out["sample"] < cols)).all()
    # scalar-outputs-only mode gives the same indices
    lean = P.row_ops(dev(x), dev(u), want=("argmax", "sample", "rowmax", "rowsum"))
    assert (host(lean["sample"]) == out["sample"]).all() and (host(lean["argmax"]) == out["argmax"]).all()


def test_main_body_writes_the_reference_files(P, golden, tmp_path):
    """`primitives.main_body` (ml/primitives.spi main, :1112-1137) writes every file of the reference's
    test_text_outputs/primitives tree; the files that do not depend on the random input are parsed back with the
    fixture parser and must equal the reference's own prints exactly (same leaves, same truncation)."""
    import os
    import sys
    from conftest import GOLDEN
    if GOLDEN not in sys.path:
        sys.path.insert(0, GOLDEN)
    import make_fixtures as mf

    announce("primitives.main_body")
    root = str(tmp_path) + "/"
    P.main_body(root)
    torch.cuda.synchronize()
    fixed = {"test2": ["input_identity", "output_identity", "output_indices_map", "output_indices_reduction",
                       "output_sum_exclusive"],
             "test3": ["input_identity", "output_indices_map", "output_indices_reduce"],
             "test6": ["input_identity", "output_reduce_block", "output_reduce_grid"]}
    fixed["test4"] = fixed["test2"]
    every = {"test2": mf.ROW_NAMES, "test4": mf.ROW_NAMES, "test3": mf.GATHER_NAMES, "test6": mf.REDUCE_NAMES}
    for test, sub in [("test2", "a"), ("test2", "b"), ("test3", "a"), ("test3", "b"), ("test4", "a"), ("test4", "b"),
                      ("test6", "a")]:
        want = golden("primitives_%s_%s" % (test, sub))
        got = mf.convert_case(os.path.join(root, test, sub), every[test])
        assert set(got) == set(want), (test, sub, sorted(set(want) ^ set(got)))   # the same files exist
        for key in fixed[test]:
            assert got[key].shape == want[key].shape and (got[key] == want[key]).all(), (test, sub, key)
            assert bool(got[key + "__truncated"]) == bool(want[key + "__truncated"]), (test, sub, key)
        for key in want:                                      # input-dependent files: same extent of the print
            assert got[key].shape == want[key].shape, (test, sub, key)
    for sub in ("a", "b"):
        want = golden("primitives_test5_" + sub)
        with open(os.path.join(root, "test5", sub, "transpose.txt")) as f:
            parts = [ln for ln in f.read().splitlines() if ln.startswith("[")]
        assert len(parts) == 2
        assert (mf.to_array(*mf.parse_tensor_text(parts[0])) == want["input"]).all()
        assert (mf.to_array(*mf.parse_tensor_text(parts[1])) == want["output"]).all()
    # the sampled indices of test3 obey the mask (j < 3)
    s3 = mf.convert_case(os.path.join(root, "test3", "b"), ["output_sample_reduce"])["output_sample_reduce"]
    assert s3.shape == (1024,) and (s3 >= 0).all() and (s3 < 3).all()


@pytest.mark.parametrize("cols", [8, 64, 256, 1024])
def test_ties_and_nans_follow_the_stated_rules(P, cols):
    """The behaviours no reference output pins, held to what the header states: argmax takes the LOWEST index among
    equal maxima and index 0 for a row of NaNs (on every kernel that computes an argmax), binarize sets a bit for
    every element that is not <= 0 (a NaN sets it, -0.0 and -inf do not)."""
    announce("ties and NaNs cols=%d" % cols)
    rng = np.random.default_rng(cols)
    rows = 37
    x = rng.standard_normal((rows, cols), dtype=np.float32)
    top = x.max(axis=1) + 1
    first = rng.integers(0, cols // 2, rows)
    for r in range(rows):                      # the maximum appears at `first`, at the last column and once in between
        x[r, first[r]] = top[r]
        x[r, cols - 1] = top[r]
        x[r, (first[r] + cols - 1) // 2] = top[r]
    x[5, :] = 2.0                               # a constant row
    want = first.copy()
    want[5] = 0
    assert (orow.argmax(x) == want).all()
    assert (host(P.argmax(dev(x))) == want).all()
    u = (1 - rng.random(rows, dtype=np.float32)).astype(np.float32)
    assert (host(P.row_ops(dev(x), dev(u))["argmax"]) == want).all()
    nan_rows = np.full((3, cols), np.nan, dtype=np.float32)
    assert (host(P.argmax(dev(nan_rows))) == 0).all()
    if cols <= 256:
        odd = rng.standard_normal((rows, cols), dtype=np.float32)
        odd[:, 0] = np.nan
        odd[:, 1] = -0.0
        odd[:, 2] = -np.inf
        odd[:, 3] = np.inf
        modulo = 8
        got = host(P.binarize(dev(odd), modulo)).view(np.uint32)
        assert (got == orow.binarize(odd, modulo)).all()


def test_results_do_not_change_from_run_to_run(P):
    """Three launches of the fused row kernel and of the sum on the same inputs give the same bits (the row outputs
    leave through hand-issued stores, the sum's partial results through a polled hand-off between workgroups)."""
    announce("rows run-to-run")
    rng = np.random.default_rng(29)
    rows, cols = 65536, 256
    x = dev((rng.standard_normal((rows, cols), dtype=np.float32) * np.float32(2)).astype(np.float32))
    u = dev((1 - rng.random(rows, dtype=np.float32)).astype(np.float32))
    first = {k: v.clone() for k, v in P.row_ops(x, u).items()}
    total = P.reduce_sum(x).clone()
    for _ in range(2):
        again = P.row_ops(x, u)
        for k in first:
            assert torch.equal(first[k], again[k]), k
        assert torch.equal(P.reduce_sum(x), total)



@pytest.mark.parametrize("rows,cols", [(3, 12), (130, 64), (257, 256), (7, 1000)])
def test_l1_normalize(P, rows, cols):
    """row_map (local_l1_normalize threshold) (ml/primitives.spi:725-729) against the oracle; rows on both sides of the
    threshold, and in place."""
    announce("l1_normalize rows=%d cols=%d" % (rows, cols))
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    x[::2] *= np.float32(0.01)                       # every other row stays under the threshold
    thr = float(np.abs(x).sum(axis=1).mean())
    want = orow.l1_normalize(x, thr)
    xd = dev(x)
    got = host(P.l1_normalize(xd, thr))
    assert ogemm.rel_frobenius(got, want) < FLOAT_TOL and (got >= 0).all()
    norms = np.abs(x).sum(axis=1)
    assert (got[norms <= thr * 0.999] == np.abs(x)[norms <= thr * 0.999]).all()       # untouched rows: exact |x|
    assert np.abs(got[norms > thr].sum(axis=1) - thr).max() < 1e-5 * thr * cols ** 0.5
    P.l1_normalize(xd, thr, out=xd)
    assert (host(xd) == got).all()


@pytest.mark.parametrize("cols", [4, 64, 256, 1024])
def test_rows_whose_sum_is_subnormal(P, cols):
    """Regret matching and ln_l2 divide by a row sum.  The kernels do that with one reciprocal per row; a sum below
    2^-126 must still give the quotients (a distribution), not infinities and NaNs."""
    announce("subnormal row sums cols=%d" % cols)
    tiny = np.float32(2.0 ** -140)
    x = np.full((6, cols), -1.0, dtype=np.float32)
    x[0, 0], x[0, 1] = tiny, 3 * tiny                 # sum 2^-138
    x[1, cols - 1] = np.float32(2.0 ** -149)          # the smallest positive number alone
    x[2, :2] = np.float32(2.0 ** -127)                # sum 2^-126: the first normal number
    x[3, :4] = [1.0, 2.0, 3.0, 2.0]                   # an ordinary row between them
    x[4, 0], x[4, 2] = np.float32(2.0 ** -130), np.float32(2.0 ** -129)
    x[5, :] = 0                                       # sum exactly 0: the uniform branch
    xd = dev(x)
    want = orow.regret_matching(x)
    got = host(P.regret_matching(xd))
    assert np.isfinite(got).all() and np.abs(got - want).max() <= 2e-7 and np.abs(got.sum(axis=1) - 1).max() < 1e-6
    assert (got[0, :2] == [0.25, 0.75]).all() and got[1, cols - 1] == 1 and (got[5] == np.float32(1) / np.float32(cols)).all()
    u = np.full(6, 0.5, dtype=np.float32)
    probs, sample = P.regret_matching_and_discrete_sampling(xd, u=dev(u))[:2]
    assert (host(probs) == got).all()                                         # the fused kernel: the same bits
    assert (host(sample)[:3] == [1, cols - 1, 0]).all()
    size = min(cols, 3)
    assert np.isfinite(host(P.masked_regret_matching(xd, size))).all()
    # ln_l2: x / sum(x^2) with a subnormal sum of squares; the quotients themselves are large but finite
    y = np.zeros((2, cols), dtype=np.float32)
    y[0, 0], y[0, 1] = np.float32(2.0 ** -68), np.float32(2.0 ** -70)        # squares 2^-136, 2^-140
    y[1, :2] = [3.0, 4.0]
    got = host(P.ln_l2(dev(y)))
    want = orow.ln_l2(y)
    assert np.isfinite(got).all() and ogemm.rel_frobenius(got, want) < FLOAT_TOL


@pytest.mark.parametrize("n", [1, 5, 4096, 262144 + 3, 65536 * 256])
def test_whole_tensor_reduce_ops(P, n):
    """`reduce neutral f` over the whole device for f in +, *, max, min (ml/primitives.spi:136-197; `grid_reduce grid 0
    max`, ml/cem.spi:140): integers exact, float max / min exact, float product against float64."""
    announce("reduce ops n=%d" % n)
    rng = np.random.default_rng(n + 1)
    xf = rng.standard_normal(n, dtype=np.float32)
    xd = dev(xf)
    assert float(P.reduce_max(xd)) == float(xf.max()) and float(P.reduce_min(xd)) == float(xf.min())
    assert float(P.reduce("max", xd)) == float(orow.reduce_all(xf, "max"))
    near_one = (1 + rng.standard_normal(min(n, 1 << 16), dtype=np.float32) * np.float32(1e-3)).astype(np.float32)
    want = float(near_one.astype(np.float64).prod())
    assert abs(float(P.reduce("*", dev(near_one))) - want) <= 1e-4 * abs(want)
    xi = rng.integers(-2 ** 30, 2 ** 30, size=n, dtype=np.int32)
    xid = dev(xi)
    assert int(P.reduce("max", xid)) == int(xi.max()) and int(P.reduce("min", xid)) == int(xi.min())
    assert int(P.reduce("+", xid)) == int(orow.reduce_all(xi, "+"))           # wraps around like the device's adds
    small = rng.integers(-3, 4, size=min(n, 4096), dtype=np.int32)
    assert int(P.reduce("*", dev(small))) == int(orow.reduce_all(small, "*"))
    xu = rng.integers(0, 2 ** 62, size=min(n, 1 << 20), dtype=np.int64)
    xud = dev(xu)
    assert int(P.reduce("max", xud)) == int(xu.max()) and int(P.reduce("min", xud)) == int(xu.min())
    # all negative floats / the lowest int: the neutral elements are -inf and the type's minimum, not 0
    neg = -np.abs(xf) - 1
    assert float(P.reduce_max(dev(neg))) == float(neg.max())
    assert int(P.reduce("max", dev(np.full(max(n, 4), -2 ** 31, dtype=np.int32)))) == -2 ** 31


def test_reduce_gives_up_cleanly_and_recovers(P):
    """The wait at the end of a whole-tensor reduce is bounded.  With a bound below zero the collecting workgroup does
    not wait at all, so it stops before the other workgroups of a 256 MiB sum have published: the result is a NaN, the
    workspace's give-up counter goes up, every kernel still runs to its end, and the next call -- which finds
    whatever the late workgroups left in their slots -- is right again."""
    from ml import _lib
    announce("reduce give-up")
    x = torch.ones(1 << 26, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    before = P.reduce_give_ups()
    assert float(P.reduce_sum(x)) == float(1 << 26)
    _lib.check(_lib.lib.sp_reduce_set_poll_limit(-1))
    try:
        gave_up = P.reduce_sum(x)
        torch.cuda.synchronize()
    finally:
        _lib.check(_lib.lib.sp_reduce_set_poll_limit(0))
    assert np.isnan(float(gave_up))
    assert P.reduce_give_ups() == before + 1
    for _ in range(3):
        assert float(P.reduce_sum(x)) == float(1 << 26)
        assert int(P.reduce("max", x.view(torch.int32))) == int(np.float32(1).view(np.int32))
    assert P.reduce_give_ups() == before + 1
