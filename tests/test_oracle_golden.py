"""The NumPy oracle against every golden vector the reference holds for the row primitives
(test_text_outputs/primitives/*, written by ml/primitives.spi tests 2-6).  Printed values carry
6 decimals, so float comparisons use an absolute tolerance of 1.5e-6 (print rounding 5e-7 plus
f32 noise); integer outputs are compared exactly."""
import numpy as np
import pytest

from oracle import philox, row_ops

PRINT_TOL = 1.5e-6
ROW_CASES = ["primitives_test2_a", "primitives_test2_b", "primitives_test4_a", "primitives_test4_b"]


@pytest.mark.parametrize("case", ROW_CASES)
@pytest.mark.parametrize("shift", ["max", "mean"])
def test_softmax(golden, case, shift):
    g = golden(case)
    x = g["input"]
    want = g["output_softmax"]
    got = row_ops.softmax(x, shift=shift)
    assert np.abs(got - want).max() < PRINT_TOL
    full = g["output_softmax_scan"][..., 0]
    assert np.abs(got - full[: x.shape[0]]).max() < PRINT_TOL


@pytest.mark.parametrize("case", ROW_CASES)
def test_masked_softmax(golden, case):
    g = golden(case)
    got = row_ops.masked_softmax(g["input"], 4)
    assert np.abs(got - g["output_masked_softmax"]).max() < PRINT_TOL
    assert (got[:, 4:] == 0).all()
    got_mean = row_ops.masked_softmax(g["input"], 4, shift="mean")
    assert np.abs(got_mean - g["output_masked_softmax"]).max() < PRINT_TOL


@pytest.mark.parametrize("case", ROW_CASES)
def test_masked_softmax_11(golden, case):
    # test2 overwrites output_softmax'.txt with the masked (j < 11) softmax (ml/primitives.spi:981-986);
    # test4 writes it to output_softmax''.txt
    g = golden(case)
    key = "output_softmax_pp" if "output_softmax_pp" in g else "output_softmax_p"
    got = row_ops.masked_softmax(g["input"], 11)
    assert np.abs(got - g[key]).max() < PRINT_TOL


@pytest.mark.parametrize("case", ROW_CASES)
def test_ln_l2(golden, case):
    g = golden(case)
    assert np.abs(row_ops.ln_l2(g["input"]) - g["output_ln"]).max() < PRINT_TOL


@pytest.mark.parametrize("case", ROW_CASES)
def test_argmax(golden, case):
    g = golden(case)
    n = g["input"].shape[0]
    want = g["output_argmax"]
    assert (row_ops.argmax(g["input"]) == want[:n]).all()
    # the full softmax table is monotone in the input, so its argmax pins all rows
    probs = g["output_softmax_scan"][..., 0]
    unique = (probs == probs.max(axis=1, keepdims=True)).sum(axis=1) == 1
    assert unique.sum() > 0.9 * len(unique)
    assert (row_ops.argmax(probs)[unique] == want[unique]).all()


@pytest.mark.parametrize("case", ROW_CASES)
@pytest.mark.parametrize("order", ["sequential", "wave"])
def test_inclusive_scan(golden, case, order):
    g = golden(case)
    p, cdf = g["output_softmax_scan"][..., 0], g["output_softmax_scan"][..., 1]
    got = row_ops.inclusive_scan_sum(p, order=order)
    # p is only known to 6 decimals: the error of a cumulative sum of n rounded terms is <= n * 5e-7
    assert np.abs(got - cdf).max() < p.shape[1] * 5e-7 + PRINT_TOL
    assert np.abs(cdf[:, -1] - 1).max() < 2e-6


@pytest.mark.parametrize("case", ROW_CASES)
def test_exclusive_scan_int(golden, case):
    g = golden(case)
    want = g["output_sum_exclusive"]
    rows, cols = want.shape
    ident = np.arange(rows * cols, dtype=np.int32).reshape(rows, cols)
    assert (g["output_identity"] == ident).all()
    assert (row_ops.exclusive_scan(ident) == want).all()
    assert (row_ops.inclusive_scan_sum(ident) - ident == want).all()


@pytest.mark.parametrize("case", ROW_CASES)
def test_index_maps(golden, case):
    g = golden(case)
    rows, cols = g["output_identity"].shape
    ii, jj = np.meshgrid(np.arange(rows), np.arange(cols), indexing="ij")
    assert (g["output_indices_map"][..., 0] == ii).all() and (g["output_indices_map"][..., 1] == jj).all()
    assert (g["output_indices_reduction"] == np.arange(rows)).all()


@pytest.mark.parametrize("case", ROW_CASES)
@pytest.mark.parametrize("order", ["sequential", "wave"])
def test_sampling_replays_reference_draws(golden, case, order):
    g = golden(case)
    p, cdf = g["output_softmax_scan"][..., 0], g["output_softmax_scan"][..., 1]
    rows, cols = p.shape
    u = philox.row_uniforms_block(rows, cols) if "test2" in case else philox.row_uniforms_grid(rows, cols)
    assert ((u > 0) & (u <= 1)).all()
    # from the printed cdf (the reference's own scan) ...
    assert (row_ops.discrete_sampling(p, u, cdf=cdf) == g["output_sampling"]).all()
    # ... and from a cdf recomputed here in either summation order
    assert (row_ops.discrete_sampling(p, u, order=order) == g["output_sampling"]).all()


@pytest.mark.parametrize("case", ROW_CASES)
def test_masked_sampling_replays_reference_draws(golden, case):
    g = golden(case)
    key = "output_softmax_pp" if "output_softmax_pp" in g else "output_softmax_p"
    p = g[key]
    rows = p.shape[0]
    full_rows, cols = g["output_identity"].shape
    u = philox.row_uniforms_block(full_rows, cols) if "test2" in case else philox.row_uniforms_grid(full_rows, cols)
    got = row_ops.discrete_sampling(p, u[:rows])
    assert (got == g["output_sampling_p"][:rows]).all()
    assert (g["output_sampling_p"] < 11).all()


@pytest.mark.parametrize("case", ["primitives_test3_a", "primitives_test3_b"])
def test_gather_masked_regret_matching_and_sampling(golden, case):
    g = golden(case)
    x = g["zip_input_output_identity_map"][..., 0]
    assert (x == g["zip_input_output_identity_map"][..., 1]).all()
    rm = row_ops.masked_regret_matching(x, 3)
    assert np.abs(rm - g["output_op_map"]).max() < PRINT_TOL
    if x.shape[0] >= 64:
        uniform_rows = (np.maximum(x[:, :3], 0).sum(axis=1) == 0)
        assert uniform_rows.sum() >= 1  # the sum == 0 -> 1/3 branch is exercised by the golden data
        assert np.abs(g["output_op_map"][uniform_rows, :3] - 1 / 3).max() < PRINT_TOL
    n_threads = g["output_sample_reduce"].shape[0]
    u = philox.row_uniforms_gather(n_threads, x.shape[1])
    p = row_ops.masked_softmax(x, 3)
    got = row_ops.discrete_sampling(p, u[: x.shape[0]])
    assert (got == g["output_sample_reduce"][: x.shape[0]]).all()
    assert (g["output_indices_reduce"] == np.arange(n_threads)).all()


def test_reduce_golden(golden):
    g = golden("primitives_test6_a")
    x = np.arange(128 * 128, dtype=np.uint64)
    assert int(row_ops.reduce_sum(x)) == int(g["output_reduce_block"]) == int(g["output_reduce_grid"]) == 134209536


@pytest.mark.parametrize("case", ["primitives_test5_a", "primitives_test5_b"])
def test_transpose_golden(golden, case):
    g = golden(case)
    assert (row_ops.transpose_inner(g["input"]) == g["output"]).all()


def test_input_stream_is_shared_between_cases(golden):
    # all tests reseed with 12344321, so their inputs start with the same N(0,1) stream
    a, b = golden("primitives_test2_a")["input"].ravel(), golden("primitives_test4_b")["input"].ravel()
    assert (a == b).all()
