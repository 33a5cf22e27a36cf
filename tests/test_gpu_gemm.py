"""GEMM C = alpha A.B^T + beta C on the GPU (through the C ABI) against the NumPy oracle.
Bar (relative Frobenius error): <= 1e-5 for f32, <= 3e-3 for f16/bf16 inputs evaluated on the
rounded inputs; exactly representable integer problems are bit-exact."""
import numpy as np
import pytest
import torch

from oracle import gemm as ogemm
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu

TOL = {"f32": 1e-5, "f16": 3e-3, "bf16": 3e-3}
TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(scope="module")
def MM():
    from ml import matmul
    return matmul


def make(rng, m, n, k, dtype, scale=None):
    scale = (1.0 / np.sqrt(k)) if scale is None else scale
    a = ogemm.round_to(rng.standard_normal((m, k), dtype=np.float32) * np.float32(scale), dtype)
    b = ogemm.round_to(rng.standard_normal((n, k), dtype=np.float32) * np.float32(scale), dtype)
    return a, b


def run(MM, a, b, dtype, **kw):
    return host(MM.matmul_abt(dev(a, TORCH[dtype]), dev(b, TORCH[dtype]), **kw))


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (128, 128, 128), (256, 256, 192), (512, 256, 64), (192, 320, 128),
                                   (1024, 1024, 256)])
def test_tiled_shapes(MM, dtype, m, n, k):
    announce("gemm tiled %s %dx%dx%d" % (dtype, m, n, k))
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a, b = make(rng, m, n, k, dtype)
    got = run(MM, a, b, dtype)
    assert ogemm.rel_frobenius(got, ogemm.gemm_abt(a, b)) < TOL[dtype]
    generic = run(MM, a, b, dtype, force_generic=True)
    assert ogemm.rel_frobenius(generic, ogemm.gemm_abt(a, b)) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("m,n,k", [(512, 512, 4096), (1024, 1024, 2048), (2048, 2048, 2048), (512, 512, 2112),
                                   (1024, 2048, 2240), (256, 256, 8192)])
def test_long_k_small_grids(MM, dtype, m, n, k):
    """16-bit shapes with at most one workgroup per compute unit and >= 32 K-tiles run on the deep LDS ring
    (8 stages of 64 x 64 tiles, 4 of 128 x 128), including K-tile counts that are no multiple of the ring length.
    Integer operands make the comparison exact, so a tile read from the wrong stage cannot hide in a tolerance."""
    announce("gemm deep ring %s %dx%dx%d" % (dtype, m, n, k))
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a, b = make(rng, m, n, k, dtype)
    assert ogemm.rel_frobenius(run(MM, a, b, dtype), ogemm.gemm_abt(a, b)) < TOL[dtype]
    ai = rng.integers(-2, 3, size=(m, k)).astype(np.float32)
    bi = rng.integers(-2, 3, size=(n, k)).astype(np.float32)
    # every K-tile of 64 gets its own weight so that a swapped or repeated tile changes the sum
    w = (np.arange(k) // 64 % 5 + 1).astype(np.float32)
    want = (ai * w).astype(np.int64) @ bi.astype(np.int64).T
    assert (run(MM, ai * w, bi, dtype).astype(np.int64) == want).all()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("k", [512, 576, 640, 704, 2048])
def test_single_tile_column_a_ring(MM, dtype, k):
    """N = 256 with enough rows for 256 x 256 tiles: the A tiles run through a three-stage ring of their own next to
    B's two stages.  K-tile counts 8..11 and 32 cover every phase of both rings and the drain at the end; integer
    operands with a weight per K-tile make a tile read from the wrong stage change the exact result."""
    announce("gemm A ring %s 65536x256x%d" % (dtype, k))
    m, n = 65536, 256
    rng = np.random.default_rng(k)
    w = (np.arange(k) // 64 % 5 + 1).astype(np.float32)
    ai = rng.integers(-2, 3, size=(m, k)).astype(np.float32) * w
    bi = rng.integers(-2, 3, size=(n, k)).astype(np.float32)
    want = ai.astype(np.float64) @ bi.astype(np.float64).T     # exact: |sum| < 2^53
    got = run(MM, ai, bi, dtype)
    assert (got.astype(np.float64) == want).all()


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("m,n,k", [(1000, 1000, 1024), (1, 4, 64), (7, 12, 128), (63, 68, 64), (65, 60, 192), (300, 1000, 256),
                                   (16384, 4, 256), (129, 132, 320), (4000, 260, 512), (2100, 2052, 128), (20000, 300, 64),
                                   (1000, 1000, 1000), (64, 64, 40), (128, 128, 72), (100, 36, 8), (256, 256, 200),
                                   (1024, 1024, 1000), (16384, 256, 32), (77, 4, 24)])
def test_ragged_m_and_n(MM, dtype, m, n, k):
    """M, N and K that no tile divides (N a multiple of 4, K of 16 bytes) run on the tiled kernels with clamped
    loads, a zero-filled last K-tile and a masked epilogue: against the oracle, exactly on integer operands, with bias + ReLU and beta,
    and without touching anything outside C (the output sits inside a larger buffer of sentinels)."""
    announce("gemm ragged %s %dx%dx%d" % (dtype, m, n, k))
    assert MM.matmul_config_tf32(False, True, m, n, k, TORCH[dtype])["m_tile"] > 0
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a, b = make(rng, m, n, k, dtype)
    assert ogemm.rel_frobenius(run(MM, a, b, dtype), ogemm.gemm_abt(a, b)) < TOL[dtype]
    ai = rng.integers(-3, 4, size=(m, k)).astype(np.float32)
    bi = rng.integers(-3, 4, size=(n, k)).astype(np.float32)
    want = ai.astype(np.float64) @ bi.astype(np.float64).T
    bias = rng.integers(-5, 6, size=n).astype(np.float32)
    c0 = rng.integers(-4, 5, size=(m, n)).astype(np.float32)
    pad = 64
    buf = torch.full((pad + m * n + pad,), -77.0, dtype=torch.float32, device="cuda")
    c = buf[pad:pad + m * n].view(m, n)
    c.copy_(dev(c0))
    MM.matmul_abt(dev(ai, TORCH[dtype]), dev(bi, TORCH[dtype]), c=c, bias=dev(bias), relu=True, alpha=1.0, beta=2.0)
    got = host(buf)
    assert (got[:pad] == -77).all() and (got[pad + m * n:] == -77).all()
    assert (got[pad:pad + m * n].reshape(m, n).astype(np.float64) == np.maximum(want + 2 * c0 + bias, 0)).all()


def test_random_small_shapes_are_exact(MM):
    """120 seeded shapes around the tile boundaries (M, N up to 330, K up to 45 chunks), all three dtypes, integer
    operands: the tiled kernels' masking of M, N and K must give the exact product, with and without bias + ReLU."""
    announce("gemm random small shapes")
    rng = np.random.default_rng(2024)
    edges = np.array([1, 2, 7, 8, 9, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 330])
    for case in range(120):
        dtype = ("f32", "f16", "bf16")[case % 3]
        per = 4 if dtype == "f32" else 8
        m = int(rng.choice(edges)) if case % 2 else int(rng.integers(1, 331))
        n = 4 * int(rng.integers(1, 84))
        k = per * int(rng.integers(1, 46))
        ai = rng.integers(-3, 4, size=(m, k)).astype(np.float32)
        bi = rng.integers(-3, 4, size=(n, k)).astype(np.float32)
        want = ai.astype(np.float64) @ bi.astype(np.float64).T
        got = run(MM, ai, bi, dtype)
        assert (got.astype(np.float64) == want).all(), (dtype, m, n, k)
        if case % 4 == 0:
            bias = rng.integers(-5, 6, size=n).astype(np.float32)
            got = host(MM.matmul_abt(dev(ai, TORCH[dtype]), dev(bi, TORCH[dtype]), bias=dev(bias), relu=True))
            assert (got.astype(np.float64) == np.maximum(want + bias, 0)).all(), (dtype, m, n, k, "bias+relu")


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_integer_inputs_are_exact(MM, dtype):
    """Small integers are exact in every dtype and every partial sum fits f32: any indexing slip
    (transposed operand, wrong fragment row, dropped K-chunk) changes the integer result."""
    announce("gemm integer exact " + dtype)
    m, n, k = 256, 512, 320
    a = ((np.arange(m * k).reshape(m, k) * 7 + 3) % 11 - 5).astype(np.float32)
    b = ((np.arange(n * k).reshape(n, k) * 5 + 1) % 13 - 6).astype(np.float32)
    want = a.astype(np.int64) @ b.astype(np.int64).T
    assert (run(MM, a, b, dtype).astype(np.int64) == want).all()
    assert (run(MM, a, b, dtype, force_generic=True).astype(np.int64) == want).all()
    ident = np.eye(256, dtype=np.float32)
    a2 = ogemm.round_to(np.random.default_rng(1).standard_normal((256, 256), dtype=np.float32), dtype)
    assert (run(MM, a2, ident, dtype) == a2).all()       # B = I  ->  C = A (not A^T)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_alpha_beta_bias_relu(MM, dtype):
    announce("gemm alpha/beta/bias/relu " + dtype)
    rng = np.random.default_rng(11)
    m, n, k = 256, 256, 128
    a, b = make(rng, m, n, k, dtype)
    c0 = rng.standard_normal((m, n), dtype=np.float32)
    bias = rng.standard_normal(n, dtype=np.float32)
    for alpha, beta in ((1.0, 1.0), (0.5, -2.0), (2.0, 0.0)):
        c = dev(c0.copy())
        MM.matmul_abt(dev(a, TORCH[dtype]), dev(b, TORCH[dtype]), c, alpha, beta)
        assert ogemm.rel_frobenius(host(c), ogemm.gemm_abt(a, b, c0, alpha, beta)) < TOL[dtype]
    # beta == 0 never reads C: NaNs must not propagate (ml/matmul/kernel.spi:152-154)
    c = torch.full((m, n), float("nan"), device="cuda")
    MM.matmul_abt(dev(a, TORCH[dtype]), dev(b, TORCH[dtype]), c, 1.0, 0.0)
    assert np.isfinite(host(c)).all()
    got = run(MM, a, b, dtype, bias=dev(bias), relu=True)
    want = ogemm.gemm_abt(a, b, bias=bias, relu=True)
    assert ogemm.rel_frobenius(got, want) < TOL[dtype]
    assert (got >= 0).all() and ((got == 0) == (want == 0)).mean() > 0.999
    with pytest.raises(AssertionError, match="alpha must not be zero"):
        MM.matmul_abt(dev(a, TORCH[dtype]), dev(b, TORCH[dtype]), alpha=0.0)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_sixteen_bit_output(MM, dtype):
    announce("gemm 16-bit output " + dtype)
    rng = np.random.default_rng(12)
    a, b = make(rng, 512, 512, 256, dtype)
    got = run(MM, a, b, dtype, out_dtype=TORCH[dtype])
    want = ogemm.gemm_abt(a, b, out_dtype=dtype)
    assert ogemm.rel_frobenius(got, want) < TOL[dtype]
    # rounding of the f32 accumulator is RNE: at most one ulp away from the rounded oracle,
    # and equal nearly everywhere
    assert (got == want).mean() > 0.98


def test_generic_shapes(MM):
    announce("gemm generic shapes")
    rng = np.random.default_rng(13)
    for dtype, (m, n, k) in (("f32", (16, 16, 8)), ("f32", (33, 7, 12)), ("f16", (100, 3, 256)), ("bf16", (5, 65, 40))):
        a, b = make(rng, m, n, k, dtype)
        assert ogemm.rel_frobenius(run(MM, a, b, dtype), ogemm.gemm_abt(a, b)) < TOL[dtype]
    a, b = make(rng, 16, 16, 8, "f32")
    assert ogemm.rel_frobenius(run(MM, a, b, "f32"), ogemm.gemm_abt_bruteforce(a, b)) < 1e-6


def test_reference_call_signature(MM):
    """matmul_tf32 a_trans b_trans alpha a b beta c with all four layouts (ml/matmul/run.spi:25)."""
    announce("gemm matmul_tf32 layouts")
    rng = np.random.default_rng(14)
    m, n, k = 128, 192, 64
    a = rng.standard_normal((m, k), dtype=np.float32)
    b = rng.standard_normal((n, k), dtype=np.float32)
    c0 = rng.standard_normal((m, n), dtype=np.float32)
    want = ogemm.gemm_abt(a, b, c0, 1.0, 1.0)
    for a_trans in (False, True):
        for b_trans in (False, True):
            am = dev(a.T.copy() if a_trans else a)
            bm = dev(b if b_trans else b.T.copy())
            c = dev(c0.copy())
            MM.matmul_tf32(a_trans, b_trans, 1.0, am, bm, 1.0, c)
            assert ogemm.rel_frobenius(host(c), want) < TOL["f32"]
    cfg = MM.matmul_config_tf32(False, True, 8192, 8192, 4096)
    assert cfg["m_tile"] > 0 and 8192 % cfg["m_tile"] == 0 and 4096 % cfg["k_tile"] == 0


def test_config1_fp32_1024(MM):
    announce("gemm config 1: f32 1024^3")
    rng = np.random.default_rng(1)
    a = rng.standard_normal((1024, 1024), dtype=np.float32)
    b = rng.standard_normal((1024, 1024), dtype=np.float32)
    got = run(MM, a, b, "f32")
    assert ogemm.rel_frobenius(got, ogemm.gemm_abt(a, b)) < TOL["f32"]
    want64 = ogemm.gemm_abt(a, b, acc=np.float64)
    assert ogemm.rel_frobenius(got, want64) < TOL["f32"]


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_config2_4096(MM, dtype):
    announce("gemm config 2: 4096^3 " + dtype)
    rng = np.random.default_rng(2)
    a, b = make(rng, 4096, 4096, 4096, dtype)
    want = ogemm.gemm_abt(a, b)
    assert ogemm.rel_frobenius(run(MM, a, b, dtype), want) < TOL[dtype]
    got16 = run(MM, a, b, dtype, out_dtype=TORCH[dtype])
    assert ogemm.rel_frobenius(got16, ogemm.round_to(want, dtype)) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_four_wave_kernel_is_exact_on_integers(MM, dtype):
    """Large 16-bit shapes run on the four-wave kernel (256 threads per tile).  Small integers make every option
    exact, so an indexing slip in its fragments, fetch offsets or epilogue changes the result: a non-square
    output, K of two, six and eleven K-tile pairs... alpha/beta, bias + ReLU, 16-bit output, a batch."""
    announce("gemm four-wave kernel, integer problems " + dtype)
    m, n = 4096, 3584
    t = TORCH[dtype]
    a = ((np.arange(m * 768, dtype=np.int64).reshape(m, 768) * 7 + 3) % 11 - 5).astype(np.float32)
    b = ((np.arange(n * 768, dtype=np.int64).reshape(n, 768) * 5 + 1) % 13 - 6).astype(np.float32)
    for k in (128, 384, 768):
        assert MM.matmul_config_tf32(False, True, m, n, k, t) == dict(m_tile=256, n_tile=256, k_tile=64, threads=256)
        ak, bk = np.ascontiguousarray(a[:, :k]), np.ascontiguousarray(b[:, :k])
        want = ak.astype(np.float64) @ bk.astype(np.float64).T      # |sum| <= 30 * 768: exact in f32
        assert (run(MM, ak, bk, dtype) == want).all(), k
    k = 384
    ak, bk = np.ascontiguousarray(a[:, :k]), np.ascontiguousarray(b[:, :k])
    want = ak.astype(np.float64) @ bk.astype(np.float64).T
    c0 = ((np.arange(m * n, dtype=np.int64).reshape(m, n) * 3) % 17 - 8).astype(np.float32)
    bias = ((np.arange(n) * 5) % 201 - 100).astype(np.float32)
    c = dev(c0.copy())
    MM.matmul_abt(dev(ak, t), dev(bk, t), c, 2.0, -3.0)
    assert (host(c) == 2.0 * want - 3.0 * c0).all()
    got = run(MM, ak, bk, dtype, bias=dev(bias), relu=True)
    assert (got == np.maximum(want + bias, 0.0)).all()
    got16 = run(MM, ak, bk, dtype, out_dtype=t)
    assert (got16 == ogemm.round_to(want.astype(np.float32), dtype)).all()
    # batch of 4 members of 1024 rows (4 x 14 tiles each), B shared
    many = host(MM.matmul_abt_batched(dev(ak.reshape(4, 1024, k), t), dev(bk, t)))
    assert (many.reshape(m, n) == want).all()


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_four_wave_kernel_on_tall_shapes_is_exact_on_integers(MM, dtype):
    """Tall 16-bit shapes (at least four times as many tile rows as tile columns) take the four-wave kernel with a
    ring of three A stages, whose A stage is a run-time offset and whose fetches are counted differently: the same
    exact-integer checks, for K of four, five and nine K-tile pairs... and every epilogue option."""
    announce("gemm four-wave kernel with three A stages, integer problems " + dtype)
    m, n = 32768, 512
    t = TORCH[dtype]
    a = ((np.arange(m * 1152, dtype=np.int64).reshape(m, 1152) * 7 + 3) % 11 - 5).astype(np.float32)
    b = ((np.arange(n * 1152, dtype=np.int64).reshape(n, 1152) * 5 + 1) % 13 - 6).astype(np.float32)
    for k in (256, 512, 640, 1152):
        assert MM.matmul_config_tf32(False, True, m, n, k, t) == dict(m_tile=256, n_tile=256, k_tile=64, threads=256)
        ak, bk = np.ascontiguousarray(a[:, :k]), np.ascontiguousarray(b[:, :k])
        want = ak.astype(np.float64) @ bk.astype(np.float64).T      # |sum| <= 30 * 1152: exact in f32
        assert (run(MM, ak, bk, dtype) == want).all(), k
    k = 640
    ak, bk = np.ascontiguousarray(a[:, :k]), np.ascontiguousarray(b[:, :k])
    want = ak.astype(np.float64) @ bk.astype(np.float64).T
    c0 = ((np.arange(m * n, dtype=np.int64).reshape(m, n) * 3) % 17 - 8).astype(np.float32)
    bias = ((np.arange(n) * 5) % 201 - 100).astype(np.float32)
    c = dev(c0.copy())
    MM.matmul_abt(dev(ak, t), dev(bk, t), c, 2.0, -3.0)
    assert (host(c) == 2.0 * want - 3.0 * c0).all()
    got = run(MM, ak, bk, dtype, bias=dev(bias), relu=True)
    assert (got == np.maximum(want + bias, 0.0)).all()
    got16 = run(MM, ak, bk, dtype, out_dtype=t)
    assert (got16 == ogemm.round_to(want.astype(np.float32), dtype)).all()
    # batch of 2 members of 16384 rows (64 x 2 tiles each), B shared
    many = host(MM.matmul_abt_batched(dev(ak.reshape(2, 16384, k), t), dev(bk, t)))
    assert (many.reshape(m, n) == want).all()


@pytest.mark.parametrize("m,n,k", [(65536, 256, 1152), (65536, 2048, 512), (4096, 512, 8192), (6144, 8192, 256),
                                   (8192, 6144, 1152), (8192, 8192, 128), (8192, 8192, 256)])
def test_streamed_and_written_through_outputs_are_exact_on_integers(MM, m, n, k):
    """The stores of C carry a cache policy chosen per launch: written through the L2, or -- operands of 140 MiB and
    more, or an output of 384 MiB and more -- streamed past the caches.  The streamed form on the eight-wave kernel
    (144 MiB of A), on the persistent four-wave kernel in two phase groups (512 MiB of C; a short-K problem with three
    tiles per compute unit; the two-stage persistent form at 18 K-tiles and at its shortest, two K-tiles, where every
    tile boundary hands over to the next tile's fetches at its first K-tile) and the written-through form on a square-ish problem, each with every epilogue option, exact on small integers."""
    announce("gemm store policies, integer problems %dx%dx%d" % (m, n, k))
    t = TORCH["bf16"]
    a = ((np.arange(m * k, dtype=np.int64).reshape(m, k) * 7 + 3) % 5 - 2).astype(np.float32)
    b = ((np.arange(n * k, dtype=np.int64).reshape(n, k) * 5 + 1) % 7 - 3).astype(np.float32)
    want = a @ b.T                                   # |sum| <= 6 * 8192: every partial sum is exact in f32, here and on the device
    ad, bd = dev(a, t), dev(b, t)
    assert (host(MM.matmul_abt(ad, bd)) == want).all()
    bias = ((np.arange(n) * 5) % 201 - 100).astype(np.float32)
    got = host(MM.matmul_abt(ad, bd, bias=dev(bias), relu=True))
    assert (got == np.maximum(want + bias, 0.0)).all()
    got16 = host(MM.matmul_abt(ad, bd, out_dtype=t).float())
    assert (got16 == ogemm.round_to(want.astype(np.float32), "bf16")).all()
    c0 = ((np.arange(m * n, dtype=np.int64).reshape(m, n) * 3) % 17 - 8).astype(np.float32)
    c = dev(c0.copy())
    MM.matmul_abt(ad, bd, c, 2.0, -3.0)
    assert (host(c) == 2.0 * want - 3.0 * c0).all()


@pytest.mark.parametrize("dtype,m,n,k", [("bf16", 2048, 2048, 2048), ("bf16", 4096, 4096, 4096), ("bf16", 65536, 256, 512),
                                         ("bf16", 65536, 1024, 512), ("bf16", 16384, 256, 256), ("f32", 2048, 2048, 512),
                                         ("f16", 1000, 1000, 1024)])
def test_results_do_not_change_from_run_to_run(MM, dtype, m, n, k):
    """Three launches on the same N(0,1) operands give the same bits (every kernel family and both store policies).
    A hazard the hardware does not interlock -- an instruction overwriting a register that a store or an MFMA has
    not read yet -- shows up exactly here: as results that differ between launches."""
    announce("gemm run-to-run %s %dx%dx%d" % (dtype, m, n, k))
    rng = np.random.default_rng(17)
    a, b = make(rng, m, n, k, dtype)
    ad, bd = dev(a, TORCH[dtype]), dev(b, TORCH[dtype])
    first = MM.matmul_abt(ad, bd)
    for _ in range(2):
        c = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        MM.matmul_abt(ad, bd, c)
        assert torch.equal(c, first)
    if dtype != "f32":
        first16 = MM.matmul_abt(ad, bd, out_dtype=TORCH[dtype])
        assert torch.equal(MM.matmul_abt(ad, bd, out_dtype=TORCH[dtype]), first16)


@pytest.mark.parametrize("dtype,out16", [("bf16", False), ("f16", False), ("bf16", True), ("f16", True)])
def test_config2_8192_sampled_rows(MM, dtype, out16):
    """8192^3, both 16-bit input types, f32 and 16-bit output: the oracle is evaluated on 192 sampled rows of C
    (a full CPU product is ~1.1 TFLOP); linearity is checked on the whole output: (2A).B^T == 2 (A.B^T) exactly
    (a factor of two commutes with every rounding involved, f16 subnormals aside)."""
    announce("gemm config 2: 8192^3 %s -> %s (sampled rows)" % (dtype, dtype if out16 else "f32"))
    rng = np.random.default_rng(3)
    n = 8192
    t = TORCH[dtype]
    a, b = make(rng, n, n, n, dtype)
    ad, bd = dev(a, t), dev(b, t)
    kw = dict(out_dtype=t) if out16 else {}
    c = MM.matmul_abt(ad, bd, **kw)
    assert c.dtype == (t if out16 else torch.float32)
    rows = rng.choice(n, 192, replace=False)
    want = ogemm.gemm_abt(a[rows], b)
    if out16:
        want = ogemm.round_to(want, dtype)
    assert ogemm.rel_frobenius(host(c[torch.from_numpy(rows).cuda()].float()), want) < TOL[dtype]
    c2 = MM.matmul_abt(ad * 2, bd, **kw)
    if out16 and dtype == "f16":
        # f16 results below 2^-14 are subnormal: their spacing is fixed at 2^-24, so the doubled sum is rounded
        # on a grid that 2 * (rounded sum) does not share.  Exact in the normal range, one step of 2^-24 below it.
        normal = c.abs() >= 2.0 ** -13
        assert torch.equal(c2[normal], (c * 2)[normal])
        assert float((c2.float() - 2 * c.float()).abs().max()) <= 2.0 ** -24
    else:
        assert torch.equal(c2, c * 2)


@pytest.mark.parametrize("k,n", [(256, 256), (512, 1024), (2048, 256)])
def test_config4_tall_skinny(MM, k, n):
    announce("gemm config 4: 65536 x %d x %d bf16" % (n, k))
    rng = np.random.default_rng(4 + k)
    m = 65536
    a, b = make(rng, m, n, k, "bf16")
    bias = rng.standard_normal(n, dtype=np.float32)
    got = run(MM, a, b, "bf16")
    assert ogemm.rel_frobenius(got, ogemm.gemm_abt(a, b)) < TOL["bf16"]
    got = run(MM, a, b, "bf16", bias=dev(bias), relu=True)
    assert ogemm.rel_frobenius(got, ogemm.gemm_abt(a, b, bias=bias, relu=True)) < TOL["bf16"]


def test_reference_self_test(MM):
    """ml/matmul/run.spi main: max |C - (A.B^T + C0)| on a smaller instance of the same recipe."""
    announce("gemm reference self-test 1024x1024x512")
    diff = float(MM.main_body(1024, 1024, 512))
    torch.cuda.synchronize()
    assert diff < 1e-3


def test_device_and_kernel_info():
    announce("device / kernel info")
    from ml import _lib
    info = _lib.device_info()
    assert info["arch"].startswith("gfx950") and info["compute_units"] >= 64 and info["wavefront_size"] == 64
    k = _lib.kernel_info("gemm_bf16_256x256")
    assert k["threads_per_block"] == 512 and k["vgprs"] > 64
    k4 = _lib.kernel_info("gemm_bf16_256x256_4w")
    assert k4["threads_per_block"] == 256 and k4["vgprs"] > 128
    for name in ("row_ops", "row_ops_scalars", "row_map"):
        kr = _lib.kernel_info(name)
        assert kr["threads_per_block"] == 256 and 0 < kr["vgprs"] <= 128
    with pytest.raises(_lib.SpiralError):
        _lib.kernel_info("no_such_kernel")


def test_clock_sample_gives_the_shader_clock():
    """Two sp_clock_sample results around a stretch of work: per SIMD sampled both times the cycle counter's advance
    over the 100 MHz counter's is the shader clock; the SIMDs of the chip agree on it, and it lies in the part's range."""
    announce("clock sample")
    from ml import _lib, matmul
    slots = 32768
    samples = torch.zeros((2, slots, 2), dtype=torch.int64, device="cuda")
    a = torch.randn((2048, 2048), device="cuda").to(torch.bfloat16)
    c = torch.empty((2048, 2048), dtype=torch.float32, device="cuda")
    for _ in range(50):
        matmul.matmul_abt(a, a, c=c)
    _lib.check(_lib.lib.sp_clock_sample(samples[0].data_ptr(), _lib.stream_ptr()))
    for _ in range(200):
        matmul.matmul_abt(a, a, c=c)
    _lib.check(_lib.lib.sp_clock_sample(samples[1].data_ptr(), _lib.stream_ptr()))
    s = host(samples)
    both = (s[0, :, 1] != 0) & (s[1, :, 1] > s[0, :, 1])
    assert both.sum() >= 512                      # most of the chip's 1024 SIMDs were reached both times
    mhz = (s[1, both, 0] - s[0, both, 0]) / (s[1, both, 1] - s[0, both, 1]) * 100.0
    med = np.median(mhz)
    assert 500 < med < 2600
    assert (np.abs(mhz - med) < 0.10 * med).mean() > 0.9      # (the XCDs settle a few percent apart under a power limit)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("e,m,n,k,shared", [(16, 1536, 64, 64, "a"), (5, 256, 256, 128, None), (3, 100, 24, 40, "a"),
                                            (4, 128, 512, 64, "b"), (40, 64, 64, 64, "a")])
def test_batched(MM, dtype, e, m, n, k, shared):
    """One launch for a whole ensemble (`matmul_ensemble`: E weight matrices, one shared input)."""
    announce("gemm batched %s e=%d %dx%dx%d shared=%s" % (dtype, e, m, n, k, shared))
    rng = np.random.default_rng(e * 1000 + m + n + k)
    a = ogemm.round_to(rng.standard_normal(((1 if shared == "a" else e), m, k), dtype=np.float32) / np.float32(np.sqrt(k)), dtype)
    b = ogemm.round_to(rng.standard_normal(((1 if shared == "b" else e), n, k), dtype=np.float32) / np.float32(np.sqrt(k)), dtype)
    t = TORCH[dtype]
    ad = dev(a[0] if shared == "a" else a, t)
    bd = dev(b[0] if shared == "b" else b, t)
    bias = rng.standard_normal(n, dtype=np.float32)
    c0 = rng.standard_normal((e, m, n), dtype=np.float32)
    cd = dev(c0)
    got = host(MM.matmul_abt_batched(ad, bd, c=cd, alpha=0.5, beta=2.0, bias=dev(bias), relu=True))
    for i in range(e):
        want = ogemm.gemm_abt(a[0 if shared == "a" else i], b[0 if shared == "b" else i], c=c0[i], alpha=0.5, beta=2.0,
                              bias=bias, relu=True)
        assert ogemm.rel_frobenius(got[i], want) < TOL[dtype]
    # every member equals the plain launch on its own operands, bit for bit
    one = host(MM.matmul_abt(dev(a[0], t), dev(b[0], t)))
    many = host(MM.matmul_abt_batched(ad, bd))
    assert (many[0] == one).all()
    with pytest.raises(AssertionError, match="K dimension"):
        MM.matmul_abt_batched(ad, dev(np.zeros((e, n, k + 8), dtype=np.float32), t))
