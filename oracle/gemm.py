"""C = alpha * A . B^T + beta * C restated in NumPy.  TEST INFRASTRUCTURE ONLY.

Semantics follow `matmul_tf32_template` with a_trans=false, b_trans=true
(ml/matmul/kernel.spi:25-49): A is (M, K) row-major, B is (N, K) row-major, C is (M, N)
row-major.  alpha must be non-zero (:49); beta == 0 means C is not read, so NaNs in the old C
do not propagate (:152-154).  The reference multiplies in TF32; this build's contract is the
f32 product of the inputs *as stored* (after rounding to bf16/f16 where those dtypes are used),
accumulated in f32, which is more accurate than TF32, so parity is stated against NumPy.

PARITY UNPINNED against the reference: it stores no GEMM vectors (ml/matmul/run.spi:54-58 prints
a max-abs-diff and never thresholds it).  tests/test_oracle_math.py pins gemm_abt by a brute-force
triple loop, identity operands, exactly representable integer inputs and the alpha/beta algebra.

bf16 has no NumPy dtype: bf16 tensors are carried as uint16 bit patterns.
"""
import numpy as np

F32 = np.float32


def f32_to_bf16_bits(x):
    """Round f32 to bf16 with round-to-nearest-even; returns uint16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    out = np.where(nan, (u >> 16) | 0x40, rounded)
    return out.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_to(x, dtype):
    """Round an f32 array to the storage dtype and return it as f32 again (the value the device
    sees).  dtype is one of "f32", "f16", "bf16"."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == "f32":
        return x
    if dtype == "f16":
        return x.astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_bits_to_f32(f32_to_bf16_bits(x))
    raise ValueError(dtype)


def gemm_abt(a, b, c=None, alpha=1.0, beta=0.0, bias=None, relu=False, out_dtype="f32", acc=np.float32):
    """C = alpha * A . B^T + beta * C (+ bias per output column, then ReLU), f32 arithmetic.

    a: (M, K) f32 values, b: (N, K) f32 values (already rounded to their storage dtype).
    bias / ReLU are this build's epilogue extension; the reference has no bias term
    (ml/layers.spi:467 `matmul` is a bare BlockMatmul)."""
    a = np.ascontiguousarray(a, dtype=acc)
    b = np.ascontiguousarray(b, dtype=acc)
    assert a.ndim == 2 and b.ndim == 2 and a.shape[1] == b.shape[1], "K of A and B must match"
    assert alpha != 0, "The alpha must not be zero."
    out = np.matmul(a, b.T)
    if alpha != 1.0:
        out = out * acc(alpha)
    if beta != 0.0:
        assert c is not None and c.shape == out.shape
        out = out + acc(beta) * np.asarray(c, dtype=acc)
    if bias is not None:
        out = out + np.asarray(bias, dtype=acc)[None, :]
    if relu:
        out = np.maximum(out, acc(0))
    out = out.astype(np.float32)
    return round_to(out, out_dtype)


def gemm_abt_bruteforce(a, b, c=None, alpha=1.0, beta=0.0):
    """Triple loop in f64 for tiny shapes (the reference's 16x16x8 smoke shape, run.spi:46)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    m, k = a.shape
    n = b.shape[0]
    out = np.zeros((m, n), dtype=np.float64)
    for i in range(m):
        for j in range(n):
            s = 0.0
            for l in range(k):
                s += a[i, l] * b[j, l]
            out[i, j] = alpha * s + (beta * c[i, j] if beta != 0.0 else 0.0)
    return out


def rel_frobenius(x, ref):
    """||x - ref||_F / ||ref||_F in f64."""
    x = np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.linalg.norm(ref.ravel())
    return float(np.linalg.norm((x - ref).ravel()) / (d if d != 0 else 1.0))


def frame(max_, min_, limit):
    """`frame` (ml/primitives.spi:17-23): walking the dimensions from the last to the first, double
    each one that is still below its maximum while the element budget `limit` stays above 1
    (halving the budget for every doubling)."""
    out = list(min_)
    for i in reversed(range(len(out))):
        if limit > 1 and out[i] < max_[i]:
            out[i] *= 2
            limit //= 2
    return tuple(out), limit


def frame_iter(iters, min_, max_, smem_bytes, elem_size=4):
    """`frame_iter` (ml/primitives.spi:30-33): `iters` rounds of `frame` under the budget
    smem_bytes / elem_size / prod(min)."""
    limit = smem_bytes // elem_size // int(np.prod(min_))
    cur = tuple(min_)
    for _ in range(iters):
        cur, limit = frame(max_, cur, limit)
    return cur


def matmul_tile_config(m, n, k, smem_bytes=96 * 1024):
    """The reference's tile heuristic `matmul_config_tf32` (ml/matmul/run.spi:8-19): grow the
    16x16 fragment towards (m, n) under the shared-memory budget, then k_tile from 8 with the
    n (resp. m) extent doubled, and assert divisibility.  96 KB -> 128x128x64 and 224 KB ->
    128x256x64 for large problems.  Returns (m_tile, n_tile, k_tile); raises AssertionError with
    the reference's messages for shapes the reference rejects."""
    m_tile, n_tile = frame_iter(6, (16, 16), (m, n), smem_bytes)
    f = lambda t: frame_iter(6, (t * 2, 8), (t * 2, k), smem_bytes)[1]
    k_tile = min(f(m_tile), f(n_tile))
    assert m % m_tile == 0, "m must be divisible by m_tile."
    assert n % n_tile == 0, "n must be divisible by n_tile."
    assert k % k_tile == 0, "k must be divisible by k_tile."
    return m_tile, n_tile, k_tile
