"""Host surface of the tiled GEMM (reference: ml/matmul/run.spi, generated ml/matmul/run.py).

`matmul_tf32(a_trans, b_trans, alpha, a, b, beta, c)` keeps the reference's name and argument
order (ml/matmul/run.spi:25); `main()` / `main_body()` keep the self-test meaning of the generated
module (random A, B, C of 8192 x 8192 x 4096, compare against a library GEMM, return the max
absolute difference; ml/matmul/run.spi:28-58).  The multiplication itself runs in
libspiral_mi355.so (sp_gemm_abt).
"""
import ctypes as C

import torch

from . import _lib
from ._lib import check, lib, ptr, stream_ptr


def matmul_config_tf32(a_trans, b_trans, m, n, k, dtype=torch.float32):
    """Tile configuration chosen for a shape (counterpart of ml/matmul/run.spi:8-19).
    Returns dict(m_tile, n_tile, k_tile, threads); m_tile == 0 means the general kernel."""
    out = [C.c_int32() for _ in range(4)]
    check(lib.sp_gemm_config(_lib.DTYPES[dtype], m, n, k, *[C.byref(o) for o in out]))
    return dict(zip(("m_tile", "n_tile", "k_tile", "threads"), (o.value for o in out)))


def matmul_abt(a, b, c=None, alpha=1.0, beta=0.0, bias=None, relu=False, out_dtype=None, force_generic=False):
    """C = alpha * A . B^T + beta * C (+ bias, ReLU).  a: (M, K), b: (N, K), both row-major and of
    the same dtype (f32, f16 or bf16).  `c` is updated in place and returned; when it is None a new
    (M, N) tensor of `out_dtype` (default f32) is allocated by torch (beta must then be 0)."""
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError("a and b must be 2-D")
    if a.dtype != b.dtype or a.dtype not in _lib.DTYPES:
        raise TypeError("a and b must share one of the dtypes f32/f16/bf16")
    m, k = a.shape
    n, kb = b.shape
    assert k == kb, "The K dimension of the A and B tensors must match."
    if c is None:
        assert beta == 0.0, "beta != 0 needs an existing C"
        c = torch.empty((m, n), dtype=out_dtype or torch.float32, device=a.device)
    assert c.shape[0] == m, "The M dimension of the A and C tensors must match."
    assert c.shape[1] == n, "The N dimension of the B and C tensors must match."
    assert alpha != 0, "The alpha must not be zero."
    flags = (_lib.GEMM_RELU if relu else 0) | (_lib.GEMM_FORCE_GENERIC if force_generic else 0)
    check(lib.sp_gemm_abt(_lib.DTYPES[a.dtype], _lib.DTYPES[c.dtype], ptr(a, name="a"), ptr(b, name="b"),
                          ptr(c, name="c"), ptr(bias, torch.float32, "bias"), m, n, k, float(alpha), float(beta),
                          flags, stream_ptr()))
    return c


def matmul_abt_batched(a, b, c=None, alpha=1.0, beta=0.0, bias=None, relu=False, out_dtype=None, force_generic=False):
    """C[e] = alpha * A[e] . B[e]^T + beta * C[e] for every batch member in ONE launch.  a: (E, M, K) or (M, K)
    (shared by all members), b: (E, N, K) or (N, K), at least one of them batched; c: (E, M, N).  This is the
    loop `graph_run_host model {ensemble}` makes around a `matmul_ensemble` layer (ml/layers.spi:336-344,468-471)."""
    if a.dtype != b.dtype or a.dtype not in _lib.DTYPES:
        raise TypeError("a and b must share one of the dtypes f32/f16/bf16")
    if a.dim() not in (2, 3) or b.dim() not in (2, 3) or (a.dim() == 2 and b.dim() == 2):
        raise ValueError("a is (E, M, K) or (M, K), b is (E, N, K) or (N, K), and one of them must carry the batch")
    e = a.shape[0] if a.dim() == 3 else b.shape[0]
    if a.dim() == 3 and b.dim() == 3:
        assert a.shape[0] == b.shape[0], "The batch dimensions of the A and B tensors must match."
    m, k = a.shape[-2:]
    n, kb = b.shape[-2:]
    assert k == kb, "The K dimension of the A and B tensors must match."
    if c is None:
        assert beta == 0.0, "beta != 0 needs an existing C"
        c = torch.empty((e, m, n), dtype=out_dtype or torch.float32, device=a.device)
    assert tuple(c.shape) == (e, m, n), "The dimensions of the C tensor must be (batch, M, N)."
    assert alpha != 0, "The alpha must not be zero."
    flags = (_lib.GEMM_RELU if relu else 0) | (_lib.GEMM_FORCE_GENERIC if force_generic else 0)
    check(lib.sp_gemm_abt_batched(_lib.DTYPES[a.dtype], _lib.DTYPES[c.dtype], ptr(a, name="a"), ptr(b, name="b"),
                                  ptr(c, name="c"), ptr(bias, torch.float32, "bias"), m, n, k, e,
                                  m * k if a.dim() == 3 else 0, n * k if b.dim() == 3 else 0, m * n, float(alpha),
                                  float(beta), flags, stream_ptr()))
    return c


def _transposed(x):
    """Materialise x^T with the library's transpose kernel (4-byte elements only)."""
    if x.dtype != torch.float32:
        raise NotImplementedError("transposed operands are supported for f32 only")
    rows, cols = x.shape
    out = torch.empty((cols, rows), dtype=x.dtype, device=x.device)
    check(lib.sp_transpose_inner_b32(ptr(x), ptr(out), 1, rows, cols, stream_ptr()))
    return out


def matmul_tf32(a_trans, b_trans, alpha, a, b, beta, c):
    """`matmul_tf32 a_trans b_trans alpha a b beta c` (ml/matmul/run.spi:25): c <- alpha * op(a) .
    op(b) + beta * c.  The native layout is a_trans=False, b_trans=True (A (M,K), B (N,K)); the
    other three are brought to it by one transpose kernel.  Products are full f32 here, not TF32."""
    if a_trans:
        a = _transposed(a)       # stored (K, M) -> (M, K)
    if not b_trans:
        b = _transposed(b)       # stored (K, N) -> (N, K)
    return matmul_abt(a, b, c, alpha, beta)


def main_body(m=512 * 16, n=512 * 16, k=512 * 8, seed=12344321):
    """The reference self-test (ml/matmul/run.spi:28-58): C <- A . B^T + C on N(0,1) f32 inputs,
    compared against a library GEMM (torch.matmul here, cuBLAS through CuPy there).  Returns the
    max absolute difference as a 0-d tensor."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    mc = torch.randn((m, n), generator=gen, device="cuda", dtype=torch.float32)
    mb = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32)
    ma = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.float32)
    d = torch.matmul(ma, mb.t()) + mc
    matmul_tf32(False, True, 1.0, ma, mb, 1.0, mc)
    return torch.max(torch.abs(mc - d))


def main():
    r = main_body()
    torch.cuda.current_stream().synchronize()  # surface device faults here, like the reference does
    return float(r)


if __name__ == "__main__":
    print(main())
