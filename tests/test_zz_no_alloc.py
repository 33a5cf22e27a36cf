"""The allocation-free sum (sp_reduce_sum_static) against sp_reduce_sum, through the C ABI: bit-identical
results for f32 (same kernel, same grid, same order of additions), exact for the integer types; two calls in
a row, the second on a smaller input, so that whatever the first call left in the library's scratch array
cannot leak into the second."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import announce

pytestmark = pytest.mark.gpu


def both(x):
    from ml import _lib
    from ml._lib import check, lib, ptr, stream_ptr
    code = {torch.float32: 0, torch.int32: 1, torch.int64: 2}[x.dtype]
    ws = torch.zeros(lib.sp_reduce_workspace_bytes(), dtype=torch.uint8, device="cuda")
    want = torch.zeros(4, dtype=x.dtype, device="cuda")
    got = torch.full((4,), 7, dtype=x.dtype, device="cuda")
    check(lib.sp_reduce_sum(code, ptr(x), ptr(want), x.numel(), ptr(ws), ws.numel(), stream_ptr()))
    check(lib.sp_reduce_sum_static(code, ptr(x), ptr(got), x.numel(), stream_ptr()))
    torch.cuda.synchronize()
    return want[0].item(), got[0].item(), got[1:].tolist()


@pytest.mark.parametrize("dtype", [torch.float32, torch.int32, torch.int64])
def test_static_sum_equals_workspace_sum_twice_in_a_row(dtype):
    announce("sp_reduce_sum_static %s" % dtype)
    rng = np.random.default_rng(5)
    for n in (65536 * 256 + 3, 100003, 1 << 20, 5):       # large (full grid), then smaller and smaller inputs
        if dtype == torch.float32:
            host = rng.standard_normal(n).astype(np.float32)
        else:
            host = rng.integers(-1000, 1000, size=n).astype(np.int32 if dtype == torch.int32 else np.int64)
        x = torch.from_numpy(host).cuda()
        want, got, rest = both(x)
        assert got == want, (n, got, want)                  # bit for bit
        assert rest == [7, 7, 7]                            # only out[0] is written
        if dtype == torch.float32:
            assert abs(got - float(host.astype(np.float64).sum())) <= 1e-6 * np.abs(host).sum()
        else:
            assert got == int(host.astype(np.int64).sum())


def test_static_sum_rejects_what_it_cannot_take():
    from ml._lib import lib
    p = C.c_void_p(0x1000)
    assert lib.sp_reduce_sum_static(0, p, p, lib.sp_reduce_sum_static_max_n() + 1, None) == -2
    assert b"beyond the maximum" in lib.sp_last_error_string()
    assert lib.sp_reduce_sum_static(0, None, p, 8, None) == -1
    assert lib.sp_reduce_sum_static(0, p, p, 0, None) == -2
    assert lib.sp_reduce_sum_static(5, p, p, 8, None) == -4
