"""CPU-side checks of the C-ABI boundary: the shared library loads, exports every symbol the
header declares, and rejects every host-checkable bad argument with an error code before any
device work (so these run without a GPU)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "spiral_mi355.h")


@pytest.fixture(scope="module")
def L():
    from ml import _lib
    return _lib


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sp_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported(L):
    names = declared_functions()
    assert len(names) >= 14
    for n in names:
        assert hasattr(L.lib, n), "libspiral_mi355.so does not export %s" % n
        assert n in L.SIGNATURES, "ml/_lib.py has no ctypes signature for %s" % n


def test_missing_library_fails_loudly(L, tmp_path):
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        L.load(str(tmp_path / "libspiral_mi355.so"))


def _err(L):
    return L.lib.sp_last_error_string().decode()


def test_gemm_argument_errors(L):
    lib = L.lib
    p = C.c_void_p(0x1000)
    args = lambda **kw: [kw.get("din", 2), kw.get("dout", 0), kw.get("A", p), kw.get("B", p), kw.get("C", p),
                         kw.get("bias", None), kw.get("M", 64), kw.get("N", 64), kw.get("K", 64),
                         kw.get("alpha", 1.0), 0.0, 0, None]
    assert lib.sp_gemm_abt(*args(A=None)) == -1 and "A is NULL" in _err(L)
    assert lib.sp_gemm_abt(*args(B=C.c_void_p(0x1004))) == -3 and "16-byte" in _err(L)
    assert lib.sp_gemm_abt(*args(M=0)) == -2
    assert lib.sp_gemm_abt(*args(K=60)) == -2 and "multiple of 8" in _err(L)
    assert lib.sp_gemm_abt(*args(din=0, K=6)) == -2 and "multiple of 4" in _err(L)
    assert lib.sp_gemm_abt(*args(din=7)) == -4
    assert lib.sp_gemm_abt(*args(din=1, dout=2)) == -4
    assert lib.sp_gemm_abt(*args(alpha=0.0)) == -5 and "alpha must not be zero" in _err(L)
    # what the kernels cannot address is refused on the host: rows longer than 512 MiB (32-bit lane offsets),
    # more blocks than a launch can number
    assert lib.sp_gemm_abt(*args(K=(1 << 28) + 8)) == -2 and "too large" in _err(L)
    assert lib.sp_gemm_abt(*args(din=0, K=(1 << 27) + 4)) == -2 and "too large" in _err(L)
    assert lib.sp_gemm_abt(*args(M=1 << 20, N=1 << 20)) == -2 and "too large" in _err(L)
    assert lib.sp_gemm_abt(*args(M=(1 << 31) + 1)) == -2


def test_batched_gemm_argument_errors(L):
    lib = L.lib
    p = C.c_void_p(0x1000)
    call = lambda **kw: lib.sp_gemm_abt_batched(0, 0, p, p, p, None, 64, 64, 64, kw.get("batch", 4), kw.get("sa", 0),
                                                kw.get("sb", 4096), kw.get("sc", 4096), 1.0, 0.0, 0, None)
    assert call(batch=0) == -2 and call(batch=70000) == -2
    assert call(sc=100) == -5 and "overlap" in _err(L)
    assert call(sb=4097) == -3
    assert call(sa=-4) == -3
    assert lib.sp_gemm_abt_batched(0, 0, None, p, p, None, 64, 64, 64, 2, 0, 4096, 4096, 1.0, 0.0, 0, None) == -1


def test_row_argument_errors(L):
    lib = L.lib
    p = C.c_void_p(0x2000)
    assert lib.sp_row_ops(None, None, None, None, None, None, None, None, 8, 8, 0, None) == -1
    assert lib.sp_row_ops(p, None, None, None, None, None, None, None, 8, 6, 0, None) == -2
    assert lib.sp_row_ops(p, None, None, None, None, None, None, None, 8, 2048, 0, None) == -2
    assert lib.sp_row_ops(p, None, None, None, None, None, None, None, 0, 8, 0, None) == -2
    assert lib.sp_row_ops(p, None, None, None, None, None, None, None, 8, 8, 1, None) == -5 and "flags" in _err(L)
    assert lib.sp_row_ops(p, None, None, None, None, None, None, p, 8, 8, 0, None) == -1  # sample without u
    assert lib.sp_row_ops(p, None, None, None, C.c_void_p(0x2008), None, None, None, 8, 8, 0, None) == -3
    assert lib.sp_row_map_f32(99, p, p, 8, 8, 0, None) == -5
    assert lib.sp_row_map_f32(L.ROW_MASKED_SOFTMAX, p, p, 8, 8, 0, None) == -5
    assert lib.sp_row_map_f32(L.ROW_MASKED_SOFTMAX, p, p, 8, 8, 9, None) == -5
    assert lib.sp_row_map_i32(L.ROW_SOFTMAX, p, p, 8, 8, None) == -5
    ph = L.PhiloxConfig(1, 0, L.PHILOX_BLOCK, 256, 24, 0, 0, 0)
    assert lib.sp_row_sample(L.ROW_SOFTMAX, p, None, None, None, None, None, p, None, 8, 8, 0, None) == -5
    assert lib.sp_row_sample(L.ROW_SOFTMAX, p, p, C.byref(ph), None, None, None, p, None, 8, 8, 0, None) == -5
    assert lib.sp_row_sample(L.ROW_LN_L2, p, p, None, None, None, None, p, None, 8, 8, 0, None) == -5
    bad = L.PhiloxConfig(1, 0, L.PHILOX_BLOCK, 100, 24, 0, 0, 0)  # 100 threads is not a multiple of cols/4 = 16
    assert lib.sp_row_sample(L.ROW_SOFTMAX, p, None, C.byref(bad), None, None, None, p, None, 8, 64, 0, None) == -5
    layer = L.PhiloxConfig(1, 0, L.PHILOX_LAYER, 256, 24, 3, 0, 0)  # 3 rows per block do not divide 8 rows
    assert lib.sp_row_sample(L.ROW_SOFTMAX, p, None, C.byref(layer), None, None, None, p, None, 8, 64, 0, None) == -5
    members = L.PhiloxConfig(1, 0, L.PHILOX_LAYER, 256, 24, 2, 3, 16)   # runs of 3 rows do not divide 8 rows
    assert lib.sp_row_sample(L.ROW_SOFTMAX, p, None, C.byref(members), None, None, None, p, None, 8, 64, 0, None) == -5
    assert lib.sp_row_get_prob(L.ROW_IDENTITY, p, None, p, 8, 8, 0, None) == -1
    assert lib.sp_row_get_prob(L.ROW_INCLUSIVE_SCAN, p, p, p, 8, 8, 0, None) == -5
    assert lib.sp_row_get_prob(L.ROW_MASKED_REGRET_MATCHING, p, p, p, 8, 8, 0, None) == -5
    assert lib.sp_row_binarize(p, p, 8, 8, 0, None) == -5 and "modulo" in _err(L)
    assert lib.sp_row_binarize(p, None, 8, 8, 7, None) == -1
    assert lib.sp_cem_resample(p, p, None, p, 8, 8, 0.1, 1.0, None) == -1
    assert lib.sp_cem_resample(p, p, p, p, 8, 6, 0.1, 1.0, None) == -2
    assert lib.sp_cem_resample_philox(p, p, 1, 0, None, 8, 8, 0.1, 1.0, None) == -1
    assert lib.sp_cem_resample_philox(p, p, 1, 6, p, 8, 8, 0.1, 1.0, None) == -5 and "multiple of 4" in _err(L)
    assert lib.sp_cem_resample_philox(p, p, 1, 0, p, 8, 6, 0.1, 1.0, None) == -2
    assert lib.sp_row_reduce_f32(0, 0, 0, p, None, 8, 8, None) == -1
    assert lib.sp_row_reduce_f32(0, 0, 0, p, p, 8, 6, None) == -2
    assert lib.sp_row_reduce_f32(9, 0, 0, p, p, 8, 8, None) == -5
    assert lib.sp_row_reduce_f32(0, 5, 0, p, p, 8, 8, None) == -5
    assert lib.sp_row_reduce_f32(0, 0, 2, p, p, 8, 8, None) == -5
    assert lib.sp_cem_update_mask(p, p, 0, None) == -2
    assert lib.sp_cem_update_mask(None, p, 4, None) == -1


def test_misc_argument_errors(L):
    lib = L.lib
    p = C.c_void_p(0x3000)
    assert lib.sp_map_f32(0, p, p, 6, None) == -2
    assert lib.sp_map_f32(0, None, p, 8, None) == -1
    assert lib.sp_reduce_sum(0, p, p, 8, p, 16, None) == -5
    big = lib.sp_reduce_workspace_bytes()
    assert lib.sp_reduce(4, 0, p, p, 8, p, big, None) == -5 and "op must be" in _err(L)     # no whole-tensor average
    assert lib.sp_reduce(2, 3, p, p, 8, p, big, None) == -4
    assert lib.sp_reduce(2, 0, p, p, 0, p, big, None) == -2
    assert lib.sp_reduce(2, 0, p, p, 8, None, big, None) == -1
    assert lib.sp_reduce_status(p, 16, C.byref(C.c_int64()), None) == -5
    assert lib.sp_reduce_status(p, big, None, None) == -1
    assert lib.sp_reduce_set_poll_limit(20000000) == -5 and lib.sp_reduce_set_poll_limit(0) == 0
    assert lib.sp_row_l1_normalize(p, p, 4, 8, 0.0, None) == -5 and "threshold" in _err(L)
    assert lib.sp_row_l1_normalize(p, None, 4, 8, 1.0, None) == -1
    assert lib.sp_reduce_workspace_bytes() >= 1024
    assert lib.sp_transpose_inner_b32(p, p, 1, 8, 8, None) == -5
    assert lib.sp_transpose_inner_b32(p, C.c_void_p(0x4000), 0, 8, 8, None) == -2
    assert lib.sp_device_info(None) == -1


def test_mlp_argument_errors(L):
    lib = L.lib
    p = C.c_void_p(0x5000)
    w = (C.c_void_p * 2)(p, p)
    dims = lambda *d: (C.c_int32 * len(d))(*d)
    call = lambda dtype=1, x=p, n=2, ws=w, d=dims(32, 64, 3), u=None, ph=None, pol=p, act=None, batch=8, head=3, mask=0: \
        lib.sp_mlp_forward(dtype, x, n, ws, None, d, u, ph, pol, act, None, batch, head, mask, None)
    assert call(dtype=0) == -4
    assert call(x=None) == -1
    assert call(n=0) == -5 and call(n=9) == -5
    assert call(d=dims(30, 64, 3)) == -2
    assert call(d=dims(32, 48, 3)) == -2
    assert call(d=dims(32, 512, 3)) == -2
    assert call(d=dims(32, 64, 128)) == -2
    assert call(batch=0) == -2
    assert call(head=7) == -5
    assert call(mask=4) == -5
    assert call(act=p) == -1  # action without u
    assert call(ws=(C.c_void_p * 2)(p, None)) == -1
    # a head that draws its own uniforms: one of u / philox, and the output width must be a row width of the
    # reference's sampling op (a multiple of 4) whose 4-column thread groups divide the block
    ph = L.PhiloxConfig(12344321, 0, L.PHILOX_LAYER, 256, 24, 8, 0, 0)
    assert call(act=p, u=p, ph=C.byref(ph)) == -5 and "at most one" in _err(L)
    assert call(act=p, ph=C.byref(ph)) == -5 and "multiple of 4" in _err(L)
    assert call(act=p, ph=C.byref(ph), d=dims(32, 64, 64), batch=24 * 8 + 1) == -5 and "rows_per_block" in _err(L)
    bad = L.PhiloxConfig(12344321, 0, 9, 256, 24, 8, 0, 0)
    assert call(act=p, ph=C.byref(bad), d=dims(32, 64, 64)) == -5 and "philox mode" in _err(L)


def test_packed_mlp_argument_errors(L):
    lib = L.lib
    p = C.c_void_p(0x6000)
    dims = lambda *d: (C.c_int32 * len(d))(*d)
    assert lib.sp_mlp_packed_bytes(4, dims(32, 256, 256, 256, 3)) == 4 * 4096 + 2 * 131072 + 8192
    assert lib.sp_mlp_packed_bytes(3, dims(128, 256, 256, 64)) == 4 * 8 * 4096 + 131072 + 8192
    assert lib.sp_mlp_packed_bytes(3, dims(32, 128, 256, 3)) == 0
    assert lib.sp_mlp_packed_bytes(2, dims(32, 256, 3)) == 0
    assert lib.sp_mlp_packed_bytes(6, dims(32, 256, 256, 256, 256, 256, 3)) == 0
    assert lib.sp_mlp_packed_bytes(4, None) == 0
    w = (C.c_void_p * 4)(p, p, p, p)
    d = dims(32, 256, 256, 256, 3)
    assert lib.sp_mlp_pack_weights(1, 4, w, d, None, 1 << 20, None) == -1
    assert lib.sp_mlp_pack_weights(0, 4, w, d, p, 1 << 20, None) == -4
    assert lib.sp_mlp_pack_weights(1, 4, w, d, p, 1000, None) == -5 and "must hold" in _err(L)
    assert lib.sp_mlp_pack_weights(1, 4, w, dims(32, 256, 128, 256, 3), p, 1 << 20, None) == -6
    assert lib.sp_mlp_pack_weights(1, 4, (C.c_void_p * 4)(p, None, p, p), d, p, 1 << 20, None) == -1
    size = lib.sp_mlp_packed_bytes(4, d)
    call = lambda dtype=1, x=p, n=4, pk=p, nbytes=size, dd=d, u=None, pol=p, act=None, logits=None, batch=8, head=1, mask=0: \
        lib.sp_mlp_forward_packed(dtype, x, n, pk, nbytes, None, dd, u, None, pol, act, logits, batch, head, mask, None)
    # a buffer packed for another stack (another layer count, another class of first width) has another size
    assert call(nbytes=lib.sp_mlp_packed_bytes(3, dims(32, 256, 256, 3))) == -5 and "another stack" in _err(L)
    assert call(nbytes=lib.sp_mlp_packed_bytes(4, dims(64, 256, 256, 256, 3))) == -5
    assert call(nbytes=size + 16) == -5
    assert call(dtype=0) == -4
    assert call(pk=None) == -1
    assert call(batch=0) == -2
    assert call(act=p) == -1                                        # action without u
    assert call(dd=dims(32, 256, 64, 256, 3)) == -6                 # a hidden width other than 256
    assert call(dd=dims(32, 256, 256, 256, 64)) == -6 and "16 outputs" in _err(L)     # wide head, no mask
    assert call(dd=dims(32, 256, 256, 256, 64), mask=3, logits=p) == -6               # wide masked head with logits
    assert call(mask=4) == -5


def test_ensemble_argument_errors(L):
    lib = L.lib
    p = C.c_void_p(0x6000)
    dims = lambda *d: (C.c_int32 * len(d))(*d)
    w2 = (C.c_void_p * 2)(p, p)
    call = lambda dtype=0, x=p, n=2, w=w2, dd=dims(128, 64, 64), members=4, u=None, pol=p, act=None, batch=64, head=2, mask=3: \
        lib.sp_mlp_forward_ensemble(dtype, x, n, w, dd, members, u, None, pol, act, batch, head, mask, None)
    assert call(dtype=1) == -4                                       # f32 only
    assert call(x=None) == -1 and call(pol=None) == -1 and call(w=None) == -1
    assert call(n=3) == -2 and "one or two layers" in _err(L)
    assert call(dd=dims(128, 32, 64)) == -2 and "hidden width" in _err(L)
    assert call(dd=dims(136, 64, 64)) == -2                         # two layers: inputs up to 128 wide
    assert call(dd=dims(20, 64, 64)) == -2                          # a multiple of 8
    assert call(mask=0) == -2 and "at most 4 computed outputs" in _err(L)
    assert call(mask=65) == -5
    assert call(members=0) == -2 and call(batch=0) == -2
    assert call(act=p) == -1                                        # an action without uniforms
    assert call(w=(C.c_void_p * 2)(p, None)) == -1
    assert call(x=C.c_void_p(0x6004)) == -3
    # one layer: inputs up to 256 wide, the same head limits
    one = (C.c_void_p * 1)(p)
    assert call(n=1, w=one, dd=dims(264, 64)) == -2
    assert call(n=1, w=one, dd=dims(256, 64), mask=5) == -2
    hash_call = lambda dtype=0, x=p, w=p, out=p, members=4, batch=64, k0=128, n=128, modulo=4096: \
        lib.sp_ensemble_binarize(dtype, x, w, out, members, batch, k0, n, modulo, None)
    assert hash_call(dtype=2) == -4
    assert hash_call(x=None) == -1 and hash_call(w=None) == -1 and hash_call(out=None) == -1
    assert hash_call(k0=260) == -2 and hash_call(k0=12) == -2 and hash_call(n=0) == -2
    assert hash_call(modulo=0) == -5 and "modulo" in _err(L)
    assert hash_call(members=70000) == -2
    assert hash_call(w=C.c_void_p(0x6008)) == -3
