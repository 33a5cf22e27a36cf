"""The build's scan for the hazards the compiler cannot see in the hand-scheduled kernels: a vector-ALU write of
a register within two wait states of an asm MFMA that reads it, or of an asm store of more than 8 bytes that has
it as data."""
import glob
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "spiral-s-ml-library_amd")


def _module():
    spec = importlib.util.spec_from_file_location("isa_check", os.path.join(PKG, "isa_check.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


LISTING = """
kernel_a:
\tv_mov_b64_e32 v[142:143], v[44:45]
\tv_mov_b64_e32 v[140:141], v[42:43]
\tv_mfma_f32_16x16x32_f16 v[140:143], a[32:35], v[82:85], v[140:143]
\tv_add_f32_e32 v116, v110, v120
\tv_mfma_f32_16x16x32_f16 v[160:163], a[36:39], v[82:85], v[160:163]
kernel_b:
\tv_mov_b64_e32 v[140:141], v[42:43]
\ts_nop 1
\tv_mfma_f32_16x16x32_f16 v[140:143], a[32:35], v[82:85], v[140:143]
\tv_accvgpr_write_b32 a32, v7
\tds_read_b128 v[90:93], v118 offset:33024
\tv_mfma_f32_16x16x32_bf16 v[140:143], a[32:35], v[82:85], v[140:143]
\tv_mov_b32_e32 v82, 0
\tglobal_load_dwordx4 a[48:51], v1, s[4:5] offset:0x400
\ts_waitcnt lgkmcnt(3)
\tv_mfma_f32_16x16x32_bf16 v[144:147], a[36:39], v[82:85], 0
"""


def test_scan_finds_writes_inside_the_wait_states_and_only_those():
    hits = _module().scan(LISTING.splitlines())
    found = [(kernel, writer.split()[0], writer.split()[1]) for _, kernel, writer, _ in hits]
    assert found == [("kernel_a", "v_mov_b64_e32", "v[142:143],"), ("kernel_a", "v_mov_b64_e32", "v[140:141],"),
                     ("kernel_b", "v_accvgpr_write_b32", "a32,")]


STORES = """
kernel_c:
\tglobal_store_dwordx4 v[2:3], v[10:13], off sc1
\tv_add_f32_e32 v12, v1, v2
\tglobal_store_dwordx4 v[2:3], v[20:23], off nt
\ts_nop 1
\tv_add_f32_e32 v22, v1, v2
\tglobal_store_dwordx2 v[2:3], v[30:31], off
\tv_add_f32_e32 v30, v1, v2
\tglobal_store_dwordx4 v[2:3], v[40:43], off
\tv_add_f32_e32 v50, v1, v2
\tv_mul_f32_e32 v43, v1, v2
\tv_mul_f32_e32 v40, v1, v2
\tbuffer_store_dwordx4 v[60:63], v5, s[0:3], 0 offen
\tv_mov_b32_e32 v5, 0
\tv_mov_b32_e32 v61, 0
"""


def test_scan_finds_writes_of_a_wide_store_s_data_inside_the_wait_states():
    hits = _module().scan(STORES.splitlines())
    found = [(writer.split()[1], store.split()[0]) for _, _, writer, store in hits]
    assert found == [("v12,", "global_store_dwordx4"), ("v43,", "global_store_dwordx4"), ("v61,", "buffer_store_dwordx4")]


RESULTS = """
kernel_d:
\tv_mfma_f32_16x16x32_f16 a[0:3], v[30:33], v[2:5], a[0:3]
\tv_mfma_f32_16x16x32_f16 a[4:7], v[30:33], v[6:9], a[4:7]
\tv_accvgpr_read_b32 v40, a2
\tv_accvgpr_read_b32 v41, a5
\ts_nop 5
\tv_accvgpr_read_b32 v42, a6
\tv_mfma_f32_16x16x32_f16 v[10:13], v[30:33], v[6:9], v[10:13]
\tv_mfma_f32_16x16x32_f16 v[10:13], v[34:37], v[6:9], v[10:13]
\ts_nop 6
\tds_write_b128 v50, v[10:13]
\ts_nop 0
\tglobal_store_dwordx4 v[52:53], v[10:13], off
\tv_mfma_f32_16x16x32_f16 a[8:11], v[30:33], v[6:9], a[8:11]
\ts_branch .LBB0_1
.LBB0_2:
\tv_accvgpr_write_b32 a8, 0
"""


def test_scan_finds_uses_of_an_mfma_result_inside_its_wait_states():
    hits = _module().scan(RESULTS.splitlines())
    found = [(user.split()[0], user.split()[1]) for _, _, user, _ in hits]
    assert found == [("v_accvgpr_read_b32", "v40,"), ("v_accvgpr_read_b32", "v41,"), ("ds_write_b128", "v50,")]


def test_built_kernels_are_clean():
    """Whatever device assembly the last build kept has no such pair (the build itself refuses to link otherwise)."""
    mod = _module()
    for path in glob.glob(os.path.join(PKG, "build", "*-gfx950.s")):
        assert mod.scan_file(path) == [], path
