#!/usr/bin/env python3
"""Build libspiral_mi355.so (HIP, gfx950) in-tree.

    python spiral-s-ml-library_amd/build.py [--force]

hipcc cross-compiles for gfx950 without a GPU.  The shared library is written next to this file;
the Python host modules under ml/ load it with ctypes and fail loudly when it is missing.
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libspiral_mi355.so")
SOURCES = ["api.hip", "row_ops.hip", "elementwise.hip", "gemm.hip", "mlp.hip", "mlp_packed.hip", "mlp_resident.hip", "mlp_pipe.hip", "mlp_ensemble.hip"]
# sources with MFMAs or wide stores in inline asm: their device assembly is kept and scanned (isa_check.py)
ASM_MFMA_SOURCES = ["gemm.hip", "mlp.hip", "mlp_packed.hip", "mlp_resident.hip", "mlp_pipe.hip", "mlp_ensemble.hip", "row_ops.hip", "elementwise.hip"]
# Kernel-argument preloading (gfx950): the first 14 dwords of a kernel's leading scalar parameters arrive in
# registers with the wave instead of through a scalar load at kernel entry (a struct parameter is not preloaded;
# the kernels that gain from it repeat the fields their first loads need as leading scalars).
EXTRA_FLAGS = {}
FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"),
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-value",
         "-Wno-unknown-warning-option",
         # the DMA blocks name M0 as clobbered; the compiler notes that M0 is a reserved register, once per use
         "-Wno-inline-asm",
         "-mllvm", "-amdgpu-kernarg-preload-count=14"]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(ln for ln in p.stdout.splitlines() if "packed-fp32-ops" not in ln)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def device_asm(src):
    return os.path.join(OBJ, src.replace(".hip", "") + "-hip-amdgcn-amd-amdhsa-gfx950.s")


def check_isa():
    """Scan the kept device assembly; raises on a vector-ALU write right in front of an MFMA that reads the register
    or right behind a store of more than 8 bytes that has it as data, and on a use of an MFMA's result too early."""
    sys.path.insert(0, HERE)
    try:
        import isa_check
    finally:
        sys.path.pop(0)
    for src in ASM_MFMA_SOURCES:
        path = device_asm(src)
        if not os.path.exists(path):
            continue
        hits = isa_check.scan_file(path)
        if hits:
            ln, kernel, writer, other = hits[0]
            raise RuntimeError("%s: %d hazards the hardware does not interlock, first at line %d in %s: '%s' next to '%s'"
                               % (path, len(hits), ln, kernel, writer, other))


def build(force=True, verbose=False):
    """Compile every HIP source and link the shared library.  Returns the library path."""
    os.makedirs(OBJ, exist_ok=True)
    cc = hipcc()
    headers = [os.path.join(CSRC, "common.h"), os.path.join(CSRC, "mlp_common.h"), os.path.join(CSRC, "philox.h"), os.path.join(ROOT, "include", "spiral_mi355.h")]
    newest_header = max(os.path.getmtime(h) for h in headers)

    def compile_one(src):
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ, src.replace(".hip", ".o"))
        if not force and os.path.exists(o) and os.path.getmtime(o) > max(os.path.getmtime(s), newest_header):
            return o
        keep = ["-save-temps=obj"] if src in ASM_MFMA_SOURCES else []
        out = _run([cc] + FLAGS + EXTRA_FLAGS.get(src, []) + keep + ["-c", s, "-o", o])
        if verbose and out.strip():
            print(out)
        if keep:        # of the intermediate files only the device assembly stays
            stem = os.path.join(OBJ, src.replace(".hip", ""))
            for tmp in glob.glob(stem + "-hip-*") + glob.glob(stem + "-host-*") + glob.glob(stem + ".hip-hip-*"):
                if tmp != device_asm(src):
                    os.remove(tmp)
        return o

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    check_isa()
    _run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
