"""ctypes binding of libspiral_mi355.so (declared in include/spiral_mi355.h)."""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# (SPIRAL_MI355_LIB names another build of the same library, e.g. one with different tuning constants)
LIB_PATH = os.environ.get("SPIRAL_MI355_LIB") or os.path.join(os.path.dirname(_HERE), "libspiral_mi355.so")

SP_F32, SP_F16, SP_BF16 = 0, 1, 2
GEMM_RELU, GEMM_FORCE_GENERIC = 0x1, 0x100
(ROW_IDENTITY, ROW_SOFTMAX, ROW_MASKED_SOFTMAX, ROW_LN_L2, ROW_REGRET_MATCHING, ROW_MASKED_REGRET_MATCHING,
 ROW_INCLUSIVE_SCAN, ROW_EXCLUSIVE_SCAN) = range(8)
PHILOX_BLOCK, PHILOX_GRID, PHILOX_GATHER, PHILOX_LAYER = 0, 1, 2, 3
MAP_COPY, MAP_RELU, MAP_TANH, MAP_SIGMOID = 0, 1, 2, 3
REDUCE_SUM, REDUCE_PROD, REDUCE_MAX, REDUCE_MIN, REDUCE_AVERAGE = 0, 1, 2, 3, 4
MAP_IN_IDENTITY, MAP_IN_SQUARE, MAP_IN_ABS = 0, 1, 2
MAP_OUT_IDENTITY, MAP_OUT_SQRT = 0, 1
HEAD_NONE, HEAD_SOFTMAX, HEAD_REGRET_MATCHING, HEAD_SOFTMAX_RM = 0, 1, 2, 3

ERROR_NAMES = {0: "SP_OK", -1: "SP_ERR_NULL", -2: "SP_ERR_SHAPE", -3: "SP_ERR_ALIGN", -4: "SP_ERR_DTYPE",
               -5: "SP_ERR_ARG", -6: "SP_ERR_UNSUPPORTED", -7: "SP_ERR_DEVICE"}


class SpiralError(RuntimeError):
    """A C-ABI call returned a negative sp_status."""

    def __init__(self, code, message):
        super().__init__("%s (%d): %s" % (ERROR_NAMES.get(code, "?"), code, message))
        self.code = code


class PhiloxConfig(C.Structure):
    _fields_ = [("seed", C.c_uint64), ("offset", C.c_uint64), ("mode", C.c_int32), ("threads_per_block", C.c_int32),
                ("blocks_per_grid", C.c_int32), ("rows_per_block", C.c_int32), ("member_rows", C.c_int64),
                ("member_draws", C.c_uint64)]


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64), ("compute_units", C.c_int32),
                ("wavefront_size", C.c_int32), ("lds_bytes_per_cu", C.c_int32), ("max_clock_khz", C.c_int32),
                ("hbm_bytes", C.c_int64), ("l2_bytes", C.c_int32)]


class KernelInfo(C.Structure):
    _fields_ = [("vgprs", C.c_int32), ("sgprs", C.c_int32), ("static_lds_bytes", C.c_int32),
                ("threads_per_block", C.c_int32), ("max_blocks_per_cu", C.c_int32)]


_P, _I64, _I32, _U32, _F = C.c_void_p, C.c_int64, C.c_int32, C.c_uint32, C.c_float

SIGNATURES = {
    "sp_last_error_string": (C.c_char_p, []),
    "sp_device_info": (C.c_int, [C.POINTER(DeviceInfo)]),
    "sp_kernel_info": (C.c_int, [C.c_char_p, C.POINTER(KernelInfo)]),
    "sp_clock_sample": (C.c_int, [_P, _P]),
    "sp_gemm_abt": (C.c_int, [C.c_int, C.c_int, _P, _P, _P, _P, _I64, _I64, _I64, _F, _F, _U32, _P]),
    "sp_gemm_abt_batched": (C.c_int, [C.c_int, C.c_int, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _F, _F,
                                      _U32, _P]),
    "sp_gemm_config": (C.c_int, [C.c_int, _I64, _I64, _I64] + [C.POINTER(C.c_int32)] * 4),
    "sp_row_ops": (C.c_int, [_P] * 8 + [_I64, _I64, _U32, _P]),
    "sp_row_map_f32": (C.c_int, [C.c_int, _P, _P, _I64, _I64, _I32, _P]),
    "sp_row_map_i32": (C.c_int, [C.c_int, _P, _P, _I64, _I64, _P]),
    "sp_row_sample": (C.c_int, [C.c_int, _P, _P, C.POINTER(PhiloxConfig), _P, _P, _P, _P, _P, _I64, _I64, _I32, _P]),
    "sp_philox_uniforms": (C.c_int, [C.POINTER(PhiloxConfig), _P, _I64, _I64, _P]),
    "sp_row_get_prob": (C.c_int, [C.c_int, _P, _P, _P, _I64, _I64, _I32, _P]),
    "sp_cem_resample": (C.c_int, [_P, _P, _P, _P, _I64, _I64, C.c_float, C.c_float, _P]),
    "sp_cem_resample_philox": (C.c_int, [_P, _P, C.c_uint64, C.c_uint64, _P, _I64, _I64, C.c_float, C.c_float, _P]),
    "sp_cem_update_mask": (C.c_int, [_P, _P, _I64, _P]),
    "sp_row_reduce_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, _P, _P, _I64, _I64, _P]),
    "sp_row_binarize": (C.c_int, [_P, _P, _I64, _I64, C.c_uint32, _P]),
    "sp_map_f32": (C.c_int, [C.c_int, _P, _P, _I64, _P]),
    "sp_row_l1_normalize": (C.c_int, [_P, _P, _I64, _I64, C.c_float, _P]),
    "sp_reduce": (C.c_int, [C.c_int, C.c_int, _P, _P, _I64, _P, _I64, _P]),
    "sp_reduce_status": (C.c_int, [_P, _I64, C.POINTER(C.c_int64), _P]),
    "sp_reduce_set_poll_limit": (C.c_int, [_I64]),
    "sp_reduce_sum": (C.c_int, [C.c_int, _P, _P, _I64, _P, _I64, _P]),
    "sp_reduce_workspace_bytes": (C.c_int64, []),
    "sp_reduce_sum_static": (C.c_int, [C.c_int, _P, _P, _I64, _P]),
    "sp_reduce_sum_static_max_n": (C.c_int64, []),
    "sp_transpose_inner_b32": (C.c_int, [_P, _P, _I64, _I64, _I64, _P]),
    "sp_mlp_forward": (C.c_int, [C.c_int, _P, _I32, C.POINTER(_P), C.POINTER(_P), C.POINTER(C.c_int32), _P,
                                 C.POINTER(PhiloxConfig), _P, _P, _P, _I64, _I32, _I32, _P]),
    "sp_mlp_packed_bytes": (C.c_int64, [_I32, C.POINTER(C.c_int32)]),
    "sp_mlp_pack_weights": (C.c_int, [C.c_int, _I32, C.POINTER(_P), C.POINTER(C.c_int32), _P, _I64, _P]),
    "sp_mlp_forward_packed": (C.c_int, [C.c_int, _P, _I32, _P, _I64, C.POINTER(_P), C.POINTER(C.c_int32), _P,
                                        C.POINTER(PhiloxConfig), _P, _P, _P, _I64, _I32, _I32, _P]),
    "sp_mlp_forward_ensemble": (C.c_int, [C.c_int, _P, _I32, C.POINTER(_P), C.POINTER(C.c_int32), _I32, _P,
                                          C.POINTER(PhiloxConfig), _P, _P, _I64, _I32, _I32, _P]),
    "sp_ensemble_binarize": (C.c_int, [C.c_int, _P, _P, _P, _I32, _I64, _I32, _I32, _U32, _P]),
}


def load(path=LIB_PATH):
    if not os.path.exists(path):
        raise RuntimeError("%s is missing: build it with `python spiral-s-ml-library_amd/build.py` "
                           "(there is no CPU fallback)" % path)
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


# Entry points that launch work; their last argument is the stream.
LAUNCHES = frozenset(("sp_gemm_abt", "sp_gemm_abt_batched", "sp_row_ops", "sp_row_map_f32", "sp_row_map_i32",
                      "sp_row_sample", "sp_philox_uniforms", "sp_row_get_prob", "sp_cem_resample", "sp_cem_resample_philox",
                      "sp_row_reduce_f32", "sp_cem_update_mask",
                      "sp_row_binarize", "sp_map_f32", "sp_reduce_sum", "sp_reduce", "sp_row_l1_normalize", "sp_reduce_sum_static", "sp_transpose_inner_b32", "sp_mlp_forward", "sp_mlp_pack_weights",
                      "sp_mlp_forward_packed", "sp_mlp_forward_ensemble", "sp_ensemble_binarize"))


class Tape:
    """The launches of one pass over a fixed set of tensors, recorded while they ran and replayable with a fresh stream
    argument.  `keep` holds every tensor whose address went into a call, so temporaries the host functions allocated
    stay alive as long as the tape does."""

    def __init__(self):
        self.calls, self.keep = [], []

    def replay(self):
        stream = stream_ptr()
        for fn, args in self.calls:
            rc = fn(*args, stream)
            if rc != 0:
                check(rc)


_tape = None


def start_tape():
    """Every launch through `lib` from now until stop_tape() is also recorded."""
    global _tape
    _tape = Tape()
    return _tape


def stop_tape():
    global _tape
    _tape = None


class _Library:
    """The C-ABI library; launches pass through a thin wrapper that feeds the active tape, if any."""

    def __init__(self, cdll):
        self._cdll = cdll

    def __getattr__(self, name):
        fn = getattr(self._cdll, name)
        if name in LAUNCHES:
            raw = fn

            def fn(*args):
                rc = raw(*args)
                if _tape is not None and rc == 0:
                    _tape.calls.append((raw, args[:-1]))
                return rc
        setattr(self, name, fn)     # looked up once
        return fn


lib = _Library(load())


def check(rc):
    if rc != 0:
        raise SpiralError(rc, lib.sp_last_error_string().decode())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr():
    """torch's current HIP stream as a hipStream_t.  The raw query skips the Stream object, which costs
    several microseconds per call: as much as a small kernel."""
    if _raw_stream is not None:
        return C.c_void_p(_raw_stream(torch.cuda.current_device()))
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


DTYPES = {torch.float32: SP_F32, torch.float16: SP_F16, torch.bfloat16: SP_BF16}


def ptr(t, dtype=None, name="tensor"):
    """Device pointer of a contiguous ROCm tensor (None passes through as NULL)."""
    if t is None:
        return None
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor" % name)
    if not t.is_cuda:
        raise ValueError("%s must live on the GPU (got %s)" % (name, t.device))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous (row-major, innermost stride 1)" % name)
    if dtype is not None and t.dtype != dtype:
        raise TypeError("%s must have dtype %s, got %s" % (name, dtype, t.dtype))
    if _tape is not None:
        _tape.keep.append(t)
    return C.c_void_p(t.data_ptr())


def device_info():
    info = DeviceInfo()
    check(lib.sp_device_info(C.byref(info)))
    return {f: (getattr(info, f).decode() if isinstance(getattr(info, f), bytes) else getattr(info, f))
            for f, _ in DeviceInfo._fields_}


def kernel_info(name):
    """Registers / LDS / resident workgroups of a named kernel (ml/max_blocks_per_sm.py counterpart)."""
    info = KernelInfo()
    check(lib.sp_kernel_info(name.encode(), C.byref(info)))
    return {f: getattr(info, f) for f, _ in KernelInfo._fields_}
