"""ctypes binding of libi_core.so (the C ABI declared in include/i.h and include/i_hip.h).

The library is looked up like the reference frontend does it
(ilang-python/ilang.py:6-28): the ILANG_CORE_LIB override first, then beside
this package.  There is no fallback: a missing library is an error.
"""
import ctypes
import os
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent


def _load():
    # PyTorch bundles its own HIP runtime; when both live in one process the
    # runtime must be torch's, so let torch load first if it is around.
    if "torch" not in sys.modules and os.environ.get("ILANG_NO_TORCH") is None:
        try:
            import torch  # noqa: F401
        except Exception:
            pass
    override = os.environ.get("ILANG_CORE_LIB")
    path = Path(override) if override else PKG / "libi_core.so"
    if not path.exists():
        raise RuntimeError(f"could not find i-core library at {path}; run `python -m i_amd.build`")
    return ctypes.CDLL(str(path))


core = _load()

vp = ctypes.c_void_p
sz = ctypes.c_size_t

core.i_error.argtypes = []
core.i_error.restype = ctypes.c_char_p

core.i_hip_attention.argtypes = [vp, vp, vp, vp, ctypes.c_int, ctypes.c_int, sz, sz, sz, sz, sz, ctypes.c_float, vp]
core.i_hip_attention.restype = ctypes.c_int
core.i_hip_attention_ex.argtypes = [vp, vp, vp, vp, ctypes.c_int, ctypes.c_int, sz, sz, sz, sz, sz, ctypes.c_float, sz, sz,
                                    ctypes.c_int, vp]
core.i_hip_attention_ex.restype = ctypes.c_int
core.i_hip_attention_opt.argtypes = [vp, vp, vp, vp, ctypes.c_int, ctypes.c_int, sz, sz, sz, sz, sz, ctypes.c_float, sz, sz,
                                     ctypes.c_char_p, vp]
core.i_hip_attention_opt.restype = ctypes.c_int
core.i_hip_gemm_opt.argtypes = [vp, vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, sz, sz, sz, sz, ctypes.c_char_p, vp]
core.i_hip_gemm_opt.restype = ctypes.c_int
core.i_hip_program_clock_probe.argtypes = [vp, vp]
core.i_hip_program_clock_probe.restype = ctypes.c_int
core.i_hip_shader_clock_probe.argtypes = [vp, ctypes.c_uint, vp]
core.i_hip_shader_clock_probe.restype = ctypes.c_int
core.i_hip_release_cached_memory.argtypes = []
core.i_hip_release_cached_memory.restype = sz
core.i_hip_program_option.argtypes = [vp, ctypes.c_char_p, ctypes.c_int]
core.i_hip_program_option.restype = ctypes.c_int
core.i_hip_program_report.argtypes = [vp]
core.i_hip_program_report.restype = vp
core.i_hip_program_row_slices.argtypes = [vp, ctypes.POINTER(ctypes.c_ubyte), ctypes.c_size_t]
core.i_hip_program_row_slices.restype = ctypes.c_int
core.i_hip_gemm_nt_bf16.argtypes = [vp, vp, vp, sz, sz, sz, sz, vp]
core.i_hip_gemm_nt_bf16.restype = ctypes.c_int
core.i_hip_gemm_nt_bf16_ex.argtypes = [vp, vp, vp, ctypes.c_int, sz, sz, sz, sz, sz, sz, vp]
core.i_hip_gemm_nt_bf16_ex.restype = ctypes.c_int
core.i_hip_gemm_nn_bf16.argtypes = [vp, vp, vp, sz, sz, sz, sz, vp]
core.i_hip_gemm_nn_bf16.restype = ctypes.c_int
core.i_hip_gemm_nt_f32.argtypes = [vp, vp, vp, sz, sz, sz, sz, vp]
core.i_hip_gemm_nt_f32.restype = ctypes.c_int
core.i_hip_row_softmax.argtypes = [vp, vp, sz, sz, vp]
core.i_hip_row_softmax.restype = ctypes.c_int
core.i_hip_convert.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, sz, vp]
core.i_hip_convert.restype = ctypes.c_int

F32, BF16 = 0, 1


def last_error():
    err = core.i_error()
    return err.decode() if err else "i-core error"


def check(code):
    if code != 0:
        raise RuntimeError(last_error())


def check_ptr(ptr):
    if not ptr:
        raise RuntimeError(last_error())
    return ptr
