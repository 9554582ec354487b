"""ctypes binding of ``libqmm.so`` (declarations in ``include/qmm.h``)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libqmm.so")

QMM_F32, QMM_BF16, QMM_F16 = 0, 1, 2
QMM_FLAG_W_BF16 = 1
QMM_FLAG_ACT_Q8K = 2
QMM_FLAG_OUT_BF16 = 4
QMM_STATIC_SCRATCH_BYTES = 64 * 1024 * 1024


class GptqConfig(C.Structure):
    _fields_ = [("bits", C.c_int32), ("group_size", C.c_int32), ("desc_act", C.c_int32), ("sym", C.c_int32)]


_i64, _int, _vp = C.c_int64, C.c_int, C.c_void_p

# name -> (restype, argtypes); every symbol include/qmm.h declares
SIGNATURES = {
    "qmm_version": (_int, []),
    "qmm_last_error": (C.c_char_p, []),
    "qmm_block_params": (_int, [_int, C.POINTER(_i64), C.POINTER(_i64)]),
    "qmm_device_info": (_int, [C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "qmm_read_probe": (_int, [_vp, _i64, _vp]),
    "qmm_mfma_probe": (_int, [_vp, _i64, _int, _int, C.POINTER(_i64), _vp]),
    "qmm_dequantize": (_int, [_int, _vp, _i64, _i64, _vp, _int, _vp]),
    "qmm_dequantize_gptq": (_int, [C.POINTER(GptqConfig), _vp, _vp, _vp, _vp, _i64, _i64, _vp, _int, _vp]),
    "qmm_quantize": (_int, [_int, _vp, _i64, _i64, _vp, _vp]),
    "qmm_quantize_gptq": (_int, [C.POINTER(GptqConfig), _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "qmm_matmul_workspace_bytes": (_i64, [_int, _int, _i64, _i64, _i64]),
    "qmm_matmul_workspace_bytes_flags": (_i64, [_int, _int, _i64, _i64, _i64, _int]),
    "qmm_matmul": (_int, [_int, C.POINTER(GptqConfig), _vp, _int, _i64, _i64, C.POINTER(_vp), _int, _i64, _vp, _vp,
                          _i64, _int, _vp]),
    "qmm_matmul_static": (_int, [_int, C.POINTER(GptqConfig), _vp, _int, _i64, _i64, C.POINTER(_vp), _int, _i64, _vp, _int,
                                 _vp]),
    "qmm_repack_bytes": (_i64, [_int, C.POINTER(GptqConfig), _i64, _i64]),
    "qmm_repack": (_int, [_int, C.POINTER(GptqConfig), C.POINTER(_vp), _int, _i64, _i64, _vp, _i64, _vp]),
    "qmm_repack_check": (_int, [_int, C.POINTER(GptqConfig), _i64, _i64, _vp, _i64, _vp]),
    "qmm_matmul_repacked_workspace_bytes": (_i64, [_int, _int, _i64, _i64, _i64]),
    "qmm_matmul_repacked": (_int, [_int, C.POINTER(GptqConfig), _vp, _int, _i64, _i64, C.POINTER(_vp), _int, _vp, _i64, _i64, _vp,
                                   _vp, _i64, _int, _vp]),
    "qmm_matmul_grouped": (_int, [_int, _vp, _int, _i64, _i64, _int, C.POINTER(_vp), C.POINTER(_i64), C.POINTER(_vp), _vp,
                                  _i64, _vp]),
    "qmm_matmul_swiglu_workspace_bytes": (_i64, [_int, _int, _i64, _i64, _i64]),
    "qmm_matmul_swiglu": (_int, [_int, _vp, _int, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _i64, _vp]),
    "qmm_matmul_rmsnorm_workspace_bytes": (_i64, [_int, _int, _i64, _i64, _i64, _int]),
    "qmm_matmul_rmsnorm": (_int, [_int, C.POINTER(GptqConfig), _vp, _int, _vp, C.c_float, _i64, _i64, C.POINTER(_vp), _int, _i64,
                                  _vp, _vp, _i64, _int, _vp]),
    "qmm_block_dots_q4_0": (_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp]),
}

_lib = None


def load() -> C.CDLL:
    """dlopen the library; a missing build is an error, never a fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is not built; run `python -m mojo_amd.build` (hipcc, gfx950). "
                "There is no fallback path without it.")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class QmmError(RuntimeError):
    pass


def check(rc: int, what: str) -> None:
    if rc == 0:
        return
    msg = load().qmm_last_error().decode("utf-8", "replace")
    if rc == -1:
        raise ValueError(f"{what}: {msg}")
    if rc == -2:
        raise NotImplementedError(f"{what}: {msg}")
    raise QmmError(f"{what} failed ({rc}): {msg}")
