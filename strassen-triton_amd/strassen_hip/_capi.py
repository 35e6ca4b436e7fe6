"""ctypes binding of libstrassen_hip.so (the C ABI declared in include/strassen_hip.h, and the
test hooks of include/strassen_hip_debug.h).

Nothing here falls back to another implementation: if the shared library is missing the
import of any product module fails with the build command to run.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libstrassen_hip.so")

# name -> (restype, argtypes); must list every symbol the two headers declare
_i64, _int, _vp, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t
_p64 = ctypes.POINTER(ctypes.c_int64)
SIGNATURES = {
    "sthip_gemm": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _p64, _p64, _p64,
                          _int, _int, _int, _int, _int, _vp, _sz, _vp]),
    "sthip_gemm_static": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _p64, _p64, _p64,
                                 _int, _int, _int, _int, _int, _vp]),
    "sthip_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _int, _int, _int, _int]),
    "sthip_strassen_matmul_n_layers": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                              _int, _int, _vp, _sz, _vp]),
    "sthip_run_accumulate": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int,
                                    _vp, _sz, _vp]),
    "sthip_linear_strassen_forward": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _vp, _sz, _vp]),
    "sthip_linear_forward": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp, _sz, _vp]),
    "sthip_auto_levels": (_int, [_i64, _i64, _i64, _int, _int]),
    "sthip_linear_weight_sums_bytes": (_sz, [_i64, _i64, _int, _int]),
    "sthip_linear_prepare_weight": (_int, [_vp, _i64, _i64, _int, _int, _vp, _sz, _vp]),
    "sthip_linear_forward_prepared": (_int, [_vp, _vp, _vp, _sz, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp, _sz, _vp]),
    "sthip_last_error": (ctypes.c_char_p, []),
    "sthip_version": (_int, []),
    "sthip_debug_transpose_read": (_int, [_vp, _vp]),
    "sthip_debug_set_stages": (_int, [_int]),
    "sthip_debug_force_tile": (_int, [ctypes.c_char_p]),
    "sthip_debug_one_launch_counters": (_int, [_vp, _i64, _i64, _i64, ctypes.POINTER(ctypes.c_uint), _vp]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the library once and attach the prototypes."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python strassen-triton_amd/build.py` "
                "(hipcc, --offload-arch=gfx950). There is no fallback implementation.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


class SthipError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libstrassen_hip error {code}: {message}")
        self.code = code


def check(code: int) -> None:
    if code != 0:
        raise SthipError(code, load().sthip_last_error().decode())
