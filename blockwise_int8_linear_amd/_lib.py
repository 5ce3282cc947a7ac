"""ctypes binding of libbi8.so (the C ABI declared in include/bi8.h).

The library is built in-tree by ``blockwise_int8_linear_amd.build`` (hipcc, gfx950).  There is no
fallback: if the shared object is missing or an entry point fails, the operators raise.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbi8.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "bi8.h")
ABI_VERSION = 5

_i64, _vp, _ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int

# name -> (restype, argtypes); mirrors include/bi8.h one to one
SIGNATURES = {
    "bi8_version": (_ci, []),
    "bi8_strerror": (ctypes.c_char_p, [_ci]),
    "bi8_quantize_rowwise": (_ci, [_vp, _ci, _vp, _vp, _i64, _i64, _i64, _i64, _ci, _vp]),
    "bi8_quantize_transposed": (_ci, [_vp, _ci, _vp, _vp, _i64, _i64, _i64, _i64, _ci, _vp]),
    "bi8_quantize_dual": (_ci, [_vp, _ci, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _ci, _vp]),
    "bi8_colsum_workspace_bytes": (_i64, [_i64, _i64]),
    "bi8_quantize_dual_colsum": (_ci, [_vp, _ci, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _ci, _vp]),
    "bi8_dequantize_rowwise": (_ci, [_vp, _vp, _vp, _ci, _i64, _i64, _i64, _i64, _ci, _vp]),
    "bi8_gemm_nt_dequant": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _vp, _ci, _i64, _i64, _i64, _i64, _i64, _i64, _ci, _vp]),
    "bi8_gemm_nt_dequant_ws": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _vp, _ci, _i64, _i64, _i64, _i64, _i64, _i64, _ci, _vp, _i64, _vp]),
    "bi8_gemm_workspace_bytes": (_i64, [_i64, _i64, _i64, _ci]),
    "bi8_static_scratch_bytes": (_i64, []),
    "bi8_gemm_nt_dequant_static": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _vp, _ci, _i64, _i64, _i64, _i64, _i64, _i64, _ci, _vp]),
    "bi8_gemm_kernel_name": (ctypes.c_char_p, [_i64, _i64, _i64, _i64, _i64, _ci, _i64]),
    "bi8_gemm_nt_partials": (_ci, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _ci, _vp]),
    "bi8_linear_few_rows": (_ci, [_vp, _ci, _vp, _vp, _vp, _ci, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _ci, _vp]),
}

ERR_UNSUPPORTED = 6

_lib = None


class Bi8Error(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load libbi8.so and bind every entry point; raises if the library has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise Bi8Error(
                f"{LIB_PATH} is missing: build it with `python -m blockwise_int8_linear_amd.build` "
                "(hipcc, --offload-arch=gfx950). There is no CPU or PyTorch fallback for these operators.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        if lib.bi8_version() != ABI_VERSION:
            raise Bi8Error(f"libbi8.so has ABI version {lib.bi8_version()}, this package expects {ABI_VERSION}; rebuild it")
        _lib = lib
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().bi8_strerror(code).decode()
        raise Bi8Error(f"{what} failed: {msg} (code {code})")
