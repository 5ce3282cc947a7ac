"""TEST INFRASTRUCTURE -- NOT PRODUCT CODE.

CPU checker for the blockwise int8 path: a scalar C restatement of the reference's
Triton kernels (``bi8_oracle.c``, loaded here through ctypes) and an independent
pure-PyTorch restatement (``oracle_torch.py``).  Only the tests, the smoke check and the
benchmark's CPU-baseline leg may import this package; the shipped package never does.

Function-by-function citations of the reference are in ``bi8_oracle.c``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
_libs: dict = {}


def build(force: bool = False) -> None:
    """Compile the C checker with gcc (both the one-thread and the OpenMP flavour)."""
    cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


def _lib(threads: bool = False):
    name = "libbi8_oracle_omp.so" if threads else "libbi8_oracle.so"
    if name not in _libs:
        path = os.path.join(_HERE, name)
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        lib.bi8o_quantize_rowwise.argtypes = [vp, ci, vp, vp, i64, i64, i64, i64, ci]
        lib.bi8o_quantize_transposed.argtypes = [vp, ci, vp, vp, i64, i64, i64, i64, ci]
        lib.bi8o_dequantize_rowwise.argtypes = [vp, vp, vp, ci, i64, i64, i64, i64, ci]
        lib.bi8o_gemm_nt_partials.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, ci]
        lib.bi8o_gemm_nt_dequant.argtypes = [vp, vp, vp, vp, vp, ci, vp, ci, i64, i64, i64, i64, i64, i64, ci]
        for f in ("bi8o_quantize_rowwise", "bi8o_quantize_transposed", "bi8o_dequantize_rowwise",
                  "bi8o_gemm_nt_partials", "bi8o_gemm_nt_dequant"):
            getattr(lib, f).restype = ci
        lib.bi8o_bf16_to_f32.argtypes = [ctypes.c_uint16]
        lib.bi8o_bf16_to_f32.restype = ctypes.c_float
        lib.bi8o_f32_to_bf16.argtypes = [ctypes.c_float]
        lib.bi8o_f32_to_bf16.restype = ctypes.c_uint16
        lib.bi8o_f16_to_f32.argtypes = [ctypes.c_uint16]
        lib.bi8o_f16_to_f32.restype = ctypes.c_float
        lib.bi8o_f32_to_f16.argtypes = [ctypes.c_float]
        lib.bi8o_f32_to_f16.restype = ctypes.c_uint16
        _libs[name] = lib
    return _libs[name]


def _cpu2d(t: torch.Tensor) -> torch.Tensor:
    assert t.dim() == 2, "2-D tensors only"
    return t.detach().cpu().contiguous()


def ceil_div(n: int, d: int) -> int:
    return -(n // -d)


def quantize_block_rowwise(x: torch.Tensor, block: int, threads: bool = False):
    """x [M,K] -> (int8 [M,K], fp32 scales [ceil(K/block), M])."""
    x = _cpu2d(x)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.int8)
    s = torch.empty((ceil_div(K, block), M), dtype=torch.float32)
    rc = _lib(threads).bi8o_quantize_rowwise(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), M, K, K, K, block)
    assert rc == 0
    return q, s


def quantize_block_transposed(x: torch.Tensor, block: int, threads: bool = False):
    """x [R,C] -> the quantization of x.t().contiguous(): (int8 [C,R], fp32 scales [ceil(R/block), C])."""
    x = _cpu2d(x)
    R, C = x.shape
    q = torch.empty((C, R), dtype=torch.int8)
    s = torch.empty((ceil_div(R, block), C), dtype=torch.float32)
    rc = _lib(threads).bi8o_quantize_transposed(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), R, C, C, R, block)
    assert rc == 0
    return q, s


def dequantize_block_rowwise(q: torch.Tensor, s: torch.Tensor, block: int, out_dtype=torch.bfloat16,
                             threads: bool = False):
    q = _cpu2d(q)
    s = _cpu2d(s).float()
    M, K = q.shape
    assert s.shape == (ceil_div(K, block), M)
    out = torch.empty((M, K), dtype=out_dtype)
    rc = _lib(threads).bi8o_dequantize_rowwise(q.data_ptr(), s.data_ptr(), out.data_ptr(), _DT[out_dtype], M, K, K, K, block)
    assert rc == 0
    return out


def gemm_nt_partials(a: torch.Tensor, w: torch.Tensor, block: int, threads: bool = False):
    """a int8 [M,K], w int8 [N,K] -> int32 [ceil(K/block), M, N] block partial dot products."""
    a, w = _cpu2d(a), _cpu2d(w)
    M, K = a.shape
    N, K2 = w.shape
    assert K == K2
    P = torch.empty((ceil_div(K, block), M, N), dtype=torch.int32)
    rc = _lib(threads).bi8o_gemm_nt_partials(a.data_ptr(), w.data_ptr(), P.data_ptr(), M, N, K, K, K, block)
    assert rc == 0
    return P


def gemm_nt_dequant(a: torch.Tensor, w: torch.Tensor, sa: torch.Tensor, sw: torch.Tensor, block: int,
                    bias=None, out_dtype=torch.bfloat16, threads: bool = False):
    """a int8 [M,K], w int8 [N,K] (the reference passes w.t()), sa [nblk,M], sw [nblk,N] -> [M,N]."""
    a, w = _cpu2d(a), _cpu2d(w)
    sa, sw = _cpu2d(sa).float(), _cpu2d(sw).float()
    M, K = a.shape
    N, K2 = w.shape
    nblk = ceil_div(K, block)
    assert K == K2 and sa.shape == (nblk, M) and sw.shape == (nblk, N)
    out = torch.empty((M, N), dtype=out_dtype)
    if bias is not None:
        bias = bias.detach().cpu().contiguous()
        assert bias.shape == (N,)
        bp, bd = bias.data_ptr(), _DT[bias.dtype]
    else:
        bp, bd = None, 0
    rc = _lib(threads).bi8o_gemm_nt_dequant(a.data_ptr(), w.data_ptr(), sa.data_ptr(), sw.data_ptr(), bp, bd,
                                           out.data_ptr(), _DT[out_dtype], M, N, K, K, K, N, block)
    assert rc == 0
    return out
