"""The in-scope names of the reference's ``triton_functions`` module (triton_functions.py:142, :218, :221, :492, :510,
:533), so that ``from triton_functions import ...`` lines keep working once
:func:`blockwise_int8_linear_amd.compat.install` has registered this module under that name.  Everything here runs the
HIP kernels of libbi8.so; the reference's broken or dead helpers (plain ``int8_matmul``, ``groupwise_quantize``) are
not provided.

``python -m blockwise_int8_linear_amd.triton_functions`` prints the reference's own sweep (M = N from 2048 to 14336,
K = 512, triton_functions.py:521-566) as a table of TOP/s."""
from __future__ import annotations

import torch

from . import block_linear_config
from .ops import (  # noqa: F401
    ceil_div,
    dequantize_block_rowwise,
    int8_matmul_block64_rowwise_dequantize,
    quantize_block_rowwise,
)

__all__ = ["ceil_div", "dequantize_block_rowwise", "int8_matmul_block64_rowwise_dequantize", "quantize_block_rowwise",
           "fast_matmulT", "copy_then_matmul", "benchmark"]


def fast_matmulT(a, b):
    """a [M,K] @ b [N,K].T with both operands block-quantized on the fly (triton_functions.py:510-513)."""
    a_int8, a_state = quantize_block_rowwise(a)
    b_int8, b_state = quantize_block_rowwise(b)
    return int8_matmul_block64_rowwise_dequantize(a_int8, b_int8.t(), a_state, b_state)


def copy_then_matmul(a, b):
    """dense matmul plus one copy of each operand: the memory traffic of a quantize pass (triton_functions.py:515-518)"""
    return torch.matmul(torch.clone(a), torch.clone(b))


def _do_bench(fn, warmup=5, rep=20, quantiles=(0.5, 0.2, 0.8)):
    """milliseconds per call at the given quantiles; one pair of events per call, like triton.testing.do_bench"""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(rep):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    t = torch.tensor(times)
    return [torch.quantile(t, q).item() for q in quantiles]


def benchmark(sizes=None, K=512, providers=("dense", "int8 matmul", "blockwise_int8", "blockwise_int8_quantise", "dense+copy"),
              print_data=True):
    """The reference's sweep (triton_functions.py:521-566): square M = N, fixed K = 512, operands of
    INPUT_OUTPUT_TORCH_TYPE; TOP/s = 2*M*N*K / median time, with the 0.2 / 0.8 quantiles.
      dense                    torch.matmul in bf16 (hipBLASLt)               -- the reference's 'cublas' line
      int8 matmul              the vendor library's plain int8 GEMM, int32 out, no scales (torch._int_mm, hipBLASLt) on
                               the quantized codes -- the reference's line of that name (triton_functions.py:547-552, there
                               through its torch_cublas_matmul_int8 extension)
      blockwise_int8           the int8 GEMM with fused dequantize alone, operands quantized beforehand
      blockwise_int8_quantise  quantize both operands + that GEMM
      dense+copy               copy_then_matmul
    Returns {provider: [(M, median, q80, q20), ...]}."""
    sizes = sizes or [1024 * i for i in range(2, 16, 2)]
    dtype = block_linear_config.INPUT_OUTPUT_TORCH_TYPE
    rows = {p: [] for p in providers}
    for M in sizes:
        N = M
        a = torch.randn((M, K), device="cuda", dtype=dtype)
        b = torch.randn((K, N), device="cuda", dtype=dtype)
        for p in providers:
            if p == "dense":
                a16, b16 = a.to(torch.bfloat16), b.to(torch.bfloat16)
                fn = lambda: torch.matmul(a16, b16)
            elif p == "int8 matmul":
                qa, _ = quantize_block_rowwise(a)
                qb, _ = quantize_block_rowwise(b.t().contiguous())
                qbt = qb.t()                        # [K,N], K contiguous: the layout the blockwise GEMM is given too
                fn = lambda: torch._int_mm(qa, qbt)
            elif p == "dense+copy":
                fn = lambda: copy_then_matmul(a, b)
            elif p == "blockwise_int8":
                bt = b.t().contiguous()
                qa, sa = quantize_block_rowwise(a)
                qb, sb = quantize_block_rowwise(bt)
                fn = lambda: int8_matmul_block64_rowwise_dequantize(qa, qb.t(), sa, sb)
            elif p == "blockwise_int8_quantise":
                bt = b.t().contiguous()
                fn = lambda: fast_matmulT(a, bt)
            else:
                raise ValueError(f"unknown provider {p!r}")
            ms, lo, hi = _do_bench(fn)
            perf = lambda t: 2 * M * N * K * 1e-12 / (t * 1e-3)
            rows[p].append((M, perf(ms), perf(hi), perf(lo)))
    if print_data:
        print(f"{'M=N':>7} " + " ".join(f"{p:>24}" for p in providers) + f"   (TOP/s, K={K}, block {block_linear_config.GROUP_SIZE})")
        for i, M in enumerate(sizes):
            print(f"{M:>7} " + " ".join(f"{rows[p][i][1]:>24.1f}" for p in providers))
    return rows


if __name__ == "__main__":
    benchmark()
