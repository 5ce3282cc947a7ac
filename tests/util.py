"""Helpers shared by the tests: golden-vector loading and seeded workload construction."""
from __future__ import annotations

import json
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def load_golden(name: str):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def bits_to_tensor(bits, dtype: str) -> torch.Tensor:
    """list of binary32 bit patterns (exactly representable in `dtype`) -> 1-D tensor of that dtype"""
    f = torch.from_numpy(np.array(bits, dtype=np.uint32).view(np.float32).copy())
    t = f.to(DTYPES[dtype])
    assert torch.equal(t.float(), f), "golden input is not representable in its dtype"
    return t


def f32_from_bits(bits) -> torch.Tensor:
    return torch.from_numpy(np.array(bits, dtype=np.uint32).view(np.float32).copy())


def outlier_tensor(M: int, K: int, dtype=torch.bfloat16, seed: int = 0, frac: float = 1e-3, scale: float = 50.0):
    """~N(0,1) with a seeded `frac` of the entries multiplied by `scale` (the round-trip workload)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    E = M * K
    g1 = torch.Generator().manual_seed(seed + 1)
    n_out = int(E * frac)
    if n_out:
        pos = torch.randperm(E, generator=g1)[:n_out]            # distinct positions: exactly n_out outliers
        x.view(-1)[pos] *= scale
    return x.to(dtype)


class config_as:
    """set block_linear_config.GROUP_SIZE / INPUT_OUTPUT_TORCH_TYPE for the duration of a with-block"""

    def __init__(self, pkg, block=None, out=None):
        self.cfg, self.block, self.out = pkg.block_linear_config, block, out

    def __enter__(self):
        self.old = (self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE)
        if self.block:
            self.cfg.GROUP_SIZE = self.block
        if self.out:
            self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.out

    def __exit__(self, *a):
        self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.old


def gemm_reference(A, W, sa, sw, block, bias, out_dtype):
    """the CPU checker's GEMM output for int8 codes A [M,K], W [N,K] and scales [nblk,M], [nblk,N], and the magnitude
    sum_j |term_j| that bounds what a different fp32 summation order can change"""
    from oracle import oracle_torch
    P = oracle_torch.gemm_nt_partials(A, W, block)
    ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw, block, bias, out_dtype)
    mag = torch.zeros(P.shape[1:], dtype=torch.float64)
    for j in range(P.shape[0]):
        mag += P[j].abs().double() * sa[j].double()[:, None] * sw[j].double()[None, :]
    return ref, mag / (127.0 * 127.0)


def assert_gemm_close(C, ref, mag, tol):
    """|C - ref| <= tol * |ref| + 4e-6 * mag elementwise (tol = 1e-3 for fp32 outputs, 1e-2 for 16-bit outputs)"""
    err = (C.double() - ref.double()).abs()
    bound = tol * ref.double().abs() + 4e-6 * mag + 1e-30
    if not (err <= bound).all():
        i = (err - bound).argmax()
        raise AssertionError(f"max violation at flat index {i.item()}: got {C.reshape(-1)[i].item()} want {ref.reshape(-1)[i].item()} "
                             f"(err {err.reshape(-1)[i].item():.3e}, bound {bound.reshape(-1)[i].item():.3e})")


def assert_close_rms(got, ref, tol, bias=None):
    """elementwise |got - ref| <= tol * (|ref| + |bias|) + 3e-4 * rms(ref): the relative bound of the output type, plus
    an absolute term for elements that are small through cancellation (their error scales with the terms, not the
    sum).  The bias is added to the ROUNDED product in the output type (triton_functions.py:127-131), so where product
    and bias cancel, one unit in the last place of the product is large against the sum: the relative bound counts both,
    and the second rounding (of the sum) may move the result by one more unit in the last place of the output type."""
    ulp = {torch.float32: 2.0 ** -23, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[got.dtype]
    got, ref = got.double(), ref.double()
    rms = ref.pow(2).mean().sqrt().item()
    err = (got - ref).abs()
    bound = tol * ref.abs() + 3e-4 * rms + 1e-30
    if bias is not None:
        bound = bound + 2 * tol * bias.double().abs() + ulp * ref.abs()
    if not (err <= bound).all():
        i = (err - bound).argmax()
        raise AssertionError(f"{int((err > bound).sum())} of {err.numel()} outside the bound; worst at flat index {i.item()}: got "
                             f"{got.reshape(-1)[i].item()} want {ref.reshape(-1)[i].item()} (rms {rms:.3e})")
