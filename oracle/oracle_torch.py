"""TEST INFRASTRUCTURE -- NOT PRODUCT CODE.

Pure-PyTorch (CPU, eager) restatement of the reference's blockwise int8 math.  The reference has no CPU
path (every launcher asserts ``x.is_cuda``, triton_functions.py:229, :496), so this file is the
"PyTorch CPU path" that the benchmark times on the host cores, and a second, independently written
checker next to ``bi8_oracle.c``.  Eager torch ops round once per op, so the arithmetic is the same
IEEE binary32 sequence as the C file's.

    quantize_block_rowwise            triton_functions.py:207-216, :221-233
    dequantize_block_rowwise          triton_functions.py:483-490, :492-500
    gemm_nt_partials                  triton_functions.py:115
    int8_matmul_block_dequantize      triton_functions.py:106-131, :142-168
    linear_forward / linear_backward  block_linear.py:71-80, :83-112
    linear_wint8_forward / _backward  block_linear.py:42-67 as intended (see the functions)

NaN inputs are outside this file's domain (``amax`` propagates them; the C checker ignores them).
"""
from __future__ import annotations

import torch


def ceil_div(n: int, d: int) -> int:
    return -(n // -d)


def _blocked(x: torch.Tensor, block: int) -> torch.Tensor:
    """[M,K] -> fp32 [M, nblk, block], zero padded (zeros never change an absmax, and quantize to 0)."""
    M, K = x.shape
    nblk = ceil_div(K, block)
    xf = x.float()
    if nblk * block != K:
        xf = torch.nn.functional.pad(xf, (0, nblk * block - K))
    return xf.reshape(M, nblk, block)


def quantize_block_rowwise(x: torch.Tensor, block: int):
    M, K = x.shape
    xb = _blocked(x, block)
    s = xb.abs().amax(dim=-1)                                   # :210-211  [M, nblk]
    safe = torch.where(s > 0, s, torch.ones_like(s))
    quot = xb / safe.unsqueeze(-1)                              # :212  x / max_val
    codes = torch.round(127.0 * quot)                           # :212  llrint(127. * ...), half to even
    codes = torch.where(s.unsqueeze(-1) > 0, codes, torch.zeros_like(codes))
    q = codes.to(torch.int8).reshape(M, -1)[:, :K].contiguous()
    return q, s.t().contiguous()                                # :214-216, :227  scales are [nblk, M]


def quantize_block_transposed(x: torch.Tensor, block: int):
    return quantize_block_rowwise(x.t().contiguous(), block)    # block_linear.py:93-94, :100-103


def dequantize_block_rowwise(q: torch.Tensor, s: torch.Tensor, block: int, out_dtype=torch.bfloat16):
    M, K = q.shape
    inv127 = torch.tensor(1.0 / 127.0, dtype=torch.float32)     # :499
    srow = s.float().t().repeat_interleave(block, dim=1)[:, :K]  # scale of element (m,k) = s[k//block, m]
    out = (srow * q.float()) * inv127                           # :487, left to right
    return out.to(out_dtype)


def gemm_nt_partials(a: torch.Tensor, w: torch.Tensor, block: int) -> torch.Tensor:
    """int32 [nblk, M, N].  fp32 bmm is exact here: every partial sum is an integer below 2**24
    (block * 127**2 = 2,064,512 for block 128), so neither FMA nor summation order can round."""
    assert block * 127 * 127 < (1 << 24)
    ab = _blocked(a, block).permute(1, 0, 2)                    # [nblk, M, B]
    wb = _blocked(w, block).permute(1, 2, 0)                    # [nblk, B, N]
    return torch.bmm(ab, wb).to(torch.int32)


def int8_matmul_block_dequantize(a, w, sa, sw, block: int, bias=None, out_dtype=torch.bfloat16):
    """a int8 [M,K]; w int8 [N,K] (the reference receives it as the view w.t()); sa [nblk,M]; sw [nblk,N]."""
    P = gemm_nt_partials(a, w, block).float()
    div = torch.tensor(1.0 / (127.0 * 127.0), dtype=torch.float32)   # :143
    acc = torch.zeros(P.shape[1:], dtype=torch.float32)
    sa, sw = sa.float(), sw.float()
    for j in range(P.shape[0]):                                 # :107, ascending
        acc = acc + sw[j][None, :] * (sa[j][:, None] * (P[j] * div))   # :120
    c = acc.to(out_dtype)                                       # :127
    if bias is not None:
        c = c + bias.to(out_dtype)                              # :129-131, add in the output dtype
    return c


def linear_forward(x, W, bias, block: int, out_dtype=torch.bfloat16):
    X = x.reshape(-1, x.shape[-1])                              # block_linear.py:72
    xq, sx = quantize_block_rowwise(X, block)                   # :78
    wq, sw = quantize_block_rowwise(W, block)                   # :79
    out = int8_matmul_block_dequantize(xq, wq, sx, sw, block, bias, out_dtype)   # :80
    return out.reshape(*x.shape[:-1], -1)


def linear_backward(G3, x, W, block: int, out_dtype=torch.bfloat16, has_bias=True):
    G = G3.reshape(-1, G3.shape[-1])                            # block_linear.py:84
    X = x.reshape(-1, x.shape[-1])
    gq, gs = quantize_block_rowwise(G, block)                   # :92
    wtq, wts = quantize_block_rowwise(W.t().contiguous(), block)            # :93-94
    grad_X = int8_matmul_block_dequantize(gq, wtq, gs, wts, block, None, out_dtype)   # :95
    xtq, xts = quantize_block_rowwise(X.t().contiguous(), block)            # :100, :102
    gtq, gts = quantize_block_rowwise(G.t().contiguous(), block)            # :101, :103
    grad_W = int8_matmul_block_dequantize(gtq, xtq, gts, xts, block, None, out_dtype)  # :104
    grad_b = G.sum(dim=0) if has_bias else None                 # :110
    return grad_X.reshape(*x.shape), grad_W, grad_b


def linear_wint8_forward(x, wq, sw, bias, block: int, out_dtype=torch.bfloat16):
    """The forward pass block_linear.py:43-47 set out to be: the weight arrives quantized along K (wq int8 [N,K],
    sw [nblk,N]), the activations are quantized here (the reference's line :47 forgets to, and so passes its
    arguments one position off), one GEMM."""
    X = x.reshape(-1, x.shape[-1])                              # :45
    xq, sx = quantize_block_rowwise(X, block)
    out = int8_matmul_block_dequantize(xq, wq, sx, sw, block, bias, out_dtype)   # :47
    return out.reshape(*x.shape[:-1], -1)


def linear_wint8_backward(G3, x, wtq, wts, block: int, out_dtype=torch.bfloat16, has_bias=True):
    """The backward pass block_linear.py:49-67 set out to be.  grad_X = G @ W contracts over the output features, so
    it needs the weight quantized along N: wtq int8 [K,N], wts [ceil(N/block), K] (the reference's line :57 multiplies
    with the K-blocked codes and their scales, which have the wrong shape for that).  grad_W and grad_bias as :58-65."""
    G = G3.reshape(-1, G3.shape[-1])                            # :51
    X = x.reshape(-1, x.shape[-1])
    gq, gs = quantize_block_rowwise(G, block)                   # :56
    grad_X = int8_matmul_block_dequantize(gq, wtq, gs, wts, block, None, out_dtype)     # :57, on the N-blocked copy
    xtq, xts = quantize_block_rowwise(X.t().contiguous(), block)            # :59, :61
    gtq, gts = quantize_block_rowwise(G.t().contiguous(), block)            # :60, :62
    grad_W = int8_matmul_block_dequantize(gtq, xtq, gts, xts, block, None, out_dtype)   # :63
    grad_b = G.sum(dim=0) if has_bias else None                 # :65
    return grad_X.reshape(*x.shape), grad_W, grad_b
