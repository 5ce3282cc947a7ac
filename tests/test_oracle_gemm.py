"""Pins the CPU checker's block GEMM (oracle/): exact golden vectors (Python ints + rounded Fractions),
int64 einsum brute force for the partials, special cases that reduce to a library matmul, fp64
evaluation of the closed form, and the forward/backward wiring against dense fp32 algebra."""
import numpy as np
import pytest
import torch

import oracle
from oracle import oracle_torch
from util import f32_from_bits, load_golden


def _rand_codes(g, *shape):
    return torch.randint(-127, 128, shape, generator=g, dtype=torch.int32).to(torch.int8)


@pytest.mark.parametrize("impl", ["c", "torch"])
def test_gemm_golden(impl):
    for case in load_golden("kat_gemm.json"):
        A = torch.tensor(case["A"], dtype=torch.int8)
        W = torch.tensor(case["W"], dtype=torch.int8)
        sa = torch.stack([f32_from_bits(r) for r in case["sa_bits"]])
        sw = torch.stack([f32_from_bits(r) for r in case["sw_bits"]])
        B = case["block"]
        if impl == "c":
            P = oracle.gemm_nt_partials(A, W, B)
            C = oracle.gemm_nt_dequant(A, W, sa, sw, B, None, torch.float32)
        else:
            P = oracle_torch.gemm_nt_partials(A, W, B)
            C = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw, B, None, torch.float32)
        assert P.tolist() == case["P"]
        # bit-exact: the expected values were rounded after every operation in the reference's order
        assert torch.equal(C.double(), torch.tensor(case["C_f32"], dtype=torch.float64))


@pytest.mark.parametrize("shape", [(253, 257, 234), (129, 266, 75), (389, 138, 45), (16, 8, 512)])
@pytest.mark.parametrize("block", [32, 64, 128])
def test_partials_bruteforce_int64(shape, block):
    M, N, K = shape      # odd shapes listed (commented out) at triton_functions.py:583-588
    g = torch.Generator().manual_seed(M * 7 + block)
    A, W = _rand_codes(g, M, K), _rand_codes(g, N, K)
    nblk = -(-K // block)
    Ap = np.zeros((M, nblk * block), np.int64); Ap[:, :K] = A.numpy()
    Wp = np.zeros((N, nblk * block), np.int64); Wp[:, :K] = W.numpy()
    ref = np.einsum("mjk,njk->jmn", Ap.reshape(M, nblk, block), Wp.reshape(N, nblk, block))
    assert np.abs(ref).max() <= block * 127 * 127
    for P in (oracle.gemm_nt_partials(A, W, block), oracle_torch.gemm_nt_partials(A, W, block)):
        assert P.dtype == torch.int32 and np.array_equal(P.numpy().astype(np.int64), ref)
    # saturating inputs reach the bound exactly
    A1 = torch.full((2, block), 127, dtype=torch.int8); W1 = torch.full((3, block), -127, dtype=torch.int8)
    assert (oracle.gemm_nt_partials(A1, W1, block) == -block * 127 * 127).all()


def test_special_cases_reduce_to_plain_matmul():
    g = torch.Generator().manual_seed(2)
    M, N, K, B = 33, 29, 256, 64
    A, W = _rand_codes(g, M, K), _rand_codes(g, N, K)
    nblk = K // B
    exact_int = (A.double() @ W.double().t())
    # scales that are powers of two: only the P*divfactor rounding remains -> 2**-23 relative per term
    sa = torch.full((nblk, M), 4.0); sw = torch.full((nblk, N), 0.5)
    C = oracle.gemm_nt_dequant(A, W, sa, sw, B, None, torch.float32).double()
    assert torch.allclose(C, exact_int * 2.0 / (127.0 * 127.0), rtol=0, atol=2.0 * nblk * B * 127 * 127 / 127**2 * 2**-22)
    # one block: a row- and column-scaled matmul
    sa1 = torch.rand(1, M, generator=g) + 0.5; sw1 = torch.rand(1, N, generator=g) * 0.02
    C1 = oracle.gemm_nt_dequant(A[:, :B].contiguous(), W[:, :B].contiguous(), sa1, sw1, B, None, torch.float32).double()
    ref1 = (A[:, :B].double() @ W[:, :B].double().t()) * sa1.double().t() * sw1.double() / (127.0 * 127.0)
    assert torch.allclose(C1, ref1, rtol=1e-6, atol=0)
    # swapping the scale vectors of two blocks must change the result (guards a dropped/shared scale index)
    sa2 = torch.rand(nblk, M, generator=g) + 0.5; sw2 = torch.rand(nblk, N, generator=g) + 0.5
    Ca = oracle.gemm_nt_dequant(A, W, sa2, sw2, B, None, torch.float32)
    Cb = oracle.gemm_nt_dequant(A, W, sa2.flip(0).contiguous(), sw2, B, None, torch.float32)
    assert not torch.equal(Ca, Cb)


@pytest.mark.parametrize("out_dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2.0**-8), (torch.float16, 2.0**-10)])
def test_closed_form_fp64_and_bias(out_dtype, tol):
    g = torch.Generator().manual_seed(3)
    M, N, K, B = 41, 50, 200, 64     # ragged last block
    A, W = _rand_codes(g, M, K), _rand_codes(g, N, K)
    nblk = -(-K // B)
    sa = torch.rand(nblk, M, generator=g) * 4; sw = torch.rand(nblk, N, generator=g) * 0.1
    bias = torch.randn(N, generator=g)
    P = oracle.gemm_nt_partials(A, W, B).double()
    ref = (P * sa.double()[:, :, None] * sw.double()[:, None, :]).sum(0) / (127.0 * 127.0)
    mag = (P.abs() * sa.double()[:, :, None] * sw.double()[:, None, :]).sum(0) / (127.0 * 127.0)
    for impl in ("c", "torch"):
        if impl == "c":
            C = oracle.gemm_nt_dequant(A, W, sa, sw, B, None, out_dtype)
            Cb = oracle.gemm_nt_dequant(A, W, sa, sw, B, bias, out_dtype)
        else:
            C = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw, B, None, out_dtype)
            Cb = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw, B, bias, out_dtype)
        assert C.dtype == out_dtype
        assert ((C.double() - ref).abs() <= tol * mag + 1e-30).all()
        # bias is added after the cast, in the output dtype (triton_functions.py:127-131)
        expect = (C + bias.to(out_dtype))
        assert torch.equal(Cb, expect)


def test_c_and_torch_gemm_bit_identical():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(64, 384, generator=g); w = torch.randn(96, 384, generator=g) * 0.02
    for B in (32, 64, 128):
        xq, sx = oracle.quantize_block_rowwise(x, B); wq, sw = oracle.quantize_block_rowwise(w, B)
        for od in (torch.float32, torch.bfloat16):
            a = oracle.gemm_nt_dequant(xq, wq, sx, sw, B, None, od)
            b = oracle_torch.int8_matmul_block_dequantize(xq, wq, sx, sw, B, None, od)
            assert torch.equal(a, b)


def test_config1_forward_close_to_dense():
    """X fp32 [256,1024] ~N(0,1), W fp32 [1024,1024] ~N(0,0.02), block 64, fp32 out, vs the fp32 matmul."""
    g = torch.Generator().manual_seed(0)
    X = torch.randn(256, 1024, generator=g); W = torch.randn(1024, 1024, generator=g) * 0.02
    out = oracle_torch.linear_forward(X, W, None, 64, torch.float32)
    dense = X @ W.t()
    rel = (out - dense).norm() / dense.norm()
    assert out.shape == (256, 1024) and 1e-3 < rel < 3e-2, rel
    xq, sx = oracle.quantize_block_rowwise(X, 64); wq, sw = oracle.quantize_block_rowwise(W, 64)
    assert torch.equal(out, oracle.gemm_nt_dequant(xq, wq, sx, sw, 64, None, torch.float32, threads=True))


def test_backward_wiring_against_dense_algebra():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(4, 48, 128, generator=g); W = torch.randn(96, 128, generator=g) * 0.05
    G = torch.randn(4, 48, 96, generator=g)
    gX, gW, gb = oracle_torch.linear_backward(G, x, W, 64, torch.float32)
    G2, X2 = G.reshape(-1, 96), x.reshape(-1, 128)
    assert gX.shape == x.shape and gW.shape == W.shape
    assert (gX.reshape(-1, 128) - G2 @ W).norm() / (G2 @ W).norm() < 3e-2
    assert (gW - G2.t() @ X2).norm() / (G2.t() @ X2).norm() < 3e-2
    assert torch.equal(gb, G2.sum(0))


def _lossless(g, rows, cols, block, scale):
    """integers in [-127,127] times a power of two, +-127 somewhere in every block of every row: block quantization
    is lossless on it (scale 127 * 2^e, codes = the integers), so the quantized products ARE the dense products"""
    t = torch.randint(-127, 128, (rows, cols), generator=g, dtype=torch.int32).float()
    t[:, ::block] = 127.0
    t[::2, ::block] = -127.0
    return t * scale


def test_weight_only_training_functions_against_dense_algebra():
    """linear_wint8_forward / _backward (what block_linear.py:42-67 set out to be), pinned three ways: with the two
    quantized copies made from W they are linear_forward / linear_backward bit for bit; on data that block
    quantization represents exactly they equal the DENSE products G @ W, G.T @ X, X @ W.T to fp32 rounding (a
    transposed operand, scales of the other copy or blocks along the wrong dimension miss by O(1)); and grad_X does
    change when it is given the K-blocked copy's scales instead (the reference's mistake at :57)."""
    g = torch.Generator().manual_seed(11)
    B, M, K, N = 32, 96, 128, 64
    x = torch.randn(2, M // 2, K, generator=g); W = torch.randn(N, K, generator=g) * 0.05
    G = torch.randn(2, M // 2, N, generator=g); bias = torch.randn(N, generator=g)
    wq, sw = oracle_torch.quantize_block_rowwise(W, B)
    wtq, wts = oracle_torch.quantize_block_rowwise(W.t().contiguous(), B)
    for od in (torch.float32, torch.bfloat16):
        assert torch.equal(oracle_torch.linear_wint8_forward(x, wq, sw, bias, B, od), oracle_torch.linear_forward(x, W, bias, B, od))
        a = oracle_torch.linear_wint8_backward(G, x, wtq, wts, B, od)
        b = oracle_torch.linear_backward(G, x, W, B, od)
        assert all(torch.equal(u, v) for u, v in zip(a, b))
    # lossless data, N != K and M != N so that no transposition goes unnoticed
    X = _lossless(g, M, K, B, 0.25); Wl = _lossless(g, N, K, B, 2.0 ** -9)
    X[:, ::B] = 127 * 0.25; X[::3, ::B] = -127 * 0.25
    Gl = _lossless(g, M, N, B, 0.5)
    # ... also along the other direction: every column block of B rows holds a +-127 too
    for t, s in ((X, 0.25), (Wl, 2.0 ** -9), (Gl, 0.5)):
        t[::B, :] = 127 * s
    wq, sw = oracle_torch.quantize_block_rowwise(Wl, B)
    wtq, wts = oracle_torch.quantize_block_rowwise(Wl.t().contiguous(), B)
    assert torch.equal(wq.float() * (2.0 ** -9), Wl) and (sw == 127 * 2.0 ** -9).all() and torch.equal(wtq, wq.t())
    y = oracle_torch.linear_wint8_forward(X, wq, sw, None, B, torch.float32)
    gX, gW, gb = oracle_torch.linear_wint8_backward(Gl, X, wtq, wts, B, torch.float32)
    for got, dense in ((y, X.double() @ Wl.double().t()), (gX, Gl.double() @ Wl.double()), (gW, Gl.double().t() @ X.double())):
        assert got.shape == dense.shape
        assert ((got.double() - dense).abs() <= 2e-6 * dense.abs() + 1e-6 * dense.abs().max()).all()
    assert torch.equal(gb, Gl.sum(0))
    # the reference's line :57 (K-blocked codes and scales in the grad-input GEMM) is a different function
    W2 = torch.randn(K, K, generator=g) * 0.05                     # square, so that the shapes allow the mistake
    G2 = torch.randn(M, K, generator=g)
    wq2, sw2 = oracle_torch.quantize_block_rowwise(W2, B)
    wtq2, wts2 = oracle_torch.quantize_block_rowwise(W2.t().contiguous(), B)
    right, _, _ = oracle_torch.linear_wint8_backward(G2, X, wtq2, wts2, B, torch.float32)
    wrong, _, _ = oracle_torch.linear_wint8_backward(G2, X, wq2, sw2, B, torch.float32)
    dense = G2 @ W2
    assert (right - dense).norm() / dense.norm() < 3e-2 < (wrong - dense).norm() / dense.norm()
