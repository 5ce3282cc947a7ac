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
