"""Pins the CPU checker's quantizer and dequantizer (oracle/) without running the reference:
golden vectors from exact rational arithmetic, brute force on random small inputs, closed-form
invariants, and agreement of the two independently written restatements (C and PyTorch)."""
from fractions import Fraction

import numpy as np
import pytest
import torch

import exact
import oracle
from oracle import oracle_torch
from util import DTYPES, bits_to_tensor, f32_from_bits, load_golden, outlier_tensor

IMPLS = {"c": oracle.quantize_block_rowwise, "torch": oracle_torch.quantize_block_rowwise}


@pytest.mark.parametrize("impl", ["c", "torch"])
def test_quantize_golden(impl):
    for case in load_golden("kat_quantize.json"):
        x = bits_to_tensor(case["x_bits"], case["dtype"]).reshape(1, -1)
        q, s = IMPLS[impl](x, case["block"])
        assert q.shape == x.shape and s.shape == (len(case["scale_bits"]), 1), case["name"]
        assert q.view(-1).tolist() == case["codes"], case["name"]
        assert torch.equal(s.view(-1), f32_from_bits(case["scale_bits"])), case["name"]


def test_hand_vector():
    # s = 2 -> 127*(1/2) = 63.5 -> 64 (half to even), 127*(-2/2) = -127, 127*(0.5/2) = 31.75 -> 32
    x = torch.tensor([[1.0, -2.0, 0.5, 0.0]])
    q, s = oracle.quantize_block_rowwise(x, 4)
    assert q.tolist() == [[64, -127, 32, 0]] and s.tolist() == [[2.0]]
    # 2.5 -> 2 and 3.5 -> 4: proves ties go to even, not away from zero
    x = torch.tensor([[127.0, 2.5, 3.5, -2.5]])
    q, _ = oracle.quantize_block_rowwise(x, 4)
    assert q.tolist() == [[127, 2, 4, -2]]


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
def test_quantize_bruteforce_exact(dtype):
    """random small inputs against Fraction arithmetic, element by element"""
    g = torch.Generator().manual_seed(11)
    for block, K in [(16, 48), (32, 70), (128, 128)]:
        x = (torch.randn(3, K, generator=g) * torch.rand(3, 1, generator=g) * 8).to(DTYPES[dtype])
        q, s = oracle.quantize_block_rowwise(x, block)
        xf = x.float()
        for m in range(3):
            for j, k0 in enumerate(range(0, K, block)):
                xs = [exact.float_to_fraction(v) for v in xf[m, k0:k0 + block].tolist()]
                es, ec = exact.quantize_block_exact(xs)
                assert exact.float_to_fraction(s[j, m].item()) == es
                assert q[m, k0:k0 + block].tolist() == ec


@pytest.mark.parametrize("impl", ["c", "torch"])
def test_quantize_invariants(impl):
    fn = IMPLS[impl]
    g = torch.Generator().manual_seed(5)
    M, K, B = 37, 300, 64
    x = torch.randn(M, K, generator=g)
    q, s = fn(x, B)
    nblk = -(-K // B)
    assert s.shape == (nblk, M) and s.dtype == torch.float32 and q.dtype == torch.int8
    pad = torch.nn.functional.pad(x, (0, nblk * B - K)).reshape(M, nblk, B)
    # scale is bit-equal to the largest magnitude of its block, stored block-major / row-minor
    assert torch.equal(s, pad.abs().amax(-1).t())
    qp = torch.nn.functional.pad(q, (0, nblk * B - K)).reshape(M, nblk, B).int()
    # the absmax element maps to +-127, signs are preserved, |code| <= 127
    idx = pad.abs().argmax(-1, keepdim=True)
    assert torch.equal(qp.gather(-1, idx).abs(), torch.full_like(idx, 127, dtype=torch.int32))
    assert (qp.abs() <= 127).all()
    assert ((qp.sign() == pad.sign().int()) | (qp == 0)).all()
    # monotone inside a block
    order = pad.argsort(-1)
    assert (qp.gather(-1, order).diff(dim=-1) >= 0).all()
    # scaling by a power of two: same codes, scales scaled
    q2, s2 = fn(x * 8.0, B)
    assert torch.equal(q2, q) and torch.equal(s2, s * 8.0)
    # rows and blocks are independent units
    perm = torch.randperm(M, generator=g)
    qpm, spm = fn(x[perm], B)
    assert torch.equal(qpm, q[perm]) and torch.equal(spm, s[:, perm])
    qb, sb = fn(x[:, B:2 * B].contiguous(), B)
    assert torch.equal(qb, q[:, B:2 * B]) and torch.equal(sb, s[1:2])
    # error bound of the round trip: |x - s*code/127| <= s/254 (+ a few ulp)
    deq = qp.float() * s.t().unsqueeze(-1) / 127.0
    assert ((deq - pad).abs() <= s.t().unsqueeze(-1) * (1 / 254 + 1e-6)).all()


def test_c_and_torch_restatements_agree():
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        x = outlier_tensor(64, 1000, dtype, seed=3)
        for B in (32, 64, 128):
            qc, sc = oracle.quantize_block_rowwise(x, B)
            qt, st = oracle_torch.quantize_block_rowwise(x, B)
            assert torch.equal(qc, qt) and torch.equal(sc, st)
            for od in (torch.float32, torch.bfloat16, torch.float16):
                dc = oracle.dequantize_block_rowwise(qc, sc, B, od)
                dt = oracle_torch.dequantize_block_rowwise(qc, sc, B, od)
                assert torch.equal(dc, dt)
            qT, sT = oracle.quantize_block_transposed(x, B)
            qT2, sT2 = oracle_torch.quantize_block_transposed(x, B)
            assert torch.equal(qT, qT2) and torch.equal(sT, sT2)
            # definition of the transposed quantizer (block_linear.py:93-94)
            qT3, sT3 = oracle.quantize_block_rowwise(x.t().contiguous(), B)
            assert torch.equal(qT, qT3) and torch.equal(sT, sT3)


def test_zero_and_nan_blocks():
    x = torch.zeros(2, 64)
    x[1, 40] = -3.0
    q, s = oracle.quantize_block_rowwise(x, 32)
    assert s.tolist() == [[0.0, 0.0], [0.0, 3.0]]
    assert q[0].abs().sum() == 0 and q[1, 40] == -127 and q[1].abs().sum() == 127
    x[0, 3] = float("nan")
    x[0, 5] = 2.0
    q, s = oracle.quantize_block_rowwise(x, 32)
    assert s[0, 0] == 2.0 and q[0, 3] == 0 and q[0, 5] == 127


@pytest.mark.parametrize("impl", ["c", "torch"])
def test_dequantize_golden(impl):
    fn = oracle.dequantize_block_rowwise if impl == "c" else oracle_torch.dequantize_block_rowwise
    for case in load_golden("kat_dequantize.json"):
        codes = torch.tensor(case["codes"], dtype=torch.int8).reshape(1, -1)
        s = f32_from_bits([case["scale_bits"]]).reshape(1, 1)
        B = codes.shape[1]
        out = fn(codes, s, B, torch.float32).view(-1).double()
        assert torch.equal(out, torch.tensor(case["out_f32"], dtype=torch.float64))
        out = fn(codes, s, B, torch.bfloat16).view(-1).double()
        assert torch.equal(out, torch.tensor(case["out_bf16"], dtype=torch.float64))
        exp16 = case["out_f16"]
        out = fn(codes, s, B, torch.float16).view(-1).double().tolist()
        for o, e in zip(out, exp16):
            assert (e is None and np.isinf(o)) or o == e


def test_element_conversions_match_torch():
    lib = oracle._lib()
    allh = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        vals = allh.view(dt).float()
        to_f32 = getattr(lib, f"bi8o_{name}_to_f32")
        from_f32 = getattr(lib, f"bi8o_f32_to_{name}")
        for u in list(range(0, 65536, 97)) + [0, 1, 0x3FF, 0x400, 0x7BFF, 0x7C00, 0x8000, 0xFBFF, 0x7F7F, 0x7F80]:
            v = vals[u].item()
            got = to_f32(u)
            assert (np.isnan(v) and np.isnan(got)) or got == v
        g = torch.Generator().manual_seed(9)
        f = torch.randn(4000, generator=g) * torch.logspace(-30, 6, 4000)
        f = torch.cat([f, torch.tensor([65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 3.0e-8, 6.1e-5])])
        ref = f.to(dt).view(torch.int16).int() & 0xFFFF
        for x, r in zip(f.tolist(), ref.tolist()):
            assert from_f32(x) == r, (name, x)
