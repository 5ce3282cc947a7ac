"""Seeded random shapes, strides and block sizes through every operator, against the CPU checker: the cases the
hand-picked shape lists do not name (every kernel selection boundary is crossed by some of them)."""
import os
import random

import pytest
import torch

import oracle
from oracle import oracle_torch
from util import DTYPES, outlier_tensor

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"f32": 1e-3, "bf16": 1e-2, "f16": 1e-2}
N_CASES = int(os.environ.get("BI8_RANDOM_CASES", "40"))      # more cases for a longer soak


@pytest.fixture(scope="module")
def ops():
    import blockwise_int8_linear_amd as pkg
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return pkg


def _pick_dim(rng, lo, hi):
    """a dimension near a power of two / tile edge half of the time, anything in range otherwise"""
    if rng.random() < 0.5:
        base = rng.choice([16, 32, 64, 128, 256, 512, 1024])
        return max(lo, min(hi, base + rng.choice([-1, 0, 0, 1, 3, 8, 16])))
    return rng.randint(lo, hi)


@pytest.mark.parametrize("seed", range(N_CASES))
def test_gemm_random(ops, seed):
    rng = random.Random(1000 + seed)
    block = rng.choice([32, 64, 128, 128, 16, 256])
    out = rng.choice(["f32", "bf16", "f16"])
    M = rng.choice([rng.randint(1, 40), _pick_dim(rng, 1, 700)])
    N = _pick_dim(rng, 1, 700)
    K = rng.choice([128 * rng.randint(1, 12), 128 * rng.randint(16, 40), _pick_dim(rng, 1, 1500)])     # long K: split over workgroups
    pad_a, pad_w = rng.choice([0, 0, 16, 5]), rng.choice([0, 0, 32, 3])
    g = torch.Generator().manual_seed(seed)
    A = torch.randint(-127, 128, (M, K + pad_a), generator=g, dtype=torch.int32).to(torch.int8)
    W = torch.randint(-127, 128, (N, K + pad_w), generator=g, dtype=torch.int32).to(torch.int8)
    nblk = -(-K // block)
    sa = torch.rand(nblk, M, generator=g) * 3 + 0.01
    sw = torch.rand(nblk, N, generator=g) * 0.1 + 1e-4
    bias = torch.randn(N, generator=g) if rng.random() < 0.5 else None
    Ac, Wc = A[:, :K].contiguous(), W[:, :K].contiguous()
    P = oracle_torch.gemm_nt_partials(Ac, Wc, block)
    ref = oracle_torch.int8_matmul_block_dequantize(Ac, Wc, sa, sw, block, None, DTYPES[out])
    mag = torch.zeros(M, N, dtype=torch.float64)
    for j in range(nblk):
        mag += P[j].abs().double() * sa[j].double()[:, None] * sw[j].double()[None, :]
    mag /= 127.0 * 127.0
    cfg = ops.block_linear_config
    old = (cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE)
    cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = block, DTYPES[out]
    try:
        Ad, Wd = A.to(DEV)[:, :K], W.to(DEV)[:, :K]                  # views with leading dimension K + pad
        C = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sa.to(DEV), sw.to(DEV))
        Pd = ops.int8_matmul_block_partials(Ad, Wd.t())
        if bias is not None:
            Cb = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sa.to(DEV), sw.to(DEV), bias.to(DEV))
            assert torch.equal(Cb, C + bias.to(DEV).to(DTYPES[out]))
    finally:
        cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = old
    assert torch.equal(Pd.cpu(), P), f"partials differ (M={M} N={N} K={K} block={block})"
    err = (C.cpu().double() - ref.double()).abs()
    bound = TOL[out] * ref.double().abs() + 4e-6 * mag + 1e-30
    assert (err <= bound).all(), f"M={M} N={N} K={K} block={block} out={out}: max excess {(err - bound).max().item():.3e}"


@pytest.mark.parametrize("seed", range(N_CASES))
def test_quantize_dequantize_random(ops, seed):
    rng = random.Random(2000 + seed)
    block = rng.choice([32, 64, 128, 128, 16, 256, 24])
    dtype = rng.choice(["f32", "bf16", "f16"])
    M, K = _pick_dim(rng, 1, 400), rng.choice([128 * rng.randint(1, 20), _pick_dim(rng, 1, 3000)])
    pad = rng.choice([0, 0, 8, 3])
    x_cpu = outlier_tensor(M, K + pad, DTYPES[dtype], seed=seed)
    xc = x_cpu[:, :K].contiguous()
    xd = x_cpu.to(DEV)[:, :K]
    q, s = ops.quantize_block_rowwise(xd, block)
    qo, so = oracle.quantize_block_rowwise(xc, block, threads=True)
    assert torch.equal(s.cpu().view(torch.int32), so.view(torch.int32)) and torch.equal(q.cpu(), qo), (M, K, pad, block, dtype)
    qt, st = ops.quantize_block_transposed(xd, block)
    qto, sto = oracle.quantize_block_transposed(xc, block, threads=True)
    assert torch.equal(st.cpu().view(torch.int32), sto.view(torch.int32)) and torch.equal(qt.cpu(), qto), (M, K, pad, block, dtype)
    q2, s2, qt2, st2 = ops.quantize_block_dual(xd, block)               # both directions from one read: the same bits
    assert torch.equal(q2, q) and torch.equal(qt2, qt), (M, K, pad, block, dtype)
    assert torch.equal(s2.view(torch.int32), s.view(torch.int32)) and torch.equal(st2.view(torch.int32), st.view(torch.int32))
    cfg = ops.block_linear_config
    old = cfg.INPUT_OUTPUT_TORCH_TYPE
    cfg.INPUT_OUTPUT_TORCH_TYPE = DTYPES[dtype]
    try:
        d = ops.dequantize_block_rowwise(q, s, block)
    finally:
        cfg.INPUT_OUTPUT_TORCH_TYPE = old
    do = oracle.dequantize_block_rowwise(qo, so, block, DTYPES[dtype])
    view = torch.int32 if dtype == "f32" else torch.int16
    assert torch.equal(d.cpu().view(view), do.view(view)), (M, K, pad, block, dtype)


@pytest.mark.parametrize("seed", range(6))
def test_gemm_random_large(ops, seed):
    """shapes of more than 128 output tiles of 256x256 (the large-problem kernel for blocks 64 and 128), ragged edges"""
    rng = random.Random(3000 + seed)
    block = rng.choice([64, 128])
    out = rng.choice(["f32", "bf16", "f16"])
    M, N = rng.randint(3300, 4400), rng.randint(3300, 4400)
    K = 128 * rng.randint(1, 5)
    g = torch.Generator().manual_seed(seed)
    A = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    W = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    nblk = K // block
    sa = torch.rand(nblk, M, generator=g) * 3 + 0.01
    sw = torch.rand(nblk, N, generator=g) * 0.1 + 1e-4
    bias = torch.randn(N, generator=g)
    P = oracle_torch.gemm_nt_partials(A, W, block)
    ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw, block, None, DTYPES[out])
    mag = torch.zeros(M, N, dtype=torch.float64)
    for j in range(nblk):
        mag += P[j].abs().double() * sa[j].double()[:, None] * sw[j].double()[None, :]
    mag /= 127.0 * 127.0
    cfg = ops.block_linear_config
    old = (cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE)
    cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = block, DTYPES[out]
    try:
        Ad, Wd = A.to(DEV), W.to(DEV)
        C = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sa.to(DEV), sw.to(DEV))
        Cb = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sa.to(DEV), sw.to(DEV), bias.to(DEV))
    finally:
        cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = old
    assert torch.equal(Cb, C + bias.to(DEV).to(DTYPES[out]))
    err = (C.cpu().double() - ref.double()).abs()
    bound = TOL[out] * ref.double().abs() + 4e-6 * mag + 1e-30
    assert (err <= bound).all(), f"M={M} N={N} K={K} block={block} out={out}: max excess {(err - bound).max().item():.3e}"


@pytest.mark.parametrize("seed", range(N_CASES // 2))
def test_few_rows_random(ops, seed):
    """the one-kernel eval path (quantize + GEMM) against the two launchers, 1..4 rows (the one-kernel form covers one and two), random K, N, block and type"""
    rng = random.Random(4000 + seed)
    block = rng.choice([64, 128])
    dtype = rng.choice(["f32", "bf16", "f16"])
    M, K, N = rng.randint(1, 4), 128 * rng.randint(1, 48), _pick_dim(rng, 1, 3000)
    cfg = ops.block_linear_config
    old = (cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE)
    cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = block, DTYPES[dtype]
    try:
        g = torch.Generator().manual_seed(seed)
        w = (torch.randn(N, K, generator=g) * 0.02).to(DTYPES[dtype]).to(DEV)
        x = outlier_tensor(M, K, DTYPES[dtype], seed=seed).to(DEV)
        bias = torch.randn(N, generator=g).to(DTYPES[dtype]).to(DEV) if rng.random() < 0.5 else None
        Wq, Ws = ops.quantize_block_rowwise(w)
        xq, xs = ops.quantize_block_rowwise(x)
        two = ops.int8_matmul_block64_rowwise_dequantize(xq, Wq.t(), xs, Ws, bias)
        one = ops.linear_few_rows(x, Wq, Ws, bias)
    finally:
        cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = old
    if one is None:
        from blockwise_int8_linear_amd.ops import _few_rows_lds
        assert M > 2 or _few_rows_lds(M, K, block, x.element_size()) > 65536, (M, K, N, block, dtype)
    else:
        view = torch.int32 if dtype == "f32" else torch.int16
        assert torch.equal(one.view(view), two.view(view)), (M, K, N, block, dtype)
