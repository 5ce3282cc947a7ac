"""bi8_gemm_nt_dequant_ws: the contraction split over the workgroups (equal pieces of every tile, or equal runs of
(tile, stage of K) pairs) through a caller-provided workspace.
Against the CPU checker to the GEMM tolerance, and against the one-pass entry point (same numbers up to the fp32
rounding of a different summation order)."""
import ctypes

import pytest
import torch

from oracle import oracle_torch
from util import DTYPES

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"f32": 1e-3, "bf16": 1e-2, "f16": 1e-2}


@pytest.fixture(scope="module")
def lib():
    from blockwise_int8_linear_amd import _lib
    return _lib.load()


def _problem(M, N, K, block, seed):
    g = torch.Generator().manual_seed(seed)
    A = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    W = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    sa = torch.rand(K // block, M, generator=g) * 3 + 0.01
    sw = torch.rand(K // block, N, generator=g) * 0.1 + 1e-4
    bias = torch.randn(N, generator=g)
    return A, W, sa, sw, bias


def _run(lib, A, W, sa, sw, bias, block, out, ws_bytes):
    M, K = A.shape
    N = W.shape[0]
    dt = {"f32": 0, "bf16": 1, "f16": 2}[out]
    C = torch.empty(M, N, device=DEV, dtype=DTYPES[out])
    ws = torch.empty(max(ws_bytes, 1), device=DEV, dtype=torch.uint8)
    st = torch.cuda.current_stream().cuda_stream
    b = bias.to(DEV) if bias is not None else None
    rc = lib.bi8_gemm_nt_dequant_ws(A.data_ptr(), W.data_ptr(), sa.data_ptr(), sw.data_ptr(), b.data_ptr() if b is not None else None, 0,
                                    C.data_ptr(), dt, M, N, K, K, K, N, block, ws.data_ptr() if ws_bytes else None, ws_bytes, st)
    assert rc == 0
    torch.cuda.synchronize()
    return C


@pytest.mark.parametrize("out", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("M,N,K,block", [(128, 512, 8192, 128), (100, 300, 5120, 64), (80, 700, 5120, 128), (200, 130, 4096, 32),
                                         (384, 256, 8192, 64), (128, 4096, 8192, 128),
                                         # (more than 64 rows split from K = 4096 on; below that they run narrow tiles, one pass)
                                         # up to 64 rows split where the one-pass kernel would stream too much of A or take
                                         # more than one round of workgroups
                                         (33, 128, 10240, 128), (48, 700, 7168, 128), (60, 4800, 4224, 128), (40, 700, 2560, 32),
                                         # 35 stages of K in pieces of 9, 9, 9, 8
                                         (200, 300, 4480, 64),
                                         # 17 to 64 rows and a long K: narrow tiles of 32 x 64 or 64 x 64 on pieces of K
                                         (24, 2000, 8320, 64), (32, 5000, 8192, 128), (20, 8192, 10240, 128), (64, 2000, 5120, 128),
                                         (50, 1000, 12288, 64)])
def test_split_matches_checker_and_one_pass(lib, M, N, K, block, out):
    A, W, sa, sw, bias = _problem(M, N, K, block, seed=M + N + K)
    want = lib.bi8_gemm_workspace_bytes(M, N, K, block)
    assert 0 < want <= lib.bi8_static_scratch_bytes() and want % (32 * 64 * 4) == 0      # fp32 slabs of one tile (32x64 ... 128x128) each
    Ad, Wd, sad, swd = A.to(DEV), W.to(DEV), sa.to(DEV), sw.to(DEV)
    split = _run(lib, Ad, Wd, sad, swd, None, block, out, want)
    one = _run(lib, Ad, Wd, sad, swd, None, block, out, 0)
    ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw, block, None, DTYPES[out])
    P = oracle_torch.gemm_nt_partials(A, W, block)
    mag = torch.zeros(M, N, dtype=torch.float64)
    for j in range(K // block):
        mag += P[j].abs().double() * sa[j].double()[:, None] * sw[j].double()[None, :]
    mag /= 127.0 * 127.0
    bound = TOL[out] * ref.double().abs() + 4e-6 * mag + 1e-30
    assert ((split.cpu().double() - ref.double()).abs() <= bound).all()
    assert ((split.double() - one.double()).abs().cpu() <= 2 * bound).all()        # each is within the bound of the checker
    # the bias is added after the cast, in the output type (triton_functions.py:127-131): exactly this identity
    with_bias = _run(lib, Ad, Wd, sad, swd, bias, block, out, want)
    assert torch.equal(with_bias, split + bias.to(DEV).to(DTYPES[out]))


@pytest.mark.parametrize("M,N,K,block,kernel", [
    # 129 to 255 tiles of 128x128 and a long K: 256 workgroups, each a run of (tile, stage) pairs that ends inside a tile
    (2048, 1408, 16384, 64, "gemm_tile_128x128_splitk"), (1900, 1400, 16384, 128, "gemm_tile_128x128_splitk"),
    (3000, 700, 8192, 32, "gemm_tile_128x128_splitk"),
    # few tiles of 256x128 and a long K: three pieces per tile on the 256x256 kernel's loop (72 tiles x 3 pieces of 22,
    # 22 and 20 stages; 77 x 3 pieces of 44, 44, 40)
    (3072, 768, 8192, 64, "gemm_wide_256x128_splitk"), (1700, 1300, 16384, 128, "gemm_wide_256x128_splitk"),
    # 100 to 128 tiles of 128x128 and K from 8192 on: two pieces per tile on gemm_panel's square form (18 x 6 tiles, ragged edges)
    (2200, 700, 8192, 128, "gemm_panel_splitk")])
def test_more_tiles_than_half_the_chip(lib, M, N, K, block, kernel):
    """The splits of problems that fill more than half of the chip with tiles.  The checker on sampled rows (every row of
    tiles is hit), the one-pass kernel on everything."""
    A, W, sa, sw, bias = _problem(M, N, K, block, seed=M + N + K)
    want = lib.bi8_gemm_workspace_bytes(M, N, K, block)
    assert lib.bi8_gemm_kernel_name(M, N, K, K, K, block, want).decode() == kernel
    if "panel" in kernel:
        assert want == -(-M // 128) * -(-N // 128) * 2 * 128 * 128 * 4
    elif "wide" in kernel:
        tiles = -(-M // 256) * -(-N // 128)
        assert want % (256 * 128 * 4) == 0 and 160 <= want // (256 * 128 * 4) <= 256 and (want // (256 * 128 * 4)) % tiles == 0
    else:
        tiles = -(-M // 128) * -(-N // 128)
        assert want % (128 * 128 * 4) == 0 and 240 + tiles <= want // (128 * 128 * 4) <= 256 + tiles - 1
    Ad, Wd, sad, swd = A.to(DEV), W.to(DEV), sa.to(DEV), sw.to(DEV)
    split = _run(lib, Ad, Wd, sad, swd, bias, block, "f32", want)
    one = _run(lib, Ad, Wd, sad, swd, bias, block, "f32", 0)
    rows = torch.unique(torch.cat([torch.arange(0, M, 61), torch.tensor([M - 1])]))
    ref = oracle_torch.int8_matmul_block_dequantize(A[rows], W, sa[:, rows].contiguous(), sw, block, bias, torch.float32)
    P = oracle_torch.gemm_nt_partials(A[rows], W, block)
    mag = torch.zeros(len(rows), N, dtype=torch.float64)
    for j in range(K // block):
        mag += P[j].abs().double() * sa[j, rows].double()[:, None] * sw[j].double()[None, :]
    mag /= 127.0 * 127.0
    bound = 1e-3 * ref.double().abs() + 4e-6 * mag + 1e-30
    assert ((split[rows.to(DEV)].cpu().double() - ref.double()).abs() <= bound).all()
    # everything else against the one-pass result: both are sums of the same fp32 terms in different orders
    scale = one.abs().max().item()
    assert (split - one).abs().max().item() <= 2e-5 * scale
    again = _run(lib, Ad, Wd, sad, swd, bias, block, "f32", want)
    assert torch.equal(split, again)                                         # fixed order of the sum: deterministic


def test_workspace_too_small_or_absent_is_the_one_pass_result(lib):
    M, N, K, block = 128, 512, 8192, 128
    A, W, sa, sw, bias = _problem(M, N, K, block, seed=3)
    Ad, Wd, sad, swd = A.to(DEV), W.to(DEV), sa.to(DEV), sw.to(DEV)
    want = lib.bi8_gemm_workspace_bytes(M, N, K, block)
    one = _run(lib, Ad, Wd, sad, swd, bias, block, "bf16", 0)
    small = _run(lib, Ad, Wd, sad, swd, bias, block, "bf16", want - 4)
    assert torch.equal(one, small)
    C = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    rc = lib.bi8_gemm_nt_dequant(Ad.data_ptr(), Wd.data_ptr(), sad.data_ptr(), swd.data_ptr(), bias.to(DEV).data_ptr(), 0, C.data_ptr(), 1,
                                 M, N, K, K, K, N, block, torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and torch.equal(C, one)


def test_no_workspace_wanted_where_nothing_would_split(lib):
    assert lib.bi8_gemm_workspace_bytes(8192, 8192, 8192, 128) == 0       # plenty of tiles
    assert lib.bi8_gemm_workspace_bytes(16, 4096, 4096, 128) == 0         # few-row kernels
    assert lib.bi8_gemm_workspace_bytes(128, 4096, 4100, 128) == 0        # K not a multiple of 128: general kernel
    assert lib.bi8_gemm_workspace_bytes(128, 4096, 1024, 128) == 0        # eight stages of K: too few to split
    assert lib.bi8_gemm_workspace_bytes(128, 4096, 4096, 16) == 0         # block size of the general kernel


def test_operator_uses_the_split(lib):
    """through the Python operator (which allocates the workspace): same tolerance, and deterministic from call to call"""
    import blockwise_int8_linear_amd as pkg
    M, N, K, block = 128, 1024, 8192, 128
    A, W, sa, sw, bias = _problem(M, N, K, block, seed=9)
    cfg = pkg.block_linear_config
    old = (cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE)
    cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = block, torch.float32
    try:
        c1 = pkg.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa.to(DEV), sw.to(DEV), bias.to(DEV))
        c2 = pkg.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa.to(DEV), sw.to(DEV), bias.to(DEV))
    finally:
        cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = old
    ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw, block, bias, torch.float32)
    assert torch.equal(c1, c2)
    assert torch.allclose(c1.cpu(), ref, rtol=1e-4, atol=1e-4 * ref.abs().max().item())
