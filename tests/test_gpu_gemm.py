"""GPU parity of the int8 block GEMM with fused dequantize against the CPU checker: int32 block partials
bit-exact, outputs within rel 1e-3 (fp32 out) / 1e-2 (bf16, fp16 out).  All calls go through the C ABI."""
import pytest
import torch

import oracle
from oracle import oracle_torch
from util import DTYPES, f32_from_bits, load_golden

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"f32": 1e-3, "bf16": 1e-2, "f16": 1e-2}


@pytest.fixture(scope="module")
def ops():
    import blockwise_int8_linear_amd as pkg
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return pkg


class cfg_as:
    def __init__(self, ops, block=None, out=None):
        self.cfg, self.block, self.out = ops.block_linear_config, block, out

    def __enter__(self):
        self.old = (self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE)
        if self.block:
            self.cfg.GROUP_SIZE = self.block
        if self.out:
            self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.out

    def __exit__(self, *a):
        self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.old


def _codes(g, *shape):
    return torch.randint(-127, 128, shape, generator=g, dtype=torch.int32).to(torch.int8)


def _reference(A, W, sa, sw, B, bias, out_dtype):
    """checker output and the magnitude sum_j |term_j| that bounds fp32 re-association error"""
    P = oracle_torch.gemm_nt_partials(A, W, B)
    ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw, B, bias, out_dtype)
    mag = torch.zeros(P.shape[1:], dtype=torch.float64)
    for j in range(P.shape[0]):
        mag += P[j].abs().double() * sa[j].double()[:, None] * sw[j].double()[None, :]
    return P, ref, mag / (127.0 * 127.0)


def _assert_close(C, ref, mag, tol):
    err = (C.double() - ref.double()).abs()
    bound = tol * ref.double().abs() + 4e-6 * mag + 1e-30
    if not (err <= bound).all():
        i = (err - bound).argmax()
        raise AssertionError(f"max violation at flat index {i.item()}: got {C.view(-1)[i].item()} want {ref.view(-1)[i].item()} "
                             f"(err {err.view(-1)[i].item():.3e}, bound {bound.view(-1)[i].item():.3e})")


def test_gemm_golden(ops):
    for case in load_golden("kat_gemm.json"):
        A = torch.tensor(case["A"], dtype=torch.int8)
        W = torch.tensor(case["W"], dtype=torch.int8)
        sa = torch.stack([f32_from_bits(r) for r in case["sa_bits"]])
        sw = torch.stack([f32_from_bits(r) for r in case["sw_bits"]])
        with cfg_as(ops, case["block"], torch.float32):
            P = ops.int8_matmul_block_partials(A.to(DEV), W.to(DEV).t())
            C = ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa.to(DEV), sw.to(DEV))
        assert P.cpu().tolist() == case["P"]
        exp = torch.tensor(case["C_f32"], dtype=torch.float64)
        assert ((C.cpu().double() - exp).abs() <= 1e-5 * exp.abs() + 1e-12).all()


# (M, N, K): ragged shapes from the reference's commented list (triton_functions.py:583-588), then shapes that
# select each tiled kernel (K multiple of 128): 64x128, 128x128 and 256x128 tiles, and (the last four, >= 160
# tiles of 256x256) the 256x256-tile kernel of block 128 with an even, an odd and a longer run of K stages
# and with a single stage
SHAPES = [(253, 257, 234), (129, 266, 75), (389, 138, 45), (256, 512, 512), (1, 384, 256), (16, 1000, 1024),
          (64, 128, 128), (48, 700, 640), (100, 300, 384), (300, 500, 512), (1024, 512, 512), (3584, 3584, 256), (3500, 3700, 384),
          (2304, 4500, 1152), (2560, 4096, 128),
          (4400, 4501, 384),       # 324 tiles of 256x256, ragged edges: one round on the 256x256 kernel, the last four rows of tiles on 128x128 tiles
          (5200, 5101, 384),       # 420 tiles: more than one per workgroup of the persistent grid
          (5, 130, 66048)]         # a long contraction for the few-row kernel: 516 stages


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("block", [32, 64, 128])
def test_partials_bit_exact(ops, shape, block):
    M, N, K = shape
    g = torch.Generator().manual_seed(M + N + K + block)
    A, W = _codes(g, M, K), _codes(g, N, K)
    P = ops.int8_matmul_block_partials(A.to(DEV), W.to(DEV).t(), block)
    ref = oracle_torch.gemm_nt_partials(A, W, block)
    assert P.dtype == torch.int32 and P.shape == ref.shape
    assert torch.equal(P.cpu(), ref)
    if M * N * K <= 64 * 1024 * 1024:
        assert torch.equal(ref, oracle.gemm_nt_partials(A, W, block, threads=True))


def test_partials_saturated(ops):
    A = torch.full((130, 256), 127, dtype=torch.int8)
    W = torch.full((70, 256), -127, dtype=torch.int8)
    P = ops.int8_matmul_block_partials(A.to(DEV), W.to(DEV).t(), 128)
    assert (P == -128 * 127 * 127).all()


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("block", [32, 64, 128])
@pytest.mark.parametrize("out", ["f32", "bf16"])
def test_gemm_dequant_parity(ops, shape, block, out):
    M, N, K = shape
    g = torch.Generator().manual_seed(M * 3 + N + K + block)
    A, W = _codes(g, M, K), _codes(g, N, K)
    nblk = -(-K // block)
    sa = torch.rand(nblk, M, generator=g) * 4 + 0.01
    sw = torch.rand(nblk, N, generator=g) * 0.1 + 1e-4
    bias = torch.randn(N, generator=g)
    _, ref, mag = _reference(A, W, sa, sw, block, None, DTYPES[out])
    with cfg_as(ops, block, DTYPES[out]):
        Ad, Wd, sad, swd = A.to(DEV), W.to(DEV), sa.to(DEV), sw.to(DEV)
        C = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sad, swd)
        Cb = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sad, swd, bias.to(DEV))
    assert C.dtype == DTYPES[out] and C.shape == (M, N)
    _assert_close(C.cpu(), ref, mag, TOL[out])
    # bias is added after the cast, in the output dtype (triton_functions.py:127-131): an exact identity
    assert torch.equal(Cb, C + bias.to(DEV).to(DTYPES[out]))


def test_gemm_fp16_out_and_bias_dtypes(ops):
    g = torch.Generator().manual_seed(1)
    M, N, K, B = 200, 260, 512, 128
    A, W = _codes(g, M, K), _codes(g, N, K)
    sa = torch.rand(K // B, M, generator=g); sw = torch.rand(K // B, N, generator=g) * 0.05
    _, ref, mag = _reference(A, W, sa, sw, B, None, torch.float16)
    with cfg_as(ops, B, torch.float16):
        C = ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa.to(DEV), sw.to(DEV))
        _assert_close(C.cpu(), ref, mag, TOL["f16"])
        for bd in (torch.float32, torch.bfloat16, torch.float16):
            bias = torch.randn(N, generator=g).to(bd)
            Cb = ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa.to(DEV), sw.to(DEV), bias.to(DEV))
            assert torch.equal(Cb, C + bias.to(DEV).to(torch.float16))


@pytest.mark.parametrize("out", ["bf16", "f16"])
@pytest.mark.parametrize("block", [64, 128])
def test_bias_dtypes_on_the_persistent_kernel(ops, out, block):
    """gemm_wide stages the bias of a tile's 256 columns in LDS as one dword per column, whatever its type; a workgroup
    that walks on to a second tile fetches that tile's bias after a barrier.  Odd N: the last tile's bias ends mid-dword."""
    from blockwise_int8_linear_amd import _lib
    g = torch.Generator().manual_seed(7 + block)
    M, N, K = 5200, 5101, 256
    assert _lib.load().bi8_gemm_kernel_name(M, N, K, K, K, block, 0).decode() == "gemm_wide"
    A, W = _codes(g, M, K).to(DEV), _codes(g, N, K).to(DEV)
    sa = (torch.rand(K // block, M, generator=g) + 0.1).to(DEV)
    sw = (torch.rand(K // block, N, generator=g) * 0.05 + 1e-3).to(DEV)
    with cfg_as(ops, block, DTYPES[out]):
        C = ops.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw)
        for bd in (torch.float32, torch.bfloat16, torch.float16):
            bias = (torch.randn(N, generator=g) * 3).to(bd).to(DEV)
            Cb = ops.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw, bias)
            assert torch.equal(Cb, C + bias.to(DTYPES[out]))             # added after the cast, in the output dtype


@pytest.mark.parametrize("M,N,K", [(7, 11008, 4224), (16, 11008, 4608), (3, 8192, 4224), (17, 11008, 4224), (32, 8192, 4352), (25, 4096, 2048)])
def test_small_batches_against_many_columns_call_after_call(ops, M, N, K):
    """3 to 32 rows against more than 6144 columns and a K beyond 4096 run gemv_staged with four waves per workgroup, two or three workgroups
    per CU (the last shape: eight waves, one workgroup per CU).  Every wave streams W and A through a private LDS ring with direct-to-LDS loads; a load that overwrites a slot
    must not be issued while the stage before is still reading it (a load of A, which the CU's L1 holds for the younger
    workgroups, can land within an LDS read's latency: such workgroups used to return wrong sums now and then).  Ten calls
    on fresh weights, each compared with the same rows run through the tile kernels inside a 33-row problem."""
    from blockwise_int8_linear_amd import _lib
    block = 128
    assert _lib.load().bi8_gemm_kernel_name(M, N, K, K, K, block, 0).decode() == "gemv_staged"
    with cfg_as(ops, block, torch.float32):
        for it in range(10):
            g = torch.Generator().manual_seed(1000 * M + it)
            W, A = _codes(g, N, K).to(DEV), _codes(g, M, K).to(DEV)
            sa = (torch.rand(K // block, M, generator=g) + 0.5).to(DEV)
            sw = (torch.rand(K // block, N, generator=g) * 0.02 + 1e-3).to(DEV)
            Ap = torch.zeros(33, K, device=DEV, dtype=torch.int8)
            Ap[:M] = A
            sap = torch.zeros(K // block, 33, device=DEV)
            sap[:, :M] = sa
            want = ops.int8_matmul_block64_rowwise_dequantize(Ap, W.t(), sap, sw)[:M]
            for _ in range(3):
                got = ops.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw)
                bad = (got - want).abs() > 1e-4 * want.abs() + 1e-5
                assert not bad.any(), f"round {it}: {int(bad.sum())} elements off in workgroups {sorted(set((bad.nonzero()[:, 1] // 16).tolist()))[:8]}"
        # and one of them against the CPU checker
        ref = oracle_torch.int8_matmul_block_dequantize(A.cpu(), W.cpu(), sa.cpu(), sw.cpu(), block, None, torch.float32)
        assert ((got.cpu() - ref).abs() <= 1e-3 * ref.abs() + 1e-6).all()


def test_operand_layouts(ops):
    """b given as a contiguous [K,N] tensor, operands that are column slices of wider buffers, misaligned views"""
    g = torch.Generator().manual_seed(2)
    M, N, K, B = 150, 200, 384, 128
    Abig, Wbig = _codes(g, M, K + 64).to(DEV), _codes(g, N, K + 48).to(DEV)
    sa = torch.rand(K // B, M, generator=g).to(DEV); sw = torch.rand(K // B, N, generator=g).to(DEV)
    with cfg_as(ops, B, torch.float32):
        A, W = Abig[:, 16:16 + K], Wbig[:, 32:32 + K]                        # aligned starts, ld > K
        base = ops.int8_matmul_block64_rowwise_dequantize(A.contiguous(), W.contiguous().t(), sa, sw)
        assert torch.equal(ops.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw), base)
        assert torch.equal(ops.int8_matmul_block64_rowwise_dequantize(A, W.t().contiguous(), sa, sw), base)
        A2, W2 = Abig[:, 3:3 + K], Wbig[:, 5:5 + K]                          # misaligned -> fallback kernel
        ref = ops.int8_matmul_block64_rowwise_dequantize(A2.contiguous(), W2.contiguous().t(), sa, sw)
        got = ops.int8_matmul_block64_rowwise_dequantize(A2, W2.t(), sa, sw)
        assert (got - ref).abs().max() <= 1e-5 * ref.abs().max()
        with pytest.raises(AssertionError, match="incompatible dimensions"):
            ops.int8_matmul_block64_rowwise_dequantize(A, W[:, :-1].t(), sa, sw)


# decode-like shapes (few rows): (M, N, K); K a multiple of 128 selects the few-row kernel, 200 and 1000 do not
FEW_ROWS = [(1, 32, 128), (1, 4096, 4096), (2, 33, 256), (7, 1000, 1152), (16, 4096, 1024), (31, 500, 2048),
            (32, 96, 8192), (32, 2049, 384), (5, 300, 200), (32, 64, 1000)]


@pytest.mark.parametrize("shape", FEW_ROWS)
@pytest.mark.parametrize("block", [32, 64, 128])
def test_few_rows_parity(ops, shape, block):
    """M <= 32 (one token / a small decode batch): outputs against the checker for every output dtype, bias as an
    exact identity, and row r of a batch equal to the same row computed alone (no cross-row leakage)"""
    M, N, K = shape
    g = torch.Generator().manual_seed(7 * M + N + K + block)
    A, W = _codes(g, M, K), _codes(g, N, K)
    nblk = -(-K // block)
    sa = torch.rand(nblk, M, generator=g) * 4 + 0.01
    sw = torch.rand(nblk, N, generator=g) * 0.1 + 1e-4
    sa[nblk // 2, M // 2] = 0.0                                    # an all-zero block has scale 0
    bias = torch.randn(N, generator=g)
    Ad, Wd, sad, swd = A.to(DEV), W.to(DEV), sa.to(DEV), sw.to(DEV)
    for out in ("f32", "bf16", "f16"):
        _, ref, mag = _reference(A, W, sa, sw, block, None, DTYPES[out])
        with cfg_as(ops, block, DTYPES[out]):
            C = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sad, swd)
            Cb = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sad, swd, bias.to(DEV))
            r = M - 1
            Cr = ops.int8_matmul_block64_rowwise_dequantize(Ad[r:r + 1], Wd.t(), sad[:, r:r + 1].contiguous(), swd)
        assert C.dtype == DTYPES[out] and C.shape == (M, N)
        _assert_close(C.cpu(), ref, mag, TOL[out])
        assert torch.equal(Cb, C + bias.to(DEV).to(DTYPES[out]))
        # one row alone may run a different kernel than the batch (other summation order): same bound as against the checker
        _assert_close(Cr[0].cpu(), ref[r], mag[r], TOL[out])
        assert ((Cr[0].double() - C[r].double()).abs().cpu() <= 2 * TOL[out] * ref[r].double().abs() + 8e-6 * mag[r]).all()


def test_few_rows_operand_views(ops):
    """few-row kernel on operands that are column slices of wider buffers (leading dimension > K)"""
    g = torch.Generator().manual_seed(11)
    M, N, K, B = 8, 200, 512, 128
    Abig, Wbig = _codes(g, M, K + 64).to(DEV), _codes(g, N, K + 48).to(DEV)
    sa = torch.rand(K // B, M, generator=g).to(DEV); sw = torch.rand(K // B, N, generator=g).to(DEV)
    with cfg_as(ops, B, torch.float32):
        A, W = Abig[:, 16:16 + K], Wbig[:, 32:32 + K]
        base = ops.int8_matmul_block64_rowwise_dequantize(A.contiguous(), W.contiguous().t(), sa, sw)
        assert torch.equal(ops.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw), base)
        _, ref, mag = _reference(A.cpu(), W.cpu(), sa.cpu(), sw.cpu(), B, None, torch.float32)
        _assert_close(base.cpu(), ref, mag, TOL["f32"])


@pytest.mark.parametrize("block", [32, 64, 128])
def test_vocabulary_sized_contraction(ops, block):
    """K not a multiple of 128 with an odd leading dimension (the GPT-2 vocabulary 50257 as contraction, scaled
    down): the operator pads the codes with zeros and runs the tiled kernels; same numbers as the checker, and the
    same as the general kernel on a problem small enough to stay there"""
    g = torch.Generator().manual_seed(block)
    M, N, K = 300, 200, 5027
    A, W = _codes(g, M, K), _codes(g, N, K)
    nblk = -(-K // block)
    sa = torch.rand(nblk, M, generator=g) + 0.1
    sw = torch.rand(nblk, N, generator=g) * 0.05 + 1e-3
    bias = torch.randn(N, generator=g)
    _, ref, mag = _reference(A, W, sa, sw, block, None, torch.float32)
    with cfg_as(ops, block, torch.float32):
        Ad, Wd, sad, swd = A.to(DEV), W.to(DEV), sa.to(DEV), sw.to(DEV)
        C = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sad, swd)
        Cb = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sad, swd, bias.to(DEV))
        small = ops.int8_matmul_block64_rowwise_dequantize(Ad[:8], Wd[:16].t(), sad[:, :8].contiguous(), swd[:, :16].contiguous())
    _assert_close(C.cpu(), ref, mag, TOL["f32"])
    assert torch.equal(Cb, C + bias.to(DEV))
    _assert_close(small.cpu(), ref[:8, :16], mag[:8, :16], TOL["f32"])
    assert ((small - C[:8, :16]).abs().cpu().double() <= 8e-6 * mag[:8, :16] + 2e-3 * ref[:8, :16].abs().double()).all()


@pytest.mark.parametrize("block", [16, 48, 256])
def test_other_block_sizes_run_the_general_kernel(ops, block):
    g = torch.Generator().manual_seed(block)
    M, N, K = 70, 90, 480
    A, W = _codes(g, M, K), _codes(g, N, K)
    nblk = -(-K // block)
    sa = torch.rand(nblk, M, generator=g) + 0.1
    sw = torch.rand(nblk, N, generator=g) * 0.05 + 1e-3
    P_ref, ref, mag = _reference(A, W, sa, sw, block, None, torch.float32)
    with cfg_as(ops, block, torch.float32):
        C = ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa.to(DEV), sw.to(DEV))
        P = ops.int8_matmul_block_partials(A.to(DEV), W.to(DEV).t())
    _assert_close(C.cpu(), ref, mag, TOL["f32"])
    assert torch.equal(P.cpu(), P_ref)


@pytest.mark.parametrize("block", [256, 512, 1024])
@pytest.mark.parametrize("shape", [(300, 500, 2048), (2048, 2304, 1024), (2944, 2944, 1536), (40, 700, 1280), (300, 500, 1000)])
@pytest.mark.parametrize("out", ["f32", "bf16"])
def test_blocks_above_128_run_the_block_128_kernels(ops, block, shape, out):
    """Blocks of 256, 512, 1024 codes: the operator repeats every scale row block/128 times and runs the GEMM at block 128
    (a block's partial is folded in pieces of 128 codes that share its scales).  Against the checker at the real block
    size, to the GEMM tolerance; K = 1536 and 1280 end in a partial block, K = 1000 also goes through the zero-padded copy.
    With every scale 1 and small codes the pieces add up exactly: the output is the block partials' sum, rounded once."""
    M, N, K = shape
    g = torch.Generator().manual_seed(block + M + K)
    A, W = _codes(g, M, K), _codes(g, N, K)
    nblk = -(-K // block)
    sa = torch.rand(nblk, M, generator=g) + 0.1
    sw = torch.rand(nblk, N, generator=g) * 0.05 + 1e-3
    bias = torch.randn(N, generator=g)
    P_ref, ref, _ = _reference(A, W, sa, sw, block, None, DTYPES[out])
    # the terms that are rounded and added are those of the pieces of 128 codes: where a block's pieces cancel, the error
    # scales with the pieces, not with the block's partial (which can be exactly 0)
    rows = -(-K // 128)
    _, _, mag = _reference(A, W, sa.repeat_interleave(block // 128, 0)[:rows], sw.repeat_interleave(block // 128, 0)[:rows], 128, None, DTYPES[out])
    with cfg_as(ops, block, DTYPES[out]):
        C = ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa.to(DEV), sw.to(DEV))
        Cb = ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa.to(DEV), sw.to(DEV), bias.to(DEV))
    assert C.dtype == DTYPES[out]
    _assert_close(C.cpu(), ref, mag, TOL[out])
    assert torch.equal(Cb, C + bias.to(DEV).to(DTYPES[out]))
    from blockwise_int8_linear_amd import _lib
    lib = _lib.load()
    k128 = -(-K // 128) * 128
    split = "splitk" in lib.bi8_gemm_kernel_name(M, N, k128, k128, k128, 128, lib.bi8_gemm_workspace_bytes(M, N, k128, 128)).decode()
    if out == "f32" and not split:                  # (a split of K scales every piece before it adds them)
        small = torch.randint(-3, 4, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
        with cfg_as(ops, block, torch.float32):
            C1 = ops.int8_matmul_block64_rowwise_dequantize(small.to(DEV), W.to(DEV).t(), torch.ones(nblk, M, device=DEV), torch.ones(nblk, N, device=DEV))
        want = oracle_torch.gemm_nt_partials(small, W, block).sum(0).float() * torch.tensor(1.0 / (127.0 * 127.0), dtype=torch.float32)
        assert torch.equal(C1.cpu(), want)


def test_empty_dimensions(ops):
    """M = 0 and N = 0 give empty outputs; K = 0 gives zeros (plus bias), for few and for many rows"""
    with cfg_as(ops, 128, torch.float32):
        for M, N in ((0, 256), (300, 0), (0, 0)):
            a = torch.empty(M, 256, device=DEV, dtype=torch.int8)
            w = torch.empty(N, 256, device=DEV, dtype=torch.int8)
            c = ops.int8_matmul_block64_rowwise_dequantize(a, w.t(), torch.empty(2, M, device=DEV), torch.empty(2, N, device=DEV))
            assert c.shape == (M, N)
            assert ops.int8_matmul_block_partials(a, w.t()).shape == (2, M, N)
        for M, N in ((3, 40), (200, 300), (4096, 4096)):
            a = torch.empty(M, 0, device=DEV, dtype=torch.int8)
            w = torch.empty(N, 0, device=DEV, dtype=torch.int8)
            sa, sw = torch.empty(0, M, device=DEV), torch.empty(0, N, device=DEV)
            bias = torch.randn(N, device=DEV)
            c = ops.int8_matmul_block64_rowwise_dequantize(a, w.t(), sa, sw)
            assert c.shape == (M, N) and (c == 0).all()
            cb = ops.int8_matmul_block64_rowwise_dequantize(a, w.t(), sa, sw, bias)
            assert torch.equal(cb, bias.expand(M, N))
            assert ops.int8_matmul_block_partials(a, w.t()).shape == (0, M, N)


def test_end_to_end_vs_dense_config1(ops):
    """X fp32 [256,1024] ~N(0,1); W fp32 [1024,1024] ~N(0,0.02); block 64; fp32 out, compared to the fp32
    matmul and to the checker's forward."""
    g = torch.Generator().manual_seed(0)
    X = torch.randn(256, 1024, generator=g); W = torch.randn(1024, 1024, generator=g) * 0.02
    with cfg_as(ops, 64, torch.float32):
        xq, sx = ops.quantize_block_rowwise(X.to(DEV))
        wq, sw = ops.quantize_block_rowwise(W.to(DEV))
        out = ops.int8_matmul_block64_rowwise_dequantize(xq, wq.t(), sx, sw)
        P = ops.int8_matmul_block_partials(xq, wq.t())
    xqo, sxo = oracle.quantize_block_rowwise(X, 64); wqo, swo = oracle.quantize_block_rowwise(W, 64)
    assert torch.equal(xq.cpu(), xqo) and torch.equal(wq.cpu(), wqo) and torch.equal(sx.cpu(), sxo) and torch.equal(sw.cpu(), swo)
    Pref, ref, mag = _reference(xqo, wqo, sxo, swo, 64, None, torch.float32)
    assert torch.equal(P.cpu(), Pref)
    _assert_close(out.cpu(), ref, mag, 1e-3)
    dense = X @ W.t()
    rel = (out.cpu() - dense).norm() / dense.norm()
    assert 1e-3 < rel < 3e-2


@pytest.mark.parametrize("block", [128])
def test_headline_shape_8192(ops, block):
    """M=N=K=8192, bf16 out.  Too big for the scalar checker, so: (i) 96 sampled rows and 96 sampled columns
    against the checker, (ii) every block partial of a 256x256 corner bit-exact, (iii) the result of a row
    subset equals the same rows of the full result (tiles are independent)."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(8192, 8192, generator=g).to(torch.bfloat16)
    w = (torch.randn(8192, 8192, generator=g) * 0.02).to(torch.bfloat16)
    with cfg_as(ops, block, torch.bfloat16):
        xq, sx = ops.quantize_block_rowwise(x.to(DEV))
        wq, sw = ops.quantize_block_rowwise(w.to(DEV))
        C = ops.int8_matmul_block64_rowwise_dequantize(xq, wq.t(), sx, sw)
        rows = torch.randperm(8192, generator=g)[:96]
        cols = torch.randperm(8192, generator=g)[:96]
        xq_c, wq_c, sx_c, sw_c = xq.cpu(), wq.cpu(), sx.cpu(), sw.cpu()
        _, ref, mag = _reference(xq_c[rows], wq_c, sx_c[:, rows].contiguous(), sw_c, block, None, torch.bfloat16)
        _assert_close(C[rows.to(DEV)].cpu(), ref, mag, 1e-2)
        _, ref, mag = _reference(xq_c, wq_c[cols], sx_c, sw_c[:, cols].contiguous(), block, None, torch.bfloat16)
        _assert_close(C[:, cols.to(DEV)].cpu(), ref, mag, 1e-2)
        sub = ops.int8_matmul_block64_rowwise_dequantize(xq[4096:4096 + 512], wq.t(), sx[:, 4096:4096 + 512].contiguous(), sw)
        assert torch.equal(sub, C[4096:4096 + 512])
        P = ops.int8_matmul_block_partials(xq[-256:], wq[-256:].t())
    assert torch.equal(P.cpu(), oracle_torch.gemm_nt_partials(xq_c[-256:], wq_c[-256:], block))
    dense = (x[rows].float() @ w.float().t())
    rel = (C[rows.to(DEV)].cpu().float() - dense).norm() / dense.norm()
    assert rel < 3e-2


def _run_nonfinite_few_rows(ops, A, W, block, g):
    """the same for the kernel of one or two rows: row 0 has an infinite scale in the last block and a NaN scale in
    the first, row 1 an infinite scale on a block whose codes are all zero; then a column scale of inf"""
    M, K = A.shape
    N = W.shape[0]
    nblk = K // block
    j = nblk - 1
    A[1, j * block:] = 0
    sa = torch.rand(nblk, M, generator=g) + 0.1
    sw = torch.rand(nblk, N, generator=g) * 0.05 + 1e-3
    with cfg_as(ops, block, torch.float32):
        run = lambda sa_, sw_: ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa_.to(DEV), sw_.to(DEV)).cpu()
        sa2 = sa.clone()
        sa2[j, 0] = sa2[j, 1] = float("inf")
        ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa2, sw, block, None, torch.float32)
        got = run(sa2, sw)
        assert ref[1].isnan().all() and ref[0].isinf().sum() > N // 2
        assert torch.equal(got.isnan(), ref.isnan()) and torch.equal(got[ref.isinf()], ref[ref.isinf()])
        sa2[0, 0] = float("nan")
        assert run(sa2, sw).isnan().all()
        sw2 = sw.clone()
        sw2[j, 2] = float("inf")
        ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw2, block, None, torch.float32)
        got = run(sa, sw2)
        assert ref[1, 2].isnan() and ref[0, 2].isinf()
        assert torch.equal(got.isnan(), ref.isnan()) and torch.equal(got[ref.isinf()], ref[ref.isinf()])
        fin = torch.isfinite(ref)
        assert ((got[fin] - ref[fin]).abs() <= 1e-3 * ref[fin].abs() + 1e-6).all()


# (M, N, K, kernel family)
NONFINITE_SHAPES = [(300, 500, 512, "gemm_panel"), (1500, 1500, 256, "gemm_panel_square"), (16, 6400, 256, "gemm_panel_few_rows"),
                    (1500, 1500, 256, "gemm_tile_128x128", 32), (2600, 2900, 256, "gemm_wide"), (5200, 5100, 256, "gemm_wide"),
                    (4400, 4500, 256, "gemm_wide+gemm_tile_128x128"), (2048, 2304, 256, "gemm_wide_256x128"),
                    (8, 256, 512, "gemv_staged"), (24, 256, 512, "gemv_staged_two_row_groups"), (24, 256, 512, "gemm_skinny", 32),
                    (70, 90, 200, "gemm_generic"), (8, 256, 2560, "gemv_staged_long"), (2, 256, 1536, "gemv_rows")]


@pytest.mark.parametrize("shape", NONFINITE_SHAPES, ids=lambda s: s[3])
def test_infinite_and_nan_scales(ops, shape):
    """A block that held an infinity has scale inf.  The reference's sw * (sx * (P * div)) (triton_functions.py:120)
    then gives +-inf where the block partial P is not 0 and NaN where it is.  A ROW scale of inf or NaN gives exactly
    that in every kernel.  A COLUMN scale of inf gives it in the few-row and general kernels; the tiled kernels
    (M > 32, and gemm_panel's 32-row tiles for 3 rows or more against 5120 columns or more), whose fold computes fma(1.5*2^23 + P, b, -1.5*2^23 * b), give NaN for the whole column instead of +-inf:
    the one place where non-finite results differ from the reference's, pinned here.  Everything else stays finite."""
    from blockwise_int8_linear_amd import _lib
    M, N, K, family = shape[:4]
    block = shape[4] if len(shape) > 4 else 128 if K % 128 == 0 else 64
    assert _lib.load().bi8_gemm_kernel_name(M, N, K, K, K, block, 0).decode() == family.replace("_long", "").replace("_two_row_groups", "").replace("_square", "").replace("_few_rows", "")
    g = torch.Generator().manual_seed(M + N)
    A, W = _codes(g, M, K), _codes(g, N, K)
    nblk = -(-K // block)
    j = nblk - 1
    if M <= 2:
        _run_nonfinite_few_rows(ops, A, W, block, g)
        return
    A[5, j * block:] = 0                            # this row's partial of block j is 0 for every column
    sa = torch.rand(nblk, M, generator=g) + 0.1
    sw = torch.rand(nblk, N, generator=g) * 0.05 + 1e-3
    with cfg_as(ops, block, torch.float32):
        run = lambda sa_, sw_: ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa_.to(DEV), sw_.to(DEV)).cpu()
        # row scales: inf on rows 3 and 5 (row 5 has P = 0), -inf on row 4, NaN on row 7
        sa2 = sa.clone()
        sa2[j, 3] = sa2[j, 5] = float("inf")
        sa2[j, 4] = float("-inf")
        sa2[j, 7] = float("nan")
        ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa2, sw, block, None, torch.float32)
        got = run(sa2, sw)
        assert ref[5].isnan().all() and ref[7].isnan().all() and ref[3].isinf().sum() > N // 2
        assert torch.equal(got.isnan(), ref.isnan()) and torch.equal(got.isinf(), ref.isinf())
        assert torch.equal(got[ref.isinf()], ref[ref.isinf()])             # the signs of the infinities
        fin = torch.isfinite(ref)
        assert fin[8:].all() and ((got[fin] - ref[fin]).abs() <= 1e-3 * ref[fin].abs() + 1e-6).all()
        # a column scale of inf
        sw2 = sw.clone()
        sw2[j, 2] = float("inf")
        ref = oracle_torch.int8_matmul_block_dequantize(A, W, sa, sw2, block, None, torch.float32)
        got = run(sa, sw2)
        assert ref[5, 2].isnan() and ref[:, 2].isinf().sum() >= M - 3
        if family in ("gemv_staged", "gemv_staged_long", "gemv_staged_two_row_groups", "gemm_skinny", "gemm_generic"):
            assert torch.equal(got.isnan(), ref.isnan()) and torch.equal(got[ref.isinf()], ref[ref.isinf()])
        else:
            assert got[:, 2].isnan().all()
        other = torch.ones(N, dtype=torch.bool)
        other[2] = False
        assert torch.isfinite(got[:, other]).all() and ((got[:, other] - ref[:, other]).abs() <= 1e-3 * ref[:, other].abs() + 1e-6).all()
