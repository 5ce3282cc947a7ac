"""The one-kernel quantize + GEMM of the eval path for one or two rows (bi8_linear_few_rows) against the two launchers it
replaces -- same bits -- and against the CPU checker; the cases it does not cover hand back to the two launchers."""
import pytest
import torch

from oracle import oracle_torch
from util import DTYPES, outlier_tensor

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"f32": 1e-3, "bf16": 1e-2, "f16": 1e-2}


@pytest.fixture(scope="module")
def pkg():
    import blockwise_int8_linear_amd as p
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return p


class cfg_as:
    def __init__(self, pkg, block, out):
        self.cfg, self.block, self.out = pkg.block_linear_config, block, out

    def __enter__(self):
        self.old = (self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE)
        self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.block, self.out

    def __exit__(self, *a):
        self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.old


def _weights(pkg, N, K, dtype, seed):
    w = (torch.randn(N, K, generator=torch.Generator().manual_seed(seed)) * 0.02).to(dtype)
    q, s = pkg.quantize_block_rowwise(w.to(DEV))
    return w, q, s


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("block", [64, 128])
@pytest.mark.parametrize("M,K,N", [(1, 128, 16), (1, 4096, 4096), (2, 1024, 50), (2, 640, 1000), (2, 5120, 300),
                                   (1, 11008, 4096), (2, 256, 17), (1, 5120, 33)])
def test_same_bits_as_the_two_launchers(pkg, M, K, N, block, dtype):
    dt = DTYPES[dtype]
    with cfg_as(pkg, block, dt):
        w, Wq, Ws = _weights(pkg, N, K, dt, seed=K + N)
        x_cpu = outlier_tensor(M, K, dt, seed=M * 7 + K)
        x = x_cpu.to(DEV)
        bias = torch.randn(N, generator=torch.Generator().manual_seed(5)).to(dt).to(DEV)
        xq, xs = pkg.quantize_block_rowwise(x)
        from blockwise_int8_linear_amd.ops import _few_rows_lds
        fits = _few_rows_lds(M, K, block, x.element_size()) <= 65536      # x, its codes and the scales sit in LDS
        assert fits or (K > 8192 and dtype == "f32")
        for b in (None, bias):
            two = pkg.int8_matmul_block64_rowwise_dequantize(xq, Wq.t(), xs, Ws, b)
            one = pkg.linear_few_rows(x, Wq, Ws, b)
            if not fits:
                assert one is None
                continue
            assert one is not None and one.dtype == dt and one.shape == (M, N)
            view = torch.int32 if dtype == "f32" else torch.int16
            assert torch.equal(one.view(view), two.view(view)), (M, K, N, block, dtype, b is not None)
        if K * N <= 1 << 22 and fits:
            ref = oracle_torch.linear_forward(x_cpu, w, None, block, dt)
            one = pkg.linear_few_rows(x, Wq, Ws, None).cpu()
            rel = ((one.double() - ref.double()).norm() / ref.double().norm()).item()
            assert rel < TOL[dtype], rel


def test_special_blocks(pkg):
    """zero blocks, a NaN element, an inf element, subnormal and huge magnitudes: same codes and scales as the row
    quantizer, so the same output bits (NaN compares through the bit pattern)"""
    M, K, N, block, dt = 2, 768, 64, 128, torch.float32
    with cfg_as(pkg, block, dt):
        _, Wq, Ws = _weights(pkg, N, K, dt, seed=1)
        x = torch.randn(M, K, generator=torch.Generator().manual_seed(2))
        x[0, :128] = 0.0
        x[0, 130] = float("nan")
        x[1, 260] = float("inf")
        x[1, 384:512] *= 1e-42
        x[0, 512:640] *= 1e35
        x = x.to(DEV)
        xq, xs = pkg.quantize_block_rowwise(x)
        two = pkg.int8_matmul_block64_rowwise_dequantize(xq, Wq.t(), xs, Ws)
        one = pkg.linear_few_rows(x, Wq, Ws)
        assert torch.equal(one.view(torch.int32), two.view(torch.int32))


def test_row_views_and_padding(pkg):
    """x a row slice of a wider buffer, W with a padded leading dimension"""
    M, K, N, block, dt = 2, 768, 96, 64, torch.bfloat16
    with cfg_as(pkg, block, dt):
        _, Wq, Ws = _weights(pkg, N, K, dt, seed=3)
        Wpad = torch.zeros(N, K + 64, dtype=torch.int8, device=DEV)
        Wpad[:, :K] = Wq
        xbig = outlier_tensor(5, K + 32, dt, seed=4).to(DEV)
        x = xbig[1:3, :K]
        xq, xs = pkg.quantize_block_rowwise(x)
        two = pkg.int8_matmul_block64_rowwise_dequantize(xq, Wq.t(), xs, Ws)
        one = pkg.linear_few_rows(x, Wpad[:, :K], Ws)
        assert torch.equal(one.view(torch.int16), two.view(torch.int16))


def test_uncovered_cases_return_none(pkg):
    dt = torch.bfloat16
    with cfg_as(pkg, 128, dt):
        _, Wq, Ws = _weights(pkg, 32, 256, dt, seed=6)
        x5 = torch.randn(5, 256).to(dt).to(DEV)
        assert pkg.linear_few_rows(x5, Wq, Ws) is None and pkg.linear_few_rows(x5[:3], Wq, Ws) is None   # five rows, three rows
        assert pkg.linear_few_rows(x5[:1].float(), Wq, Ws) is None                # x not of the configured type
        xodd = torch.randn(1, 257).to(dt).to(DEV)[:, 1:]                          # rows not 16-byte aligned
        assert pkg.linear_few_rows(xodd, Wq, Ws) is None
    with cfg_as(pkg, 32, dt):
        assert pkg.linear_few_rows(x5[:1], Wq, torch.ones(8, 32, device=DEV)) is None   # block 32
    with cfg_as(pkg, 128, dt):
        _, Wq, Ws = _weights(pkg, 16, 16384, dt, seed=7)
        assert pkg.linear_few_rows(torch.randn(2, 16384).to(dt).to(DEV), Wq, Ws) is None   # two such rows and their codes exceed the LDS budget
        one = pkg.linear_few_rows(torch.randn(1, 16384).to(dt).to(DEV), Wq, Ws)
        assert one is not None and torch.isfinite(one.float()).all()


def test_module_decode_uses_it_and_matches_prefill_rows(pkg):
    """BlockInt8Linear in eval mode: a one-row call equals the matching row of a many-row call to tolerance (different
    kernels) and equals the two-launcher result bit for bit"""
    K, N, block, dt = 1024, 512, 128, torch.bfloat16
    torch.manual_seed(11)
    with cfg_as(pkg, block, dt):
        lin = pkg.BlockInt8Linear(K, N, bias=True, device=DEV, dtype=dt).eval()
        x = torch.randn(2, 40, K, device=DEV).to(dt)
        with torch.no_grad():
            full = lin(x)
            one = lin(x[1:2, 7:8])
            xq, xs = pkg.quantize_block_rowwise(x[1, 7:8])
            two = pkg.int8_matmul_block64_rowwise_dequantize(xq, lin.W_int8.t(), xs, lin.state_W, lin.bias)
        assert one.shape == (1, 1, N)
        assert torch.equal(one.view(-1), two.view(-1))
        assert torch.allclose(one.float().view(-1), full[1, 7].float(), rtol=2e-2, atol=1e-3)
