"""Every GEMM kernel family and the quantizers give the same bits call after call on the same operands, and a few of a
problem's rows pushed through a different kernel (inside a 200-row problem, which runs on the tile kernels) give the same
numbers to the output type's tolerance.  A race between waves or workgroups shows here as a difference between two calls
long before it shows against the CPU checker on a small problem: the shapes are the BASELINE configs' (Llama-7B and
GPT-2-small layers), where several workgroups share a CU and most of the chip is busy."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

GEMM_SHAPES = [(1, 11008, 4096), (2, 4096, 11008), (5, 4096, 4096), (16, 12288, 4096), (24, 11008, 4096), (64, 4096, 4096), (128, 11008, 4096),
               (256, 4096, 11008), (1024, 4096, 4096), (2048, 4096, 4096), (1536, 11008, 4096), (3072, 768, 8192), (8192, 2304, 768), (4352, 4096, 2048)]


@pytest.fixture(scope="module")
def pkg():
    import blockwise_int8_linear_amd as p
    return p


def _codes(g, *shape):
    return torch.randint(-127, 128, shape, generator=g, dtype=torch.int32).to(torch.int8).to(DEV)


@pytest.mark.parametrize("block", [128, 64])
@pytest.mark.parametrize("shape", GEMM_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_gemm_call_after_call(pkg, shape, block):
    M, N, K = shape
    cfg = pkg.block_linear_config
    old = (cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE)
    cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = block, torch.bfloat16
    try:
        for it in range(2):
            g = torch.Generator().manual_seed(it * 7919 + M + N + K + block)
            A, W = _codes(g, M, K), _codes(g, N, K)
            sa = (torch.rand(K // block, M, generator=g) + 0.5).to(DEV)
            sw = (torch.rand(K // block, N, generator=g) * 0.02 + 1e-3).to(DEV)
            y1 = pkg.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw)
            y2 = pkg.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw)
            assert torch.equal(y1, y2), f"{int((y1 != y2).sum())} elements differ between two calls"
            rows = torch.randperm(M, generator=g)[:min(M, 8)].to(DEV)
            Ar = torch.zeros(200, K, device=DEV, dtype=torch.int8)
            Ar[:len(rows)] = A[rows]
            sr = torch.zeros(K // block, 200, device=DEV)
            sr[:, :len(rows)] = sa[:, rows]
            y3 = pkg.int8_matmul_block64_rowwise_dequantize(Ar, W.t(), sr, sw)[:len(rows)].float()
            d = (y1[rows].float() - y3).abs()
            assert (d <= 2e-2 * y3.abs() + 2e-3 * y3.abs().mean()).all()
    finally:
        cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = old


@pytest.mark.parametrize("block", [128, 64, 32])
@pytest.mark.parametrize("shape", [(8192, 768), (8192, 3072), (768, 768), (2000, 1000), (16, 4096)], ids=lambda s: "x".join(map(str, s)))
def test_quantizers_call_after_call(pkg, shape, block):
    R, C = shape
    for dt in (torch.bfloat16, torch.float32):
        x = torch.randn(R, C, generator=torch.Generator().manual_seed(R + C + block)).to(dt).to(DEV)
        q1, s1 = pkg.quantize_block_rowwise(x, block)
        q2, s2 = pkg.quantize_block_rowwise(x, block)
        assert torch.equal(q1, q2) and torch.equal(s1, s2)
        a, b = pkg.quantize_block_dual(x, block), pkg.quantize_block_dual(x, block)
        assert all(torch.equal(u, v) for u, v in zip(a, b))
        assert torch.equal(a[0], q1) and torch.equal(a[1], s1)
        qt, st = pkg.quantize_block_rowwise(x.t().contiguous(), block)
        assert torch.equal(a[2], qt) and torch.equal(a[3], st)


@pytest.mark.parametrize("M,N,K,block", [(1536, 11008, 4096, 128), (3072, 768, 8192, 64), (24, 11008, 4096, 128), (128, 4096, 4096, 128),
                                         (4352, 4096, 2048, 128)])
def test_plans_of_several_launches_in_a_hip_graph(pkg, M, N, K, block):
    """the cut (256x256 kernel + tile kernel), the split (tile kernel + reduce, with its workspace from torch's allocator)
    and the few-row kernel recorded into a HIP graph: every replay, with eager work between the replays, equals the eager
    call"""
    cfg = pkg.block_linear_config
    old = (cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE)
    cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = block, torch.bfloat16
    try:
        g = torch.Generator().manual_seed(M + N)
        A, W = _codes(g, M, K), _codes(g, N, K)
        sa = (torch.rand(K // block, M, generator=g) + 0.5).to(DEV)
        sw = (torch.rand(K // block, N, generator=g) * 0.02 + 1e-3).to(DEV)
        bias = torch.randn(N, generator=g).to(torch.bfloat16).to(DEV)
        eager = pkg.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw, bias)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            pkg.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw, bias)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = pkg.int8_matmul_block64_rowwise_dequantize(A, W.t(), sa, sw, bias)
        for _ in range(3):
            out.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
            torch.randn(1 << 20, device=DEV).sum().item()              # eager work and a synchronization between replays
    finally:
        cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = old
