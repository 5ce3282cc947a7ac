"""GPU parity of the block quantizer / dequantizer / transposed quantizer with the CPU checker:
int8 codes and fp32 scales bit-exact, dequantized values bit-exact.  Every call goes through the
C ABI of libbi8.so (ops -> ctypes)."""
import pytest
import torch

import oracle
from util import DTYPES, bits_to_tensor, f32_from_bits, load_golden, outlier_tensor

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import blockwise_int8_linear_amd as pkg
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return pkg


def _check_quant(ops, x_cpu, block, transposed=False):
    x = x_cpu.to(DEV)
    if transposed:
        q, s = ops.quantize_block_transposed(x, block)
        qo, so = oracle.quantize_block_transposed(x_cpu, block, threads=True)
    else:
        q, s = ops.quantize_block_rowwise(x, block)
        qo, so = oracle.quantize_block_rowwise(x_cpu, block, threads=True)
    torch.cuda.synchronize()
    assert q.dtype == torch.int8 and s.dtype == torch.float32
    assert q.shape == qo.shape and s.shape == so.shape
    sc, qc = s.cpu(), q.cpu()
    assert torch.equal(sc.view(torch.int32), so.view(torch.int32)), "scales differ"
    if not torch.equal(qc, qo):
        bad = (qc != qo).nonzero()
        raise AssertionError(f"{bad.shape[0]} codes differ, first at {bad[0].tolist()}: got {qc[tuple(bad[0])]} want {qo[tuple(bad[0])]}")
    return q, s


def test_quantize_golden(ops):
    for case in load_golden("kat_quantize.json"):
        x = bits_to_tensor(case["x_bits"], case["dtype"]).reshape(1, -1)
        q, s = ops.quantize_block_rowwise(x.to(DEV), case["block"])
        assert q.cpu().view(-1).tolist() == case["codes"], case["name"]
        assert torch.equal(s.cpu().view(-1), f32_from_bits(case["scale_bits"])), case["name"]
        # the same block repeated over 40 rows x 3 blocks exercises the vector kernels where the shape allows
        n, B = x.shape[1], case["block"]
        if n % B == 0:
            xx = x.repeat(40, 3).to(DEV)
            q2, s2 = ops.quantize_block_rowwise(xx, B)
            assert torch.equal(q2.cpu(), torch.tensor(case["codes"], dtype=torch.int8).repeat(40, 3)), case["name"]
            assert torch.equal(s2.cpu(), f32_from_bits(case["scale_bits"]).reshape(-1, 1).repeat(3, 40)), case["name"]


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("block", [16, 32, 64, 128, 256])
def test_quantize_parity_seeded(ops, dtype, block):
    for (M, K) in [(256, 1024), (37, 4096), (1, 11008), (130, 2048 + 8 * 5), (5, 1000), (19, 333), (9, 5027)]:
        x = outlier_tensor(M, K, DTYPES[dtype], seed=M + K + block)
        _check_quant(ops, x, block)


@pytest.mark.parametrize("block", [8, 24, 100, 512, 1024, 2048])
def test_quantize_unusual_blocks(ops, block):
    x = outlier_tensor(33, 4096, torch.bfloat16, seed=block)
    _check_quant(ops, x, block)
    _check_quant(ops, x.float(), block)
    _check_quant(ops, x[:, :1500].contiguous(), block, transposed=True)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
def test_quantize_special_values(ops, dtype):
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(1)
    x = torch.randn(64, 1024, generator=g)
    x[0] = 0.0                                   # all-zero blocks
    x[1, :128] = 0.0
    x[2] *= 1e-30 if dtype != "f16" else 1e-6    # tiny scales
    x[3] *= 1e-41 if dtype != "f16" else 3e-7    # subnormal scales
    x[4] *= 1e30 if dtype != "f16" else 1e3      # huge scales
    x[5, 7] = float("inf")
    x[6, 9] = float("nan")
    x[7, 100] = float("-inf")
    x[7, 101] = float("nan")
    x[8, ::2] = -0.0
    x = x.to(dt)
    for block in (32, 128):
        _check_quant(ops, x, block)
        _check_quant(ops, x, block, transposed=True)
        _check_quant(ops, x[:, :1001].contiguous(), block)      # generic kernels see the same values


@pytest.mark.parametrize("block", [32, 64, 128])
def test_roundtrip_full_size_bf16(ops, block):
    """[8192,8192] bf16 ~N(0,1) with 0.1% of the entries x50, bit-exact against the checker at full size,
    plus the properties that do not depend on it."""
    x_cpu = outlier_tensor(8192, 8192, torch.bfloat16, seed=0)
    q, s = _check_quant(ops, x_cpu, block)
    x = x_cpu.to(DEV)
    xb = x.float().reshape(8192, -1, block)
    qb = q.reshape(8192, -1, block).int()
    idx = xb.abs().argmax(-1, keepdim=True)
    assert (qb.gather(-1, idx).abs() == 127).all()                         # the absmax element saturates
    q2, s2 = ops.quantize_block_rowwise(x * 4, block)                       # power-of-two equivariance
    assert torch.equal(q2, q) and torch.equal(s2, s * 4)
    import blockwise_int8_linear_amd as pkg
    d = pkg.dequantize_block_rowwise(q, s, block)
    do = oracle.dequantize_block_rowwise(q.cpu(), s.cpu(), block, torch.bfloat16, threads=True)
    assert torch.equal(d.cpu().view(torch.int16), do.view(torch.int16))
    err = (d.float().reshape(8192, -1, block) - xb).abs()
    bound = s.t().unsqueeze(-1) * (1 / 254 + 2.0 ** -8)                     # half a code step + bf16 rounding
    assert (err <= bound).all()
    mse = (err ** 2).mean().item()
    assert 0 < mse < 1e-2


@pytest.mark.parametrize("out", ["f32", "bf16", "f16"])
def test_dequantize_parity(ops, out):
    cfg = ops.block_linear_config
    old = cfg.INPUT_OUTPUT_TORCH_TYPE
    cfg.INPUT_OUTPUT_TORCH_TYPE = DTYPES[out]
    try:
        for case in load_golden("kat_dequantize.json"):
            codes = torch.tensor(case["codes"], dtype=torch.int8).reshape(1, -1)
            s = f32_from_bits([case["scale_bits"]]).reshape(1, 1)
            d = ops.dequantize_block_rowwise(codes.to(DEV), s.to(DEV), codes.shape[1]).cpu().double().view(-1)
            exp = case[f"out_{out}"]
            for got, e in zip(d.tolist(), exp):
                assert (e is None and got in (float("inf"), float("-inf"))) or got == e
        g = torch.Generator().manual_seed(3)
        for (M, K, B) in [(64, 2048, 128), (33, 1040, 16), (7, 999, 64), (16, 4096, 1024), (3, 70, 24), (5, 5027, 128)]:
            q = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
            s = torch.rand(-(-K // B), M, generator=g) * 3
            d = ops.dequantize_block_rowwise(q.to(DEV), s.to(DEV), B)
            do = oracle.dequantize_block_rowwise(q, s, B, DTYPES[out])
            assert d.dtype == DTYPES[out] and torch.equal(d.cpu().view(torch.int32 if out == "f32" else torch.int16),
                                                           do.view(torch.int32 if out == "f32" else torch.int16))
    finally:
        cfg.INPUT_OUTPUT_TORCH_TYPE = old


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("block", [32, 64, 128])
def test_quantize_transposed_equals_two_step(ops, dtype, block):
    # the last four: odd row lengths of the source and/or of the output (unaligned loads / byte stores in the tile
    # kernel), among them the GPT-2 vocabulary as either dimension; the last two: more tiles than one patch of the tile
    # order in both directions, with and without ragged last bands / chunks
    for (R, C) in [(256, 512), (8192, 768), (300, 1000), (1000, 72), (129, 64), (64, 50257 // 8 * 8),
                   (300, 517), (517, 304), (333, 77), (64, 50257), (50257, 64), (2181, 2115), (2304, 4160)]:
        x_cpu = outlier_tensor(R, C, DTYPES[dtype], seed=R + C)
        q, s = _check_quant(ops, x_cpu, block, transposed=True)
        x = x_cpu.to(DEV)
        q2, s2 = ops.quantize_block_rowwise(x.t().contiguous(), block)      # block_linear.py:93-94
        assert torch.equal(q, q2) and torch.equal(s, s2)


def test_strided_and_edge_inputs(ops):
    big = outlier_tensor(64, 3000, torch.bfloat16, seed=5).to(DEV)
    view = big[:, 8:8 + 2048]                         # leading dimension 3000, 16-byte aligned start
    q, s = ops.quantize_block_rowwise(view, 128)
    q2, s2 = ops.quantize_block_rowwise(view.contiguous(), 128)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    view = big[:, 3:3 + 2048]                         # misaligned start -> generic kernel
    q, s = ops.quantize_block_rowwise(view, 128)
    q2, s2 = ops.quantize_block_rowwise(view.contiguous(), 128)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    tview = big.t()                                   # columns not contiguous -> copied by the wrapper
    q, s = ops.quantize_block_rowwise(tview, 64)
    q2, s2 = ops.quantize_block_transposed(big, 64)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    e = torch.empty(0, 128, device=DEV, dtype=torch.bfloat16)
    q, s = ops.quantize_block_rowwise(e, 128)
    assert q.shape == (0, 128) and s.shape == (1, 0)
    with pytest.raises(AssertionError):
        ops.quantize_block_rowwise(torch.zeros(4, 128), 128)                # CPU tensor: `assert x.is_cuda`
    with pytest.raises(ValueError):
        ops.quantize_block_rowwise(torch.zeros(2, 4, 128, device=DEV), 128)  # 2-D only, like `m, k = x.shape`
    with pytest.raises(TypeError):
        ops.quantize_block_rowwise(torch.zeros(4, 128, device=DEV, dtype=torch.float64), 128)


def test_scale_dtype_follows_config(ops):
    cfg = ops.block_linear_config
    x = outlier_tensor(32, 512, torch.bfloat16, seed=2).to(DEV)
    q, s = ops.quantize_block_rowwise(x)
    assert s.dtype == torch.float32 and s.shape == (512 // cfg.GROUP_SIZE, 32)
    cfg.SHARED_EXP_TORCH_TYPE = torch.bfloat16
    try:
        q2, s2 = ops.quantize_block_rowwise(x)
        assert s2.dtype == torch.bfloat16 and torch.equal(s2, s.to(torch.bfloat16)) and torch.equal(q2, q)
        d = ops.dequantize_block_rowwise(q2, s2)
        assert d.dtype == cfg.INPUT_OUTPUT_TORCH_TYPE
    finally:
        cfg.SHARED_EXP_TORCH_TYPE = torch.float32
