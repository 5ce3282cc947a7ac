"""bi8_quantize_dual (both quantization directions from one pass) against the CPU checker and against the two
single-direction entry points: int8 codes and fp32 scales bit-exact in both outputs."""
import pytest
import torch

import oracle
from util import DTYPES, outlier_tensor

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import blockwise_int8_linear_amd as pkg
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return pkg


def _same(a, b):
    return torch.equal(a.view(torch.int32) if a.dtype == torch.float32 else a, b.view(torch.int32) if b.dtype == torch.float32 else b)


def _check(ops, x_cpu, block, x_dev=None):
    x = x_cpu.to(DEV) if x_dev is None else x_dev
    q, s, qt, st = ops.quantize_block_dual(x, block)
    qo, so = oracle.quantize_block_rowwise(x_cpu, block, threads=True)
    qto, sto = oracle.quantize_block_transposed(x_cpu, block, threads=True)
    assert q.shape == qo.shape and s.shape == so.shape and qt.shape == qto.shape and st.shape == sto.shape
    assert _same(s.cpu(), so), "row scales differ"
    assert _same(st.cpu(), sto), "column scales differ"
    assert torch.equal(q.cpu(), qo), f"{(q.cpu() != qo).sum().item()} row codes differ"
    assert torch.equal(qt.cpu(), qto), f"{(qt.cpu() != qto).sum().item()} column codes differ"
    q1, s1 = ops.quantize_block_rowwise(x, block)
    q2, s2 = ops.quantize_block_transposed(x, block)
    assert torch.equal(q, q1) and _same(s, s1) and torch.equal(qt, q2) and _same(st, s2)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("block", [32, 64, 128])
def test_dual_parity(ops, dtype, block):
    # whole tiles, ragged tiles in either direction, a single partial tile, one row, one 16-byte column group, many
    # tiles per workgroup (more than 768 tiles), and shapes of the training configurations
    for (R, C) in [(256, 256), (128, 128), (300, 1000), (1000, 72), (129, 64), (5, 8), (1, 4096), (4096, 8),
                   (8192, 768), (768, 3072), (2176, 2304), (77, 1048), (2181, 2115)]:
        _check(ops, outlier_tensor(R, C, DTYPES[dtype], seed=R * 3 + C + block), block)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_dual_cases_the_one_pass_kernel_does_not_take(ops, dtype):
    """other block sizes, odd row lengths and misaligned views run the two single-direction kernels: same results"""
    for (R, C, block) in [(200, 264, 16), (96, 520, 256), (90, 77, 64), (64, 517, 128), (300, 50257 // 50, 32)]:
        _check(ops, outlier_tensor(R, C, DTYPES[dtype], seed=R + C), block)
    big = outlier_tensor(130, 700, DTYPES[dtype], seed=9)
    _check(ops, big[:, 3:3 + 512].contiguous(), 128, x_dev=big.to(DEV)[:, 3:3 + 512])        # misaligned start
    _check(ops, big[:, 8:8 + 512].contiguous(), 128, x_dev=big.to(DEV)[:, 8:8 + 512])        # aligned view, ld 700


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("block", [64, 128])
def test_dual_rows_of_odd_length(ops, dtype, block):
    """rows that are only element-aligned (the GPT-2 vocabulary, 50257, as the row length) with 16-byte aligned
    transposed rows: one pass with unaligned 16-byte accesses, the last chunk of each row element by element"""
    for (R, C) in [(256, 50257), (128, 517), (384, 1001), (64, 9), (1024, 131), (272, 4099)]:
        _check(ops, outlier_tensor(R, C, DTYPES[dtype], seed=R + C + block), block)
    big = outlier_tensor(130, 700, DTYPES[dtype], seed=11)
    _check(ops, big[:128, 3:3 + 515].contiguous(), block, x_dev=big.to(DEV)[:128, 3:3 + 515])     # view at an odd element offset


def test_dual_special_values(ops):
    x = torch.randn(256, 256, generator=torch.Generator().manual_seed(1))
    x[0, :128] = 0.0                       # zero row block
    x[:128, 5] = 0.0                       # zero column block
    x[3, 130] = float("nan")
    x[140, 7] = float("inf")
    x[200, 128:256] *= 1e-42               # subnormal block
    x[128:256, 200] *= 1e36                # huge column block
    for block in (64, 128):
        _check(ops, x, block)


def test_dual_full_size(ops):
    """[8192, 8192] bf16, block 128: against the two single-direction kernels (themselves checked against the CPU at
    this size), and a 256 x 8192 slab against the CPU checker"""
    x = outlier_tensor(8192, 8192, torch.bfloat16, seed=0).to(DEV)
    q, s, qt, st = ops.quantize_block_dual(x, 128)
    q1, s1 = ops.quantize_block_rowwise(x, 128)
    q2, s2 = ops.quantize_block_transposed(x, 128)
    assert torch.equal(q, q1) and _same(s, s1) and torch.equal(qt, q2) and _same(st, s2)
    qo, so = oracle.quantize_block_rowwise(x[4096:4352].cpu(), 128, threads=True)
    assert torch.equal(q[4096:4352].cpu(), qo) and _same(s[:, 4096:4352].cpu().contiguous(), so)


def test_dual_empty(ops):
    e = torch.empty(0, 128, device=DEV, dtype=torch.bfloat16)
    q, s, qt, st = ops.quantize_block_dual(e, 128)
    assert q.shape == (0, 128) and s.shape == (1, 0) and qt.shape == (128, 0) and st.shape == (0, 128)


def _colsum_bound(x_cpu, out_dtype):
    """what a different fp32 summation order and the final cast can change: 2^-22 of the column's sum of magnitudes,
    plus one unit in the last place of the output type"""
    ulp = {torch.float32: 2.0 ** -23, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[out_dtype]
    mag = x_cpu.double().abs().sum(0)
    return 2.0 ** -22 * mag + ulp * x_cpu.double().sum(0).abs() + 1e-30


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("block", [32, 64, 128])
def test_dual_with_column_sums(ops, dtype, block):
    """bi8_quantize_dual_colsum: the same four outputs as bi8_quantize_dual bit for bit, and the column sums of x (the
    bias gradient G.sum(dim=0), block_linear.py:110) in x's type; shapes of the one-pass kernel and of the fallbacks"""
    for (R, C) in [(256, 256), (300, 1000), (1000, 72), (129, 64), (5, 8), (1, 4096), (8192, 768), (2181, 2115), (90, 77), (384, 1001)]:
        x_cpu = torch.randn(R, C, generator=torch.Generator().manual_seed(R + C + block)).to(DTYPES[dtype])
        x = x_cpu.to(DEV)
        q, s, qt, st, sums = ops.quantize_block_dual_colsum(x, block)
        q0, s0, qt0, st0 = ops.quantize_block_dual(x, block)
        assert torch.equal(q, q0) and _same(s, s0) and torch.equal(qt, qt0) and _same(st, st0)
        assert sums.shape == (C,) and sums.dtype == x.dtype
        ref = x_cpu.sum(dim=0)                                   # the reference's expression, on the CPU
        assert ((sums.cpu().double() - ref.double()).abs() <= _colsum_bound(x_cpu, x.dtype)).all()
        # the sums do not depend on the block size or on which kernel made them (block 16 runs the fallback kernels)
        assert _same(sums.float(), ops.quantize_block_dual_colsum(x, 16)[4].float())
        # small integers add up exactly in any order
        xi = torch.randint(-8, 9, (R, C), generator=torch.Generator().manual_seed(C)).to(DTYPES[dtype])
        got = ops.quantize_block_dual_colsum(xi.to(DEV), block)[4]
        assert torch.equal(got.cpu(), xi.double().sum(0).to(DTYPES[dtype]))


def test_dual_with_column_sums_special_and_empty(ops):
    x = torch.randn(300, 200, generator=torch.Generator().manual_seed(4))
    x[7, 3] = float("inf")
    x[9, 4] = float("nan")
    x[11, 5] = float("inf"); x[200, 5] = float("-inf")
    sums = ops.quantize_block_dual_colsum(x.to(DEV), 64)[4].cpu()
    ref = x.sum(0)
    assert sums[3] == float("inf") and sums[4].isnan() and sums[5].isnan()
    ok = torch.isfinite(ref)
    assert torch.equal(torch.isfinite(sums), ok) and ((sums[ok] - ref[ok]).abs() <= 1e-4).all()
    e = torch.empty(0, 128, device=DEV, dtype=torch.bfloat16)
    out = ops.quantize_block_dual_colsum(e, 128)
    assert out[0].shape == (0, 128) and out[4].shape == (128,) and (out[4] == 0).all()


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
def test_padded_code_buffers_hold_the_same_codes(ops, dtype):
    """The training path keeps the codes in buffers whose rows are padded to whole K-blocks, i.e. rows that start on 16-byte
    boundaries whatever the column count: there the row codes of 16-bit inputs leave as 16-byte stores (a row's whole line in
    one instruction), also where a row ends after the first 8 codes of such a store.  Same codes and scales as unpadded."""
    from blockwise_int8_linear_amd import ops as _ops
    for (R, C, block) in [(300, 1000, 128), (1000, 72, 64), (64, 520, 128), (257, 136, 128), (128, 8, 64)]:
        x = outlier_tensor(R, C, DTYPES[dtype], seed=R + C).to(DEV)
        q, s, qt, st = ops.quantize_block_dual(x, block)
        qp, sp, qtp, stp, q_store, qt_store = _ops._quantize_block_dual(x, block, True)
        assert q_store.shape[1] % 16 == 0 and q_store.shape[1] >= C and q_store.data_ptr() % 16 == 0
        assert torch.equal(qp, q) and torch.equal(qtp, qt) and _same(sp, s) and _same(stp, st)
        assert (q_store[:, C:] == 0).all() and (qt_store[:, R:] == 0).all()          # the padding stays zero
