"""The int32 block partials of the kernels that produce the shipped outputs, recovered bit for bit.

bi8_gemm_nt_partials runs its own kernel instantiations; the kernels behind bi8_gemm_nt_dequant (gemm_wide, the
software-pipelined gemm_tile, gemm_panel, gemv_staged, gemm_skinny, the split of K) and bi8_linear_few_rows fold every partial
into an fp32 accumulator straight away and never store it.  Here each of them is made to hand a partial back through
its output: column scales all 1, row scales 1 for ONE K-block j and 0 for every other block, so that

    C[m,n] = fl( P_j[m,n] * fl32(1/127^2) )          (every other block adds exactly 0)

and P_j = round(C * 127^2) exactly: |P_j| <= 128 * 127^2 < 2^21 is an exact fp32 integer through the fold, and the
one or two roundings that follow move C * 127^2 by less than 0.26.  16-bit outputs keep 8 (bf16) or 11 (fp16)
significant bits, so those kernels are run on codes in {-1, 0, 1} (|P_j| <= 128, still exact after the cast); a
mis-routed 16-byte chunk of an operand changes such partials as surely as full-range ones.
Expected partials come from the CPU checker (the reference's tl.dot, triton_functions.py:115)."""
import pytest
import torch

from oracle import oracle_torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


@pytest.fixture(scope="module")
def ops():
    import blockwise_int8_linear_amd as pkg
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return pkg


class cfg_as:
    def __init__(self, ops, block, out):
        self.cfg, self.block, self.out = ops.block_linear_config, block, out

    def __enter__(self):
        self.old = (self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE)
        self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.block, self.out

    def __exit__(self, *a):
        self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.old


def _codes(g, rows, K, full_range):
    if full_range:
        c = torch.randint(-127, 128, (rows, K), generator=g, dtype=torch.int32)
        c[0] = 127                                  # saturated rows: the largest partial there is, +-128 * 127^2
        c[-1] = -127
    else:
        c = torch.randint(-1, 2, (rows, K), generator=g, dtype=torch.int32)
    return c.to(torch.int8)


def _blocks_to_check(nblk):
    return sorted(set(range(nblk)) if nblk <= 6 else {0, 1, nblk // 2, nblk - 2, nblk - 1})


def _kernel(ops, M, N, K, block, ws, lda=None):
    from blockwise_int8_linear_amd import _lib
    return _lib.load().bi8_gemm_kernel_name(M, N, K, lda or K, K, block, ws).decode()


def _device_codes(A, pitch):
    """A on the device, as a view of a buffer whose rows are `pitch` codes apart"""
    if pitch == A.shape[1]:
        return A.to(DEV)
    view = torch.empty((A.shape[0], pitch), device=DEV, dtype=torch.int8)[:, :A.shape[1]]
    view.copy_(A)
    return view


# (M, N, K, block, kernel the shipped operator runs on it)
CASES = [
    (2944, 2944, 512, 128, "gemm_wide"),            # 144 tiles of 256x256, four stages
    (2944, 2900, 384, 128, "gemm_wide"),            # odd number of stages (the loop runs a padding stage), ragged N
    (2944, 2944, 512, 64, "gemm_wide"),             # two K-blocks per stage
    (2900, 2944, 384, 64, "gemm_wide"),
    (5200, 5200, 384, 128, "gemm_wide"),            # 441 tiles: workgroups of the persistent grid walk on to a second tile
    (5200, 5100, 256, 64, "gemm_wide"),
    # 324 tiles = one full round and 68: the leading 14 rows of tiles on the 256x256 kernel, the other rows on 128x128 tiles
    (4400, 4500, 384, 128, "gemm_wide+gemm_tile_128x128"),
    (4500, 4400, 256, 64, "gemm_wide+gemm_wide_256x128"),          # ... on the same loop, 256x128 tiles from tile row 14 on
    (2048, 8900, 256, 128, "gemm_wide+gemm_tile_128x128"),         # cut by columns: 8 x 35 tiles, the last 3 columns of tiles apart
    (2000, 8900, 384, 64, "gemm_wide+gemm_tile_128x128"),
    (4352, 4096, 2048, 128, "gemm_wide+gemm_tile_64x128_splitk"),  # the rest (one row of 16 tiles) splits K
    (4353, 4096, 256, 128, "gemm_wide+gemm_tile_128x128"),         # the rest is 257 rows: its last tiles hold one row
    (4400, 4097, 384, 128, "gemm_wide+gemm_tile_128x128"),         # ... one column
    (4097, 4096, 256, 128, "gemm_wide+gemm_tile_64x128"),          # a rest of a single row still runs on tiles
    (4097, 4096, 2048, 64, "gemm_wide+gemm_tile_64x128_splitk"),
    (4300, 4096, 4096, 64, "gemm_wide+gemm_tile_128x128_splitk"),
    (2944, 2944, 256, 32, "gemm_wide"),             # block 32: the 32x32x32-MFMA form, four K-blocks per stage
    (2900, 2944, 384, 32, "gemm_wide"),
    (2048, 2304, 512, 128, "gemm_wide_256x128"),    # 256x128 tiles on the 256x256 kernel's loop, 64x64 per wave
    (2000, 2304, 384, 128, "gemm_wide_256x128"),    # odd number of stages, ragged M
    (2048, 4096, 512, 64, "gemm_wide_256x128"),
    (2048, 2304, 512, 64, "gemm_wide_256x128"),
    (8192, 768, 256, 64, "gemm_wide_256x128"),
    (8100, 760, 384, 64, "gemm_wide_256x128"),      # ragged M and N
    # rows of A 4 MiB apart put the operand beyond the 32-bit offsets of the 256x256 kernel's loop: the tile kernel's
    # software-pipelined block-128 instantiation, and its three-buffer form at block 64 (sixth entry: row pitch of A)
    (600, 11008, 256, 128, "gemm_tile_256x128", (1 << 22) - 128),
    (600, 11008, 256, 64, "gemm_tile_256x128", (1 << 22) - 128),
    (1500, 1500, 512, 32, "gemm_tile_128x128"),
    (1024, 3072, 640, 64, "gemm_tile_128x128"),     # block 64: more tiles of 128 x 64 than one round of gemm_panel's square form
    (300, 500, 512, 32, "gemm_tile_128x128"),
    # narrow tiles, the whole K in one workgroup: tiles of 128 rows x 16, 32, 48 or 64 columns, or -- where one round of them is at
    # most 64 columns wide -- of 64 rows x 16 ... 64 columns; one to many rows of tiles, one stage of K to thirty-two, odd and even
    # numbers of stages, ragged edges
    (300, 500, 512, 128, "gemm_panel"),             # 5 x 32 tiles of 64 x 16, the last row of tiles 44 rows, the last column 4
    (128, 4096, 1024, 128, "gemm_panel"),           # 2 x 128 tiles of 64 x 32
    (128, 64, 128, 128, "gemm_panel"),              # a single stage
    (100, 48, 256, 64, "gemm_panel"),
    (100, 8000, 640, 128, "gemm_panel"),            # 2 x 125 tiles of 64 x 64, five stages
    (200, 3000, 1152, 64, "gemm_panel"),            # 4 x 63 tiles of 64 x 48, two K-blocks per stage, nine stages
    (128, 11008, 384, 64, "gemm_panel"),            # 230 tiles of 128 x 48
    (65, 16000, 256, 128, "gemm_panel"),            # 250 tiles of 128 x 64
    (512, 4090, 4096, 128, "gemm_panel"),           # 4 x 64 tiles of 128 x 64, 32 stages
    (1000, 500, 384, 128, "gemm_panel"),            # 16 x 16 tiles of 64 x 32
    (30000, 16, 256, 128, "gemm_panel"),            # 235 x 1 tiles of 128 x 16: tall and one tile wide
    # ... and for 33 to 64 rows tiles of 64 rows, the waves as 4 x 2: 32, 64, 96 and 128 columns per tile
    (48, 5000, 640, 64, "gemm_panel"),              # 157 tiles of 32 columns, the last 8 columns wide
    (48, 700, 640, 64, "gemm_panel"),
    (64, 4096, 1024, 128, "gemm_panel"),            # 128 tiles of 32 columns
    (33, 64, 128, 128, "gemm_panel"),               # one stage, one tile of which the second wave column is empty
    (64, 11008, 4096, 128, "gemm_panel"),           # 230 tiles of 48 columns in the 64-column form, 32 stages
    (50, 24000, 256, 128, "gemm_panel"),            # 250 tiles of 96 columns
    (40, 24000, 384, 64, "gemm_panel"),             # ... two K-blocks per stage
    (64, 32000, 384, 128, "gemm_panel"),            # 250 tiles of 128 columns
    (60, 30000, 256, 128, "gemm_panel"),            # 235 tiles of 128 columns; (48, 20000): 250 of 80 in the 96-column form
    (48, 20000, 256, 128, "gemm_panel"),
    # ... and, up to 4096 columns, two rows of 32-row tiles
    (64, 4096, 2048, 128, "gemm_panel"),            # 2 x 128 tiles of 32 x 32
    (48, 3072, 4096, 64, "gemm_panel"),             # 2 x 96 tiles, the second row of tiles 16 rows, 32 stages
    (33, 3100, 640, 128, "gemm_panel"),             # 2 x 97 tiles, the second row of tiles a single row, the last column 28 wide
    # ... and for 3 to 32 rows against 5120 columns or more tiles of 32 rows, the waves as 2 x 4 (64, 128, 192 or 256 columns),
    # of which a tile takes as few 16-column subtiles as give one tile per CU
    (7, 8192, 2048, 128, "gemm_panel"),             # 256 tiles of 32 columns (the waves' last two columns and second row group empty)
    (12, 11008, 2048, 64, "gemm_panel"),            # 230 tiles of 48 columns
    (17, 8192, 2048, 128, "gemm_panel"),
    (29, 11008, 1024, 64, "gemm_panel"),
    (32, 6144, 4096, 128, "gemm_panel"),            # 192 tiles of 32 columns, 32 stages
    (5, 6150, 256, 128, "gemm_panel"),              # 193 tiles, the last 6 columns wide
    (16, 5120, 640, 128, "gemm_panel"),             # 160 tiles of 32 columns
    (24, 30000, 384, 128, "gemm_panel"),            # 235 tiles of 128 columns
    (20, 40000, 384, 64, "gemm_panel"),             # 250 tiles of 160 columns in the 192-column form, two K-blocks per stage
    (3, 50000, 128, 128, "gemm_panel"),             # 241 tiles of 208 columns in the 256-column form, one stage
    (2304, 2304, 256, 32, "gemm_tile_128x128"),
    (48, 5000, 640, 32, "gemm_tile_64x128"),
    (48, 700, 1280, 64, "gemv_staged"),             # four groups of 16 rows
    (64, 2048, 2048, 128, "gemv_staged"),
    (33, 1000, 2048 + 128, 128, "gemv_staged"),
    (1, 384, 512, 128, "gemv_rows"),
    (2, 1000, 4096 + 384, 128, "gemv_rows"),        # more than four runs of 1 KiB per row, the last one partial
    (2, 700, 2048 + 128, 64, "gemv_rows"),
    (1, 300, 8192 + 384, 128, "gemv_rows"),         # one row, K from 8192 on: six runs of every weight row in flight
    (1, 200, 9216, 64, "gemv_rows"),
    (3, 384, 512, 128, "gemv_staged"),
    (16, 1000, 4096, 128, "gemv_staged"),           # eight stages per wave
    (7, 1000, 1152, 64, "gemv_staged"),
    (7, 8192, 4224, 128, "gemv_staged"),            # more than 6144 columns: four waves per workgroup, several workgroups per CU
    (12, 11008, 4224, 64, "gemv_staged"),
    (24, 500, 640, 128, "gemv_staged"),             # two groups of 16 rows
    (32, 1000, 2048 + 128, 64, "gemv_staged"),
    (17, 8192, 4224, 128, "gemv_staged"),           # ... four waves per workgroup, two workgroups per CU
    (29, 11008, 4224, 64, "gemv_staged"),
    (24, 500, 640, 32, "gemm_skinny"),              # block 32, five stages of K: nothing to split
    (24, 500, 2048, 32, "gemm_tile_64x128_splitk"),
    (16, 300, 1024, 32, "gemm_skinny"),
    (128, 1024, 16384, 128, "gemm_tile_64x128_splitk"),
    # the square form (more than 128 rows): 4 x 2 waves of 32 x 64, tiles of 128 x 128, at block 64 (waves of 32 x 32) 128 x 64
    (1024, 4096, 1024, 128, "gemm_panel"),          # 256 tiles, eight stages
    (1500, 1500, 640, 128, "gemm_panel"),           # 144 tiles, ragged on both edges, five stages
    (300, 10000, 128, 128, "gemm_panel"),           # 3 x 79 tiles, one stage
    (512, 4000, 1152, 64, "gemm_panel"),            # 4 x 63 tiles of 128 x 64, two K-blocks per stage, nine stages
    (2000, 1000, 256, 64, "gemm_panel"),            # 16 x 16 tiles
    (512, 4096, 8192, 128, "gemm_panel_splitk"),    # 128 tiles, two pieces of 32 stages
    (1000, 1000, 8320, 64, "gemm_panel_splitk"),    # 8 x 16 tiles, two pieces of 33 and 32 stages
    # narrow tiles on pieces of K (65 to 128 rows, K from 4224 to 12288): 128 x 64 tiles, at block 64 128 x 32
    (128, 1024, 8192, 128, "gemm_panel_splitk"),    # 16 tiles, eight pieces of eight stages
    (65, 4100, 4224, 128, "gemm_panel_splitk"),     # 65 tiles (the last 4 columns wide), three pieces of 11 stages
    (100, 300, 5120, 64, "gemm_panel_splitk"),      # ten tiles of 32 columns, five pieces of eight stages, two K-blocks per stage
    # ... and for 17 to 64 rows against a long K: tiles of 32 x 64 or 64 x 64
    (32, 4096, 8192, 128, "gemm_panel_splitk"),     # 64 tiles, four pieces of 16 stages
    (17, 5000, 8320, 64, "gemm_panel_splitk"),      # 79 tiles (the last 8 columns wide), three pieces of 22, 22 and 21 stages
    (30, 8192, 10240, 128, "gemm_panel_splitk"),    # 128 tiles, two pieces of 40 stages
    (64, 2048, 11008, 128, "gemm_panel_splitk"),    # 32 tiles of 64 x 64, eight pieces of 11 stages
    (33, 2000, 5120, 64, "gemm_panel_splitk"),      # 32 tiles (the last 16 columns wide), five pieces of eight stages
    (256, 2048, 8192, 64, "gemm_tile_128x128_splitk"),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c[:4])) + "-" + c[4])
@pytest.mark.parametrize("out", ["f32", "bf16"])
def test_partials_of_the_shipping_kernels(ops, case, out):
    from blockwise_int8_linear_amd import _lib
    M, N, K, block, kernel = case[:5]
    lda = case[5] if len(case) > 5 else K
    ws = _lib.load().bi8_gemm_workspace_bytes(M, N, K, block)          # what the operator asks for and passes
    assert _kernel(ops, M, N, K, block, ws, lda) == kernel
    g = torch.Generator().manual_seed(M + 3 * N + K + block)
    full = out == "f32"
    A, W = _codes(g, M, K, full), _codes(g, N, K, full)
    nblk = K // block
    P_ref = oracle_torch.gemm_nt_partials(A, W, block)                  # int32 [nblk, M, N]
    Ad, Wd = _device_codes(A, lda), W.to(DEV)
    sw = torch.ones(nblk, N, device=DEV)
    with cfg_as(ops, block, DT[out]):
        for j in _blocks_to_check(nblk):
            sa = torch.zeros(nblk, M, device=DEV)
            sa[j] = 1.0
            C = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), sa, sw)
            assert C.dtype == DT[out]
            got = torch.round(C.double() * (127.0 * 127.0)).to(torch.int32)
            want = P_ref[j].to(DEV)
            if not torch.equal(got, want):
                bad = (got != want).nonzero()
                m, n = bad[0].tolist()
                raise AssertionError(f"{kernel}: K-block {j}: {bad.shape[0]} partials differ, first at ({m},{n}): "
                                     f"got {got[m, n].item()} want {want[m, n].item()}")
        if full and "splitk" not in kernel:
            # every scale 1: where the running sums of the partials stay below 2^24 (everywhere but the saturated rows
            # and columns of a long K) the accumulator holds their exact integer sum, and the output is that sum
            # times fl32(1/127^2), rounded once
            exact = P_ref.long().abs().sum(0) < (1 << 24)
            assert exact.float().mean() > 0.9
            C = ops.int8_matmul_block64_rowwise_dequantize(Ad, Wd.t(), torch.ones(nblk, M, device=DEV), sw)
            want = P_ref.sum(0).float() * torch.tensor(1.0 / (127.0 * 127.0), dtype=torch.float32)
            assert torch.equal(C.cpu()[exact], want[exact])


@pytest.mark.parametrize("case", CASES[:2] + CASES[4:7], ids=lambda c: "x".join(map(str, c[:4])) + "-" + c[4])
def test_partials_of_the_f16_instantiations(ops, case):
    M, N, K, block, kernel = case[:5]
    g = torch.Generator().manual_seed(K + block)
    A, W = _codes(g, M, K, False), _codes(g, N, K, False)
    nblk = K // block
    P_ref = oracle_torch.gemm_nt_partials(A, W, block)
    sw = torch.ones(nblk, N, device=DEV)
    with cfg_as(ops, block, torch.float16):
        j = nblk - 1
        sa = torch.zeros(nblk, M, device=DEV)
        sa[j] = 1.0
        C = ops.int8_matmul_block64_rowwise_dequantize(A.to(DEV), W.to(DEV).t(), sa, sw)
        assert torch.equal(torch.round(C.double() * (127.0 * 127.0)).to(torch.int32).cpu(), P_ref[j])


@pytest.mark.parametrize("block", [64, 128])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("M", [1, 2])
def test_partials_of_the_one_launch_decode_linear(ops, block, dtype, M):
    """bi8_linear_few_rows quantizes x itself, so x is built to quantize to known codes: integers in one K-block j
    with a +-127 among them (scale 127, codes = the integers), zeros elsewhere (scale 0, codes 0).  Then
    C = fl(fl(127 * P_j) * fl32(1/127^2)) with column scales 1."""
    N, K = 700, 2048
    nblk = K // block
    g = torch.Generator().manual_seed(block + M)
    full = dtype == "f32"
    W = _codes(g, N, K, False)                                          # |127 * P_j| stays below 2^24
    for j in _blocks_to_check(nblk)[:4]:
        codes = torch.zeros(M, K, dtype=torch.int32)
        if full:
            codes[:, j * block:(j + 1) * block] = torch.randint(-127, 128, (M, block), generator=g, dtype=torch.int32)
        else:
            codes[:, j * block:j * block + 48] = torch.randint(-1, 2, (M, 48), generator=g, dtype=torch.int32)
        codes[:, j * block + 5] = 127
        x = codes.to(DT[dtype])
        assert torch.equal(x.to(torch.int32), codes)
        P_ref = oracle_torch.gemm_nt_partials(codes.to(torch.int8), W, block)[j]
        if not full:
            assert P_ref.abs().max() < 256
        with cfg_as(ops, block, DT[dtype]):
            C = ops.linear_few_rows(x.to(DEV), W.to(DEV), torch.ones(nblk, N, device=DEV))
            assert C is not None, "the fused kernel covers this case"
            # the same through the two launches: identical bits
            xq, sx = ops.quantize_block_rowwise(x.to(DEV))
            assert torch.equal(xq.cpu().to(torch.int32), codes) and (sx[j] == 127).all() and sx.sum() == 127 * M
            C2 = ops.int8_matmul_block64_rowwise_dequantize(xq, W.to(DEV).t(), sx, torch.ones(nblk, N, device=DEV))
        assert torch.equal(C, C2)
        got = torch.round(C.double() * (127.0 * 127.0) / 127.0).to(torch.int32).cpu()
        assert torch.equal(got, P_ref)
