"""bi8_gemm_nt_dequant_ws on seeded random shapes in the ranges where the dispatch rule changes kernel or tile form (few
rows against many columns, 33 to 128 rows, tall and narrow, more than 128 rows with at most one round of 128x128 tiles, a
long K), with and without scratch memory, bias or not, all three output types.

Every case is checked twice: sampled rows (the first, the last, random ones: every row of tiles of the tall cases is
likely hit, every column is) against the CPU checker to the GEMM tolerance, and the WHOLE output against a float64
product of the same codes and scales computed by torch on the device, so that a tile that is skipped, written twice or
written to the wrong place shows wherever it lies.  Rows in front of and behind C hold a marker that must survive."""
import random

import pytest
import torch

from util import DTYPES, gemm_reference, assert_gemm_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"f32": 1e-3, "bf16": 1e-2, "f16": 1e-2}


def _cases():
    rnd = random.Random(20240607)
    out = []
    while len(out) < 48:
        cls = ("few", "few", "mid", "mid", "tall", "square", "square", "longk")[len(out) % 8]
        block = rnd.choice([64, 128, 128])
        if cls == "few":
            M, N, K = rnd.randint(3, 32), rnd.randint(4000, 40000), 128 * rnd.randint(1, 32)
        elif cls == "mid":
            M, N, K = rnd.randint(33, 128), rnd.randint(16, 16000), 128 * rnd.randint(1, 40)
        elif cls == "tall":
            M, N, K = rnd.randint(129, 3000), rnd.randint(16, 3000), 128 * rnd.randint(1, 32)
        elif cls == "square":
            M, N, K = rnd.randint(129, 2048), rnd.randint(1000, 12000), 128 * rnd.randint(1, 36)
        else:
            M, N, K = rnd.randint(3, 700), rnd.randint(16, 6000), 128 * rnd.randint(33, 100)
        if M * N > 12e6 or M * N * K > 1.5e11 or N * K > 1.2e8:
            continue
        out.append((M, N, K, block, rnd.choice(["f32", "f32", "bf16", "f16"]), rnd.random() < 0.5, rnd.random() < 0.6))
    return out


@pytest.mark.parametrize("case", _cases(), ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}-b{c[3]}-{c[4]}{'-bias' if c[5] else ''}{'-ws' if c[6] else ''}")
def test_random_shape(case):
    from blockwise_int8_linear_amd import _lib
    lib = _lib.load()
    M, N, K, block, out, with_bias, with_ws = case
    g = torch.Generator().manual_seed(M * 7 + N + K)
    A = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    W = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    sa = torch.rand(K // block, M, generator=g) * 3 + 0.01
    sw = torch.rand(K // block, N, generator=g) * 0.1 + 1e-4
    bias = torch.randn(N, generator=g).to(DTYPES[out]) if with_bias else None
    need = lib.bi8_gemm_workspace_bytes(M, N, K, block) if with_ws else 0
    kernel = lib.bi8_gemm_kernel_name(M, N, K, K, K, block, need).decode()
    Ad, Wd, sad, swd = A.to(DEV), W.to(DEV), sa.to(DEV), sw.to(DEV)
    bd = bias.to(DEV) if with_bias else None
    ws = torch.empty(max(need, 16), device=DEV, dtype=torch.uint8)
    guard = 4
    dt = {"f32": 0, "bf16": 1, "f16": 2}[out]

    def run(b):
        cbuf = torch.full((M + 2 * guard, N), 777.0, device=DEV, dtype=DTYPES[out])
        c = cbuf[guard:guard + M]
        rc = lib.bi8_gemm_nt_dequant_ws(Ad.data_ptr(), Wd.data_ptr(), sad.data_ptr(), swd.data_ptr(), b.data_ptr() if b is not None else None, dt,
                                        c.data_ptr(), dt, M, N, K, K, K, N, block, ws.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, kernel
        torch.cuda.synchronize()
        assert (cbuf[:guard] == 777.0).all() and (cbuf[guard + M:] == 777.0).all(), kernel
        return c
    C = run(None)
    if with_bias:
        # the bias is added after the cast, in the output type (triton_functions.py:127-131): exactly this identity
        assert torch.equal(run(bd), C + bd), kernel

    # sampled rows against the CPU checker
    rg = random.Random(M + N)
    rows = sorted({0, M - 1} | {rg.randrange(M) for _ in range(min(M, 14))})
    rows_t = torch.tensor(rows)
    ref, mag = gemm_reference(A[rows_t], W, sa[:, rows_t].contiguous(), sw, block, None, DTYPES[out])
    try:
        assert_gemm_close(C[rows_t.to(DEV)].cpu(), ref, mag, TOL[out])
    except AssertionError as e:
        raise AssertionError(f"{kernel}: {e}")

    # the whole output against a float64 product on the device
    full = torch.zeros(M, N, device=DEV, dtype=torch.float64)
    for j in range(K // block):
        p = Ad[:, j * block:(j + 1) * block].double() @ Wd[:, j * block:(j + 1) * block].double().t()
        full += p * sad[j].double()[:, None] * swd[j].double()[None, :]
    full = (full / (127.0 * 127.0)).to(DTYPES[out])
    err = (C.double() - full.double()).abs()
    scale = full.double().abs().max().item()
    unit = {"f32": 2e-6, "bf16": 8e-3, "f16": 1e-3}[out]         # one rounding of the output type at the largest magnitude, and the summation order
    assert not torch.isnan(C).any() and err.max().item() <= unit * scale, f"{kernel}: {err.max().item():.3e} of {scale:.3e}"


@pytest.mark.parametrize("M,N,K,block", [(16, 11008, 4096, 128), (32, 6144, 2048, 64), (64, 4096, 4096, 128), (128, 4096, 4096, 128),
                                         (300, 500, 512, 128), (1024, 4096, 2048, 128), (512, 4096, 1152, 64),
                                         (32, 4096, 11008, 128), (64, 2048, 8192, 128), (128, 4096, 11008, 128), (512, 4096, 8192, 128)])
def test_narrow_tile_kernels_call_after_call(M, N, K, block):
    """gemm_panel's forms (tiles of 32, 64 and 128 rows, the square form, the pieces of K) stream their operands through rings of
    LDS buffers filled by waves of their own, with hand-counted waits: a buffer reused too early would show now and then, not
    always.  Fresh operands three times, twelve calls each with other work on the GPU in between: every call gives the bits of
    the first (the kernels are deterministic), and the first matches a float64 product on the device."""
    from blockwise_int8_linear_amd import _lib
    lib = _lib.load()
    need = lib.bi8_gemm_workspace_bytes(M, N, K, block)
    kernel = lib.bi8_gemm_kernel_name(M, N, K, K, K, block, need).decode()
    assert kernel in ("gemm_panel", "gemm_panel_splitk")
    ws = torch.empty(max(need, 16), device=DEV, dtype=torch.uint8)
    st = torch.cuda.current_stream().cuda_stream
    for ds in range(3):
        g = torch.Generator(device=DEV).manual_seed(1000 * ds + M)
        A = torch.randint(-127, 128, (M, K), device=DEV, dtype=torch.int8, generator=g)
        W = torch.randint(-127, 128, (N, K), device=DEV, dtype=torch.int8, generator=g)
        sa = torch.rand(K // block, M, device=DEV, generator=g) + 0.5
        sw = torch.rand(K // block, N, device=DEV, generator=g) * 0.02
        first = None
        for rep in range(12):
            C = torch.full((M, N), float("nan"), device=DEV, dtype=torch.float32)
            rc = lib.bi8_gemm_nt_dequant_ws(A.data_ptr(), W.data_ptr(), sa.data_ptr(), sw.data_ptr(), None, 0, C.data_ptr(), 0,
                                            M, N, K, K, K, N, block, ws.data_ptr(), need, st)
            assert rc == 0, kernel
            if rep % 4 == 0:
                _ = (W[:64].float() @ W[:64].float().t()).sum()
            if first is None:
                first = C
            else:
                assert torch.equal(C, first), f"{kernel}: call {rep} of data set {ds} differs from the first"
        full = torch.zeros(M, N, device=DEV, dtype=torch.float64)
        for j in range(K // block):
            p = A[:, j * block:(j + 1) * block].double() @ W[:, j * block:(j + 1) * block].double().t()
            full += p * sa[j].double()[:, None] * sw[j].double()[None, :]
        full /= 127.0 * 127.0
        assert (first.double() - full).abs().max().item() <= 3e-6 * full.abs().max().item(), kernel
