"""bi8_gemm_nt_dequant_static -- the entry point that allocates nothing: the split of K writes its fp32 slabs to a
static array in device memory that the library owns.  Called here straight through the C ABI and compared bit for bit
with bi8_gemm_nt_dequant_ws (caller-provided workspace) on the same operands: two calls in a row, the second on a
smaller problem (the array still holds the first call's slabs), then a problem that does not split at all, and the
first one again; one case passes operands whose rows are longer than K (leading dimensions above K).  Outputs of the
existing entry point are themselves checked against the CPU checker.  "Allocates nothing" is checked on the device's
own count of free memory (hipMemGetInfo), which a hipMalloc inside the library would move, and on torch's allocator."""

import pytest
import torch

from util import gemm_reference

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _problem(M, N, K, block, seed):
    g = torch.Generator().manual_seed(seed)
    A = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    W = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    sa = torch.rand(K // block, M, generator=g) * 4 + 0.01
    sw = torch.rand(K // block, N, generator=g) * 0.1 + 1e-4
    bias = torch.randn(N, generator=g)
    return A, W, sa, sw, bias


def test_static_scratch_entry_point_matches_the_workspace_entry_point():
    from blockwise_int8_linear_amd import _lib
    lib = _lib.load()
    torch.cuda.set_device(0)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.bi8_static_scratch_bytes() == 32 << 20
    # (M, N, K, block, out dtype code, splits?, extra row length of A and W)  larger problem first, then a smaller one, one
    # with padded rows, one without a split, the first again
    cases = [(3072, 768, 8192, 64, 1, True, 0), (128, 1024, 8192, 128, 0, True, 0), (96, 256, 8192, 128, 1, True, 0),
             (128, 512, 8192, 128, 1, True, 256), (300, 500, 512, 128, 0, False, 0), (3072, 768, 8192, 64, 1, True, 0)]
    dts = {0: torch.float32, 1: torch.bfloat16}
    torch.cuda.synchronize()
    for i, (M, N, K, block, cdt, splits, pad) in enumerate(cases):
        A, W, sa, sw, bias = _problem(M, N, K, block, 100 + i)
        sad, swd, bd = (t.to(DEV) for t in (sa, sw, bias))
        # operands as views of buffers with rows of K + pad codes (the padding holds codes that must not be read)
        Ad = torch.full((M, K + pad), 77, device=DEV, dtype=torch.int8)[:, :K]
        Wd = torch.full((N, K + pad), -77, device=DEV, dtype=torch.int8)[:, :K]
        Ad.copy_(A)
        Wd.copy_(W)
        need = lib.bi8_gemm_workspace_bytes(M, N, K, block)
        assert (need > 0) == splits and need <= lib.bi8_static_scratch_bytes()
        ws = torch.empty(max(need, 16), device=DEV, dtype=torch.uint8)
        c_ws = torch.empty(M, N, device=DEV, dtype=dts[cdt])
        c_st = torch.full((M, N), float("nan"), device=DEV, dtype=dts[cdt])
        args = (Ad.data_ptr(), Wd.data_ptr(), sad.data_ptr(), swd.data_ptr(), bd.data_ptr(), 0)
        dims = (M, N, K, K + pad, K + pad, N, block)
        assert lib.bi8_gemm_nt_dequant_ws(*args, c_ws.data_ptr(), cdt, *dims, ws.data_ptr(), need, st) == 0
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        assert lib.bi8_gemm_nt_dequant_static(*args, c_st.data_ptr(), cdt, *dims, st) == 0
        torch.cuda.synchronize()
        # (the first call on a device makes the runtime look up the array's address; the array itself is part of the
        # loaded code object, so not even that call takes device memory)
        assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(c_st, c_ws), f"case {i}: static-scratch output differs from the workspace output"
        # and against the CPU checker; the bias is added to the rounded product in the output type, so the relative
        # bound counts the magnitudes of both, and where the products differ the rounding of the sum can add one more
        # unit in the last place of the output type
        ref, mag = gemm_reference(A, W, sa, sw, block, None, dts[cdt])
        tol, ulp = (1e-3, 2.0 ** -23) if cdt == 0 else (1e-2, 2.0 ** -7)
        full = (ref + bias.to(dts[cdt])).double()
        bound = tol * (ref.double().abs() + 2 * bias.double().abs()) + ulp * full.abs() + 4e-6 * mag
        err = (c_st.cpu().double() - full).abs()
        assert (err <= bound).all(), f"case {i}: {(err > bound).sum().item()} elements off, worst {(err - bound).max().item():.3e} over its bound"
    # bad arguments are refused before anything is looked up or launched
    assert lib.bi8_gemm_nt_dequant_static(None, None, None, None, None, 0, None, 0, 4, 4, 128, 64, 128, 4, 128, None) == 4
    assert b"scratch" in lib.bi8_strerror(7)
