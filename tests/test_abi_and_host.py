"""CPU-side checks of the boundary: libbi8.so loads and exports exactly what include/bi8.h declares, the
ctypes signatures agree with the header, argument validation answers before any launch, and the Python
layer keeps the reference's names, defaults and error behaviour.  No kernel is launched here."""
import ctypes
import inspect
import os
import re
import subprocess

import pytest
import torch
import torch.nn as nn

import blockwise_int8_linear_amd as pkg
from blockwise_int8_linear_amd import _lib, block_linear_config, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_decls():
    text = open(os.path.join(ROOT, "include", "bi8.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"(?:int64_t|int|const char \*)\s*(bi8_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = [a.strip() for a in m.group(2).split(",")] if m.group(2).strip() != "void" else []
        decls[m.group(1)] = args
    return decls


def test_library_exports_every_declared_symbol():
    decls = _header_decls()
    assert set(decls) == {"bi8_version", "bi8_strerror", "bi8_quantize_rowwise", "bi8_quantize_transposed",
                          "bi8_dequantize_rowwise", "bi8_gemm_nt_dequant", "bi8_gemm_nt_partials",
                          "bi8_linear_few_rows", "bi8_quantize_dual", "bi8_gemm_nt_dequant_ws",
                          "bi8_gemm_workspace_bytes", "bi8_gemm_kernel_name", "bi8_static_scratch_bytes",
                          "bi8_gemm_nt_dequant_static", "bi8_colsum_workspace_bytes", "bi8_quantize_dual_colsum"}
    lib = _lib.load()
    for name in decls:
        assert hasattr(lib, name), f"{name} not exported"
    # and nothing else with the library's prefix leaks out
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l and l.split()[-1].startswith("bi8_")}
    assert exported == set(decls)


def test_ctypes_signatures_match_header():
    decls = _header_decls()
    assert set(decls) == set(_lib.SIGNATURES)
    for name, args in decls.items():
        res, argtypes = _lib.SIGNATURES[name]
        assert len(args) == len(argtypes), name
        for a, t in zip(args, argtypes):
            if "*" in a:
                assert t is ctypes.c_void_p, (name, a)
            elif a.startswith("int64_t"):
                assert t is ctypes.c_int64, (name, a)
            else:
                assert a.startswith("int ") and t is ctypes.c_int, (name, a)


def test_version_and_error_strings():
    lib = _lib.load()
    assert lib.bi8_version() == _lib.ABI_VERSION == 5
    assert lib.bi8_strerror(0) == b"success"
    assert b"block" in lib.bi8_strerror(3)
    with pytest.raises(_lib.Bi8Error, match="leading dimension"):
        _lib.check(4, "x")


def test_argument_validation_happens_before_any_launch():
    """bad arguments are rejected on the host; none of these calls reaches the GPU runtime"""
    lib = _lib.load()
    p = ctypes.c_void_p(0x1000)
    assert lib.bi8_quantize_rowwise(p, 7, p, p, 4, 128, 128, 128, 128, None) == 2          # dtype
    assert lib.bi8_quantize_rowwise(p, 1, p, p, 4, 128, 128, 128, 0, None) == 3            # block
    assert lib.bi8_quantize_rowwise(p, 1, p, p, 4, 128, 64, 128, 128, None) == 4           # ldx < K
    assert lib.bi8_quantize_rowwise(p, 1, p, p, -1, 128, 128, 128, 128, None) == 4
    assert lib.bi8_quantize_rowwise(None, 1, p, p, 4, 128, 128, 128, 128, None) == 1       # null
    assert lib.bi8_quantize_rowwise(None, 1, None, None, 0, 128, 128, 128, 128, None) == 0  # empty: nothing to do
    assert lib.bi8_quantize_transposed(p, 1, p, p, 4, 128, 128, 2, 128, None) == 4         # ldq < R
    assert lib.bi8_dequantize_rowwise(p, p, p, 3, 4, 128, 128, 128, 128, None) == 2
    assert lib.bi8_gemm_nt_dequant(p, p, p, p, None, 0, p, 1, 4, 4, 128, 64, 128, 4, 128, None) == 4
    assert lib.bi8_gemm_nt_dequant(p, p, p, p, p, 9, p, 1, 4, 4, 128, 128, 128, 4, 128, None) == 2
    assert lib.bi8_gemm_nt_dequant(None, None, None, None, None, 0, None, 1, 0, 4, 128, 128, 128, 4, 128, None) == 0
    assert lib.bi8_gemm_nt_partials(p, p, None, 4, 4, 128, 128, 128, 128, None) == 1
    assert lib.bi8_quantize_dual(p, 1, p, p, p, p, 4, 128, 128, 128, 2, 128, None) == 4           # ldqt < R
    assert lib.bi8_quantize_dual(p, 1, p, p, None, p, 4, 128, 128, 128, 4, 128, None) == 1        # null qT
    # x, dtype, W, sW, bias, bias_dtype, C, M, N, K, ldx, ldw, ldc, block, stream
    assert lib.bi8_linear_few_rows(p, 1, p, p, None, 0, p, 1, 64, 256, 128, 256, 64, 128, None) == 4    # ldx < K
    assert lib.bi8_linear_few_rows(p, 1, p, None, None, 0, p, 1, 64, 256, 256, 256, 64, 128, None) == 1  # null scales
    assert lib.bi8_linear_few_rows(p, 1, p, p, None, 0, p, 5, 64, 256, 256, 256, 64, 128, None) == 6    # five rows
    assert lib.bi8_linear_few_rows(p, 1, p, p, None, 0, p, 1, 64, 256, 256, 256, 64, 32, None) == 6     # block 32
    assert lib.bi8_linear_few_rows(p, 1, p, p, None, 0, p, 1, 64, 192, 192, 192, 64, 64, None) == 6     # K % 128
    assert lib.bi8_linear_few_rows(p, 1, p, p, None, 0, p, 4, 64, 32768, 32768, 32768, 64, 128, None) == 6  # LDS budget
    assert b"covers" in lib.bi8_strerror(6)


def test_python_api_mirrors_reference_names_and_defaults():
    # triton_functions.py:221, :492, :142 and block_linear.py:16, :69, :114
    assert list(inspect.signature(ops.quantize_block_rowwise).parameters) == ["x", "fblock_size"]
    assert list(inspect.signature(ops.dequantize_block_rowwise).parameters) == ["x", "state_x", "fblock_size"]
    assert list(inspect.signature(ops.int8_matmul_block64_rowwise_dequantize).parameters) == ["a", "b", "state_x", "state_w", "bias"]
    assert inspect.signature(ops.int8_matmul_block64_rowwise_dequantize).parameters["bias"].default is None
    # the reference's positional parameters, then one keyword-only addition
    sig = inspect.signature(pkg.BlockInt8Linear.__init__).parameters
    assert list(sig) == ["self", "in_features", "out_features", "bias", "device", "dtype", "quantized_weight_training"]
    assert sig["quantized_weight_training"].kind is inspect.Parameter.KEYWORD_ONLY and sig["quantized_weight_training"].default is False
    for name in ("prepare_for_eval", "infer", "forward", "weight_quant_training"):
        assert callable(getattr(pkg.BlockInt8Linear, name))
    assert issubclass(pkg.BlockInt8Linear, nn.Linear) and issubclass(pkg.blockwise_int8_linear, torch.autograd.Function)
    # block_linear_config.py:3-5
    assert block_linear_config.GROUP_SIZE == 128
    assert block_linear_config.SHARED_EXP_TORCH_TYPE == torch.float32
    assert block_linear_config.INPUT_OUTPUT_TORCH_TYPE == torch.bfloat16


def test_cpu_tensors_are_rejected_like_the_reference():
    x = torch.zeros(4, 128)
    with pytest.raises(AssertionError):                     # `assert x.is_cuda`, triton_functions.py:229
        ops.quantize_block_rowwise(x)
    with pytest.raises(AssertionError):                     # :496
        ops.dequantize_block_rowwise(torch.zeros(4, 128, dtype=torch.int8), torch.zeros(1, 4))
    with pytest.raises(AssertionError):
        ops.int8_matmul_block64_rowwise_dequantize(torch.zeros(4, 128, dtype=torch.int8), torch.zeros(128, 4, dtype=torch.int8),
                                                   torch.zeros(1, 4), torch.zeros(1, 4))
    lin = pkg.BlockInt8Linear(128, 4)
    with pytest.raises(AssertionError):                     # no silent CPU fallback in the module either
        lin(x)


def test_model_surgery_on_cpu_modules():
    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.a = nn.Linear(8, 16)
            self.seq = nn.Sequential(nn.Linear(16, 16), nn.ReLU())

    net = Net().eval()
    w = net.a.weight.data_ptr()
    pkg.replace_linear_with_blockwise_int8(net)
    assert isinstance(net.a, pkg.BlockInt8Linear) and net.a.weight.data_ptr() == w and not net.a.training
    assert type(net.seq[0]) is nn.Linear
    assert set(net.a.state_dict()) == {"weight", "bias"}
    net.apply(pkg.replace_linear_with_blockwise_int8)
    assert isinstance(net.seq[0], pkg.BlockInt8Linear)
    # the helper that recurses by itself: every level, same storage, training flags kept
    net2 = nn.Sequential(nn.Linear(8, 8), nn.Sequential(nn.Linear(8, 8), nn.ReLU(), nn.Sequential(nn.Linear(8, 4, bias=False))))
    ptrs = [p.data_ptr() for p in net2.parameters()]
    assert pkg.replace_linear_with_blockwise_int8_recursive(net2) is net2
    lins = [m for m in net2.modules() if isinstance(m, nn.Linear)]
    assert len(lins) == 3 and all(isinstance(m, pkg.BlockInt8Linear) and m.training for m in lins)
    assert [p.data_ptr() for p in net2.parameters()] == ptrs and lins[2].bias is None
    assert not lins[0].quantized_weight_training
    # the state that the cached int8 weights are keyed on moves with in-place updates, with any optimizer step of the
    # process (optimizers that write through .data bump no version) and with an explicit invalidation
    lin = pkg.BlockInt8Linear(8, 4, quantized_weight_training=True)
    assert lin.quantized_weight_training
    seen = {lin._weight_state()}
    with torch.no_grad():
        lin.weight.mul_(2.0)
    seen.add(lin._weight_state())
    lin.weight.data.mul_(2.0)                                   # invisible ...
    assert lin._weight_state() in seen
    torch.optim.SGD([nn.Parameter(torch.zeros(1))], lr=0.1).step()         # ... unless an optimizer step went by
    seen.add(lin._weight_state())
    lin.invalidate_quantized_weight()
    seen.add(lin._weight_state())
    assert len(seen) == 4


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libbi8.so"))
    with pytest.raises(_lib.Bi8Error, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_recip_division_is_exact():
    """the quantizer's reciprocal-multiply division, restated in C with fmaf(): exhaustive over all pairs of
    16-bit inputs (one correction); for binary32 (two corrections) random pairs, pairs next to the ties of the code and
    directed hard-to-round pairs (quotients within 2^-48 of a rounding boundary) -- see tests/c/recip_division_check.c"""
    src = os.path.join(ROOT, "tests", "c", "recip_division_check.c")
    exe = "/tmp/bi8_recip_division_check"
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-fopenmp", src, "-o", exe, "-lm"], check=True)
    res = subprocess.run([exe, "50000000"], capture_output=True, text=True)
    assert res.returncode == 0, res.stdout
    assert res.stdout.count(" 0 mismatches") == 4, res.stdout


def test_reference_module_names_can_be_aliased():
    """code written against the reference's flat layout: `import block_linear_config`, `from triton_functions import ...`,
    `from block_linear import BlockInt8Linear` (block_linear.py:8-12) resolve to this package after compat.install()"""
    import importlib
    import sys

    import blockwise_int8_linear_amd as pkg
    from blockwise_int8_linear_amd import compat
    for name in ("block_linear_config", "triton_functions", "block_linear"):
        assert name not in sys.modules
    compat.install()
    try:
        cfg = importlib.import_module("block_linear_config")
        tf = importlib.import_module("triton_functions")
        bl = importlib.import_module("block_linear")
        assert cfg is pkg.block_linear_config
        assert tf.quantize_block_rowwise is pkg.quantize_block_rowwise
        assert tf.int8_matmul_block64_rowwise_dequantize is pkg.int8_matmul_block64_rowwise_dequantize
        assert tf.dequantize_block_rowwise is pkg.dequantize_block_rowwise and tf.ceil_div(7, 2) == 4
        assert bl.BlockInt8Linear is pkg.BlockInt8Linear and bl.replace_linear_with_blockwise_int8 is pkg.replace_linear_with_blockwise_int8
        old = cfg.GROUP_SIZE
        cfg.GROUP_SIZE = 64                      # one config object under both names
        assert pkg.block_linear_config.GROUP_SIZE == 64
        cfg.GROUP_SIZE = old
        compat.install()                         # idempotent
    finally:
        compat.uninstall()
    assert "triton_functions" not in sys.modules
    sys.modules["triton_functions"] = sys                      # somebody else's module of that name is not shadowed silently
    try:
        with pytest.raises(RuntimeError, match="already imported"):
            compat.install()
    finally:
        del sys.modules["triton_functions"]


def test_kernel_choice_by_shape():
    """the dispatch rule is host arithmetic: which kernel family runs which problem (no GPU call)"""
    lib = _lib.load()
    name = lambda M, N, K, block, ws=0, lda=None, ldw=None: lib.bi8_gemm_kernel_name(M, N, K, lda or K, ldw or K, block, ws).decode()
    assert name(8192, 8192, 8192, 128) == "gemm_wide" and name(8192, 8192, 8192, 64) == "gemm_wide"
    assert name(8192, 8192, 8192, 32) == "gemm_wide"                 # (the 32x32x32-MFMA form of the 256x256 kernel)
    assert name(2048, 4096, 4096, 32) == "gemm_tile_128x128"         # block 32 has no 256x128 tile
    assert name(2944, 2944, 512, 128) == "gemm_wide"                 # 12 x 12 = 144 tiles of 256x256
    # a last round of 256x256 tiles that is mostly empty: whole rows (columns) of tiles cut off for a second launch
    assert name(1536, 11008, 4096, 128) == "gemm_wide+gemm_tile_128x128" and name(2048, 11008, 4096, 128) == "gemm_wide+gemm_wide_256x128"
    assert name(1536, 11008, 4096, 128, 1 << 30) == "gemm_wide+gemm_tile_64x128_splitk"
    assert name(2048, 12288, 4096, 128) == "gemm_wide" and name(1280, 11008, 4096, 128) == "gemm_wide"   # half a round left / one round
    # more than 256 tiles of 128x128 that do not fill the chip with 256x256 tiles: the 256x256 kernel's loop on 256x128 tiles
    assert name(8192, 768, 3072, 64) == "gemm_wide_256x128" and name(8192, 768, 3072, 128) == "gemm_wide_256x128"
    assert name(2048, 4096, 4096, 128) == "gemm_wide_256x128"        # 128 tiles of 256x256: one round of 256x128 tiles
    assert name(2048, 4096, 512, 64) == "gemm_wide_256x128" and name(2048, 2304, 512, 64) == "gemm_wide_256x128"
    assert name(2048, 4096, 4096, 128, 0, 1 << 21, 4096) == "gemm_tile_256x128"     # rows 2 MiB apart: beyond its 32-bit offsets
    assert name(1500, 1500, 512, 32) == "gemm_tile_128x128" and name(48, 5000, 640, 32) == "gemm_tile_64x128"
    assert name(1024, 3072, 4096, 64) == "gemm_tile_128x128"         # block 64: 384 tiles of 128 x 64 are more than one round of the square form
    # more than 128 rows, more narrow tiles than one round, at most 256 tiles of 128 x 128 (block 64: 128 x 64): gemm_panel's square form
    assert name(1024, 4096, 4096, 128) == "gemm_panel" and name(256, 11008, 4096, 128, 1 << 30) == "gemm_panel" and name(1024, 4096, 16384, 128, 1 << 30) == "gemm_panel"
    assert name(512, 4096, 4096, 64, 1 << 30) == "gemm_panel" and name(1024, 2048, 3072, 64) == "gemm_panel" and name(2048, 1024, 768, 64) == "gemm_panel"
    assert name(1500, 1500, 512, 128) == "gemm_panel" and name(1500, 1500, 16384, 128) == "gemm_panel"     # 144 tiles: where nothing splits K
    assert name(1500, 1500, 16384, 128, 1 << 30) == "gemm_wide_256x128_splitk" and name(1500, 1500, 16384, 32, 1 << 30) == "gemm_tile_128x128_splitk"
    # ... and on two pieces of K for 100 to 128 such tiles and K from 8192 on
    assert name(512, 4096, 11008, 128, 1 << 30) == "gemm_panel_splitk" and name(1024, 2048, 8192, 128, 1 << 30) == "gemm_panel_splitk"
    assert name(1024, 1024, 8192, 64, 1 << 30) == "gemm_panel_splitk" and name(512, 4096, 8064, 128, 1 << 30) == "gemm_wide_256x128_splitk"
    assert name(512, 3072, 11008, 128, 1 << 30) == "gemm_wide_256x128_splitk"      # 96 tiles
    # more than 64 rows, at most one tile of 128 x (16 ... 64) per CU and K up to 4096: narrow tiles, the whole K in one workgroup
    assert name(300, 500, 512, 128) == "gemm_panel" and name(128, 4096, 4096, 128) == "gemm_panel" and name(65, 64, 128, 64) == "gemm_panel"
    assert name(128, 4096, 4096, 128, 1 << 30) == "gemm_panel" and name(512, 4096, 4096, 128, 1 << 30) == "gemm_panel"
    assert name(128, 11008, 4096, 64, 1 << 30) == "gemm_panel" and name(1024, 2048, 4096, 128) == "gemm_panel"
    assert name(128, 1024, 4096, 128) == "gemm_panel" and name(128, 16, 4096, 128, 1 << 30) == "gemm_panel"      # however few the tiles
    assert name(128, 4096, 4224, 128, 1 << 30) == "gemm_panel_splitk" and name(256, 4096, 4224, 128, 1 << 30) == "gemm_tile_128x128_splitk"   # a longer K: split, given scratch memory
    assert name(512, 4096, 4096, 64) == "gemm_panel"                 # block 64 stops at 48 columns, 4 x 86 tiles are more than one round: the square form
    assert name(300, 500, 512, 32) == "gemm_tile_128x128"            # block 32: not its
    # 33 to 64 rows: the same on tiles of 64 rows x 32 ... 128 columns, where gemv_staged (below) does not apply or K is at most 1024
    assert name(64, 5000, 640, 128) == "gemm_panel" and name(48, 11008, 4096, 128, 1 << 30) == "gemm_panel" and name(33, 16384, 4096, 64) == "gemm_panel"
    assert name(48, 700, 640, 128) == "gemm_panel" and name(64, 2048, 1024, 64) == "gemm_panel" and name(64, 2048, 1152, 64) == "gemv_staged"
    assert name(64, 33000, 768, 128) == "gemm_wide"                  # too many columns for one round
    # 3 to 32 rows against 5120 columns or more: the same on tiles of 32 rows x 64 ... 256 columns
    assert name(32, 11008, 768, 128) == "gemm_panel" and name(16, 11008, 4096, 64) == "gemm_panel" and name(3, 5120, 4096, 128, 1 << 30) == "gemm_panel"
    assert name(32, 11008, 4096, 64, 1 << 30) == "gemm_panel" and name(16, 32000, 4096, 128) == "gemm_panel" and name(8, 50257, 768, 128) == "gemm_panel"
    assert name(16, 5119, 4096, 128) == "gemv_staged" and name(16, 11008, 4224, 128) == "gemv_staged" and name(2, 11008, 4096, 128) == "gemv_rows"
    assert name(16, 50257, 768, 64) == "gemv_staged" and name(16, 65537, 768, 128) == "gemv_staged"      # 262 tiles of 192 / 257 of 256 columns
    assert name(1, 4096, 4096, 128) == "gemv_rows" and name(2, 11008, 4096, 64) == "gemv_rows"   # weight rows read as runs
    assert name(3, 4096, 4096, 128) == "gemv_staged" and name(16, 4096, 11008, 64) == "gemv_staged"
    assert name(2, 4096, 32768, 128) == "gemv_staged"                  # 2 x 32768 codes do not fit the few-row kernel's LDS
    assert name(16, 4096, 4096, 32) == "gemm_skinny" and name(24, 4096, 4096, 32) == "gemm_skinny"     # block 32, few rows
    assert name(24, 4096, 4096, 128) == "gemv_staged" and name(32, 4096, 11008, 64) == "gemv_staged"   # two groups of 16 rows
    assert name(24, 4096, 4096, 32, 1 << 30) == "gemm_tile_64x128_splitk"      # block 32 with scratch memory: the split tiles are ahead
    # 33 to 64 rows: one pass over W where one round of workgroups covers the columns and K is short, else the split tiles
    assert name(33, 3071, 4096, 128, 1 << 30) == "gemv_staged" and name(64, 2048, 4096, 64) == "gemv_staged" and name(48, 700, 1280, 128) == "gemv_staged"
    assert name(33, 3072, 4096, 128, 1 << 30) == "gemm_panel" and name(64, 4096, 4096, 64) == "gemm_panel"      # from 3072 columns on: narrow tiles
    assert name(64, 4096, 4224, 64) == "gemv_staged"                 # ... up to K = 4096
    assert name(48, 11008, 8192, 128, 1 << 30) == "gemm_tile_64x128_splitk" and name(48, 4096, 11008, 128, 1 << 30) == "gemm_tile_64x128_splitk"
    # 33 to 64 rows, K from 5120 to 12288, up to 2048 columns: narrow tiles of 64 rows on pieces of K
    assert name(48, 2048, 11008, 128, 1 << 30) == "gemm_panel_splitk" and name(64, 1024, 5120, 64, 1 << 30) == "gemm_panel_splitk"
    assert name(64, 2049, 8192, 128, 1 << 30) == "gemm_tile_64x128_splitk" and name(64, 2048, 4992, 128, 1 << 30) != "gemm_panel_splitk"
    assert name(64, 2048, 12416, 128, 1 << 30) == "gemm_tile_64x128_splitk"
    # 17 to 32 rows, K from 8192: tiles of 32 rows where that gives 192 workgroups of three pieces per tile or more, or two of 40 stages
    assert name(32, 4096, 8192, 128, 1 << 30) == "gemm_panel_splitk" and name(17, 2048, 11008, 64, 1 << 30) == "gemm_panel_splitk"
    assert name(32, 5120, 8192, 128, 1 << 30) == "gemm_panel_splitk" and name(17, 8192, 11008, 128, 1 << 30) == "gemm_panel_splitk"
    assert name(32, 8192, 8192, 128, 1 << 30) == "gemv_staged" and name(16, 4096, 11008, 128, 1 << 30) == "gemv_staged" and name(32, 4096, 8064, 128, 1 << 30) == "gemv_staged"
    assert name(32, 1024, 8192, 128, 1 << 30) == "gemv_staged"       # 16 tiles in eight pieces: 128 workgroups
    assert name(32, 4096, 11008, 128) == "gemv_staged" and name(32, 4096, 11008, 32, 1 << 30) != "gemm_panel_splitk"      # no scratch memory; block 32
    assert name(65, 4096, 16384, 128, 1 << 30) == "gemm_tile_128x128_splitk"
    # 65 to 128 rows and K up to 12288: narrow tiles on pieces of K
    assert name(65, 4096, 8192, 128, 1 << 30) == "gemm_panel_splitk" and name(128, 4096, 11008, 64, 1 << 30) == "gemm_panel_splitk"
    assert name(128, 4096, 12416, 128, 1 << 30) == "gemm_tile_128x128_splitk" and name(129, 4096, 8192, 128, 1 << 30) != "gemm_panel_splitk"
    assert name(1, 128, 128 * 1024, 128) == "gemv_staged"            # any K: the scales stream through LDS with the stages
    assert name(128, 4096, 8192, 128) == "gemm_panel" and name(128, 32768, 8192, 128) == "gemm_tile_128x128"   # no scratch memory: one pass
    # few tiles of 256x128 and a long K: pieces of every tile on the 256x256 kernel's loop (the GPT-2 grad-weight GEMMs)
    assert name(3072, 768, 8192, 64, 1 << 25) == "gemm_wide_256x128_splitk" and name(3072, 768, 8192, 64) == "gemm_tile_128x128"
    assert name(1024, 4096, 4096, 128, 1 << 25) == "gemm_panel"               # 256 tiles of 128 x 128: nothing to split
    ws = lib.bi8_gemm_workspace_bytes(128, 2048, 16384, 128)
    # 32 tiles of 64x128, eight workgroups each: one fp32 slab of a tile per workgroup
    assert ws == 8 * 128 * 2048 * 4 and name(128, 2048, 16384, 128, ws) == "gemm_tile_64x128_splitk"
    assert name(128, 2048, 16384, 128, ws - 1) == "gemm_panel"            # too small a workspace is not used: one pass on narrow tiles
    assert name(256, 4096, 11008, 128, 1 << 30) == "gemm_tile_128x128_splitk"         # 64 tiles, four pieces each
    # 144 tiles of 128x128: runs that end inside tiles fill the chip when K is long enough to pay for the second kernel
    assert name(3072, 768, 8192, 32, 1 << 30) == "gemm_tile_128x128_splitk" and name(3072, 768, 2048, 32, 1 << 30) == "gemm_tile_128x128"
    assert name(2048, 1408, 16384, 64, 1 << 30) == "gemm_tile_128x128_splitk"      # 176 tiles: too many for pieces of 256x128 tiles
    assert name(300, 500, 500, 128) == "gemm_generic" and name(300, 500, 512, 128, 0, 520) == "gemm_generic"
    assert name(300, 500, 512, 48) == "gemm_generic"
    assert name(0, 500, 512, 128) == "none"
    # a split never wants more than the static scratch array holds: workgroups + tiles - 1 < 512 slabs of 128 x 128 fp32
    for M in (33, 64, 100, 128, 256, 512, 1000, 2048, 3072, 4000):
        for N in (128, 768, 1024, 4096, 11008, 50257):
            for K in (1024, 4096, 11008 , 8192 * 4):
                for block in (32, 64, 128):
                    assert lib.bi8_gemm_workspace_bytes(M, N, K, block) <= lib.bi8_static_scratch_bytes(), (M, N, K, block)
    # up to 16 rows at blocks 64 / 128 no plan wants scratch memory (the Python launcher does not ask for such shapes) ...
    for M in (1, 2, 3, 8, 16):
        for N in (128, 1024, 2048, 4096, 5120, 11008, 50257):
            for K in (1024, 4096, 8192, 11008, 8192 * 4):
                for block in (64, 128):
                    assert lib.bi8_gemm_workspace_bytes(M, N, K, block) == 0, (M, N, K, block)
    # ... and from 17 on some do, and the launcher asks
    from blockwise_int8_linear_amd import ops
    assert lib.bi8_gemm_workspace_bytes(17, 4096, 11008, 128) > 0
    asked = []

    class _Probe:
        def bi8_gemm_workspace_bytes(self, *a):
            asked.append(a)
            return 0
    for M in (16, 17):
        ops._ws_need.pop((M, 4096, 11008, 128), None)
        ops._workspace(_Probe(), M, 4096, 11008, 128, None, None)
        ops._ws_need.pop((M, 4096, 11008, 128), None)
    assert asked == [(17, 4096, 11008, 128)]
