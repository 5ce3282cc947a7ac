"""Operator launchers with the reference's names, signatures and output layouts
(triton_functions.py:221-233, :492-500, :142-168), running hand-written gfx950 kernels through the
C ABI of libbi8.so.  Like the reference's launchers they allocate their outputs with torch.empty on the
input's device, enqueue on the current stream and return without synchronizing.

There is one code path: device tensors, HIP kernels.  A CPU tensor trips the same assertion as in the
reference (``assert x.is_cuda``); a missing libbi8.so raises.
"""
from __future__ import annotations

import torch

from . import _lib
from . import block_linear_config

_DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def ceil_div(n: int, d: int) -> int:
    return -(n // -d)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """hipStream_t of torch's current stream on t's device (the raw getter is ~2 us cheaper than the Stream object)"""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *a):
        return False


_NO_GUARD = _NoGuard()
_multi_device = None


def _on_device(t: torch.Tensor):
    """Context that makes t's device current for the launch; free on a one-GPU machine."""
    global _multi_device
    if _multi_device is None:
        _multi_device = torch.cuda.device_count() > 1
    return torch.cuda.device(t.device) if _multi_device else _NO_GUARD


def _float_operand(x: torch.Tensor) -> torch.Tensor:
    if x.dtype not in _DT:
        raise TypeError(f"unsupported dtype {x.dtype}: expected float32, bfloat16 or float16")
    return x if x.stride(-1) == 1 or x.numel() == 0 else x.contiguous()


def _rows(x: torch.Tensor) -> torch.Tensor:
    """2-D tensor whose rows are contiguous (leading dimension = stride(0))."""
    if x.is_contiguous():
        return x
    if x.numel() and (x.stride(1) != 1 or (x.shape[0] > 1 and x.stride(0) < x.shape[1])):
        return x.contiguous()
    return x


def _ld(x: torch.Tensor) -> int:
    return x.stride(0) if x.shape[0] > 1 else max(x.shape[1], 1)


def _scales_out(s: torch.Tensor) -> torch.Tensor:
    t = block_linear_config.SHARED_EXP_TORCH_TYPE
    return s if t == torch.float32 else s.to(t)       # the reference's store casts to the scale dtype (:216, :227)


def _scales_in(s: torch.Tensor) -> torch.Tensor:
    s = s if s.dtype == torch.float32 else s.float()
    return s if s.is_contiguous() else s.contiguous()


def quantize_block_rowwise(x: torch.Tensor, fblock_size=None):
    """x [M,K] -> (int8 codes [M,K], absmax scales [ceil(K/B), M]); triton_functions.py:221-233."""
    fblock_size = fblock_size or block_linear_config.GROUP_SIZE
    m, k = x.shape
    assert x.is_cuda
    x = _rows(_float_operand(x))
    output = torch.empty((m, k), device=x.device, dtype=torch.int8)
    # output_maxs is transposed: block-major, row-minor (:226-227)
    output_maxs = torch.empty((ceil_div(k, fblock_size), m), device=x.device, dtype=torch.float32)
    with _on_device(x):
        rc = _lib.load().bi8_quantize_rowwise(x.data_ptr(), _DT[x.dtype], output.data_ptr(), output_maxs.data_ptr(),
                                              m, k, _ld(x), max(k, 1), fblock_size, _stream(x))
    _lib.check(rc, "bi8_quantize_rowwise")
    return output, _scales_out(output_maxs)


def quantize_block_transposed(x: torch.Tensor, fblock_size=None):
    """Same result as ``quantize_block_rowwise(x.t().contiguous())`` (block_linear.py:93-94, :100-103) in one
    pass over x:  x [R,C] -> (int8 [C,R], scales [ceil(R/B), C])."""
    fblock_size = fblock_size or block_linear_config.GROUP_SIZE
    r, c = x.shape
    assert x.is_cuda
    x = _rows(_float_operand(x))
    output = torch.empty((c, r), device=x.device, dtype=torch.int8)
    output_maxs = torch.empty((ceil_div(r, fblock_size), c), device=x.device, dtype=torch.float32)
    with _on_device(x):
        rc = _lib.load().bi8_quantize_transposed(x.data_ptr(), _DT[x.dtype], output.data_ptr(), output_maxs.data_ptr(),
                                                 r, c, _ld(x), max(r, 1), fblock_size, _stream(x))
    _lib.check(rc, "bi8_quantize_transposed")
    return output, _scales_out(output_maxs)


def _code_buffer(rows: int, cols: int, device, pad: bool):
    """int8 [rows, cols]; with `pad`, a view of a buffer whose rows are padded with zero codes to a multiple of 128
    (what the tiled GEMM kernels want of a contraction dimension), so that no padded copy is needed later"""
    if pad and cols % 128 != 0 and rows > 0 and cols > 0:
        ld = ceil_div(cols, 128) * 128
        store = torch.empty((rows, ld), device=device, dtype=torch.int8)
        store[:, cols:].zero_()
        return store[:, :cols], store
    t = torch.empty((rows, cols), device=device, dtype=torch.int8)
    return t, t


def _quantize_block_dual(x: torch.Tensor, fblock_size, pad: bool, colsum: bool = False):
    r, c = x.shape
    assert x.is_cuda
    x = _rows(_float_operand(x))
    pad = pad and fblock_size in _FAST_BLOCKS
    q, q_store = _code_buffer(r, c, x.device, pad)
    qt, qt_store = _code_buffer(c, r, x.device, pad)
    s = torch.empty((ceil_div(c, fblock_size), r), device=x.device, dtype=torch.float32)
    st = torch.empty((ceil_div(r, fblock_size), c), device=x.device, dtype=torch.float32)
    lib = _lib.load()
    if colsum:
        # the column sums of x from the same read (the bias gradient when x is the output gradient)
        sums = torch.empty((c,), device=x.device, dtype=x.dtype)
        ws = torch.empty((ceil_div(r, 128) * c,), device=x.device, dtype=torch.float32)
        with _on_device(x):
            rc = lib.bi8_quantize_dual_colsum(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), qt.data_ptr(), st.data_ptr(),
                                              sums.data_ptr(), ws.data_ptr(), ws.numel() * 4, r, c, _ld(x), max(q_store.shape[1], 1),
                                              max(qt_store.shape[1], 1), fblock_size, _stream(x))
        _lib.check(rc, "bi8_quantize_dual_colsum")
        return q, _scales_out(s), qt, _scales_out(st), q_store, qt_store, sums
    with _on_device(x):
        rc = lib.bi8_quantize_dual(x.data_ptr(), _DT[x.dtype], q.data_ptr(), s.data_ptr(), qt.data_ptr(), st.data_ptr(),
                                   r, c, _ld(x), max(q_store.shape[1], 1), max(qt_store.shape[1], 1), fblock_size, _stream(x))
    _lib.check(rc, "bi8_quantize_dual")
    return q, _scales_out(s), qt, _scales_out(st), q_store, qt_store


def quantize_block_dual_colsum(x: torch.Tensor, fblock_size=None):
    """``quantize_block_dual(x)`` plus ``x.sum(dim=0)`` (fp32 accumulation, result in x's dtype) from the same pass
    over x: the output gradient's two quantizations and the bias gradient of block_linear.py:92, :101-103, :110.
    Returns (q, scales, qT, scalesT, column sums)."""
    out = _quantize_block_dual(x, fblock_size or block_linear_config.GROUP_SIZE, pad=False, colsum=True)
    return out[0], out[1], out[2], out[3], out[6]


def quantize_block_dual(x: torch.Tensor, fblock_size=None):
    """``quantize_block_rowwise(x)`` and ``quantize_block_transposed(x)`` from one pass over x:
    x [R,C] -> (int8 [R,C], scales [ceil(C/B), R], int8 [C,R], scales [ceil(R/B), C]), the same bits as the two calls.
    A training step needs both directions of X, W and G (block_linear.py:77-78, :92-94, :100-103)."""
    return _quantize_block_dual(x, fblock_size or block_linear_config.GROUP_SIZE, pad=False)[:4]


def dequantize_block_rowwise(x: torch.Tensor, state_x: torch.Tensor, fblock_size=None):
    """int8 [M,K] + scales [ceil(K/B), M] -> [M,K] of INPUT_OUTPUT_TORCH_TYPE; triton_functions.py:492-500."""
    fblock_size = fblock_size or block_linear_config.GROUP_SIZE
    out_dtype = block_linear_config.INPUT_OUTPUT_TORCH_TYPE
    assert x.is_cuda
    assert x.dtype == torch.int8, "codes must be int8"
    M, K = x.shape
    assert tuple(state_x.shape) == (ceil_div(K, fblock_size), M), "scale shape must be [ceil(K/block), M]"
    x = _rows(x)
    state_x = _scales_in(state_x)
    output = torch.empty((M, K), device=x.device, dtype=out_dtype)
    with _on_device(x):
        rc = _lib.load().bi8_dequantize_rowwise(x.data_ptr(), state_x.data_ptr(), output.data_ptr(), _DT[out_dtype],
                                                M, K, _ld(x), max(K, 1), fblock_size, _stream(x))
    _lib.check(rc, "bi8_dequantize_rowwise")
    return output


def _gemm_operands(a: torch.Tensor, b: torch.Tensor):
    assert a.is_cuda and b.is_cuda
    assert a.dtype == torch.int8 and b.dtype == torch.int8, "operands must be int8 codes"
    assert a.shape[1] == b.shape[0], "incompatible dimensions"
    a = _rows(a)
    # b is [K,N]; the kernel wants its transpose [N,K] with contiguous rows, which is what the reference's
    # callers pass (W_int8.t(), block_linear.py:80).  Anything else is copied into that layout once.
    w = b.t()
    w = _rows(w)
    return a, w


_FAST_BLOCKS = (32, 64, 128)
_PAD_MIN_WORK = 1 << 22            # M*N*K below which the general kernel is as quick as two padded copies


def _zero_padded(t, store):
    """`store` if it is t's buffer with rows padded with zero codes (see _code_buffer), else None"""
    if store is None or store is t or store.shape[0] != t.shape[0] or store.data_ptr() != t.data_ptr():
        return None
    return store


def _pad_contraction(a, w, state_x, state_w, block, a_store=None, w_store=None):
    """The tiled GEMM kernels want K to be a multiple of 128 and 16-byte aligned operand rows; a contraction like
    the GPT-2 vocabulary (50257, the grad-input GEMM of the output layer) would fall to the general kernel, which is
    ~40x slower.  Zero codes add nothing to any block partial, so such operands are copied once into buffers
    padded with zero codes up to the next multiple of 128 (and the scales with zero rows if that adds K-blocks):
    the results are the same numbers."""
    M, K = a.shape
    N = w.shape[0]
    ragged = K % 128 != 0 or _ld(a) % 16 != 0 or _ld(w) % 16 != 0 or a.data_ptr() % 16 != 0 or w.data_ptr() % 16 != 0
    if not ragged or block not in _FAST_BLOCKS or K == 0 or M * N * K < _PAD_MIN_WORK:
        return a, w, state_x, state_w, K
    k_pad = ceil_div(K, 128) * 128
    a_store, w_store = _zero_padded(a, a_store), _zero_padded(w, w_store)
    a = a_store if a_store is not None and a_store.shape[1] == k_pad else torch.nn.functional.pad(a, (0, k_pad - K))
    w = w_store if w_store is not None and w_store.shape[1] == k_pad else torch.nn.functional.pad(w, (0, k_pad - K))
    extra = k_pad // block - state_x.shape[0]
    if extra > 0:
        state_x = torch.nn.functional.pad(state_x, (0, 0, 0, extra))
        state_w = torch.nn.functional.pad(state_w, (0, 0, 0, extra))
    return a, w, state_x, state_w, k_pad


def _halve_wide_blocks(state_x, state_w, block, M, N, K):
    """A K-block of 256, 512, ... codes is two, four, ... runs of 128 codes that share their scales: with every scale row
    repeated block/128 times the GEMM runs at block 128 on the MFMA kernels, where the library itself has only its
    general kernel for such blocks (~40x slower).  Same numbers up to fp32 rounding: the int32 partial of the block is
    folded into the accumulator in pieces of 128 codes, each with the block's scales, instead of in one.  (The
    reference's kernel takes any power of two as its BLOCK_K, triton_functions.py:30, :43-56.)"""
    if block <= 128 or block % 128 != 0 or block & (block - 1) or K == 0 or M * N * K < _PAD_MIN_WORK:
        return state_x, state_w, block
    rows = ceil_div(K, 128)
    return (state_x.repeat_interleave(block // 128, dim=0)[:rows], state_w.repeat_interleave(block // 128, dim=0)[:rows], 128)


def int8_matmul_block64_rowwise_dequantize(a, b, state_x, state_w, bias=None):
    """a int8 [M,K], b int8 [K,N] (any strides), state_x [K/B, M], state_w [K/B, N], bias [N] or None
    -> [M,N] of INPUT_OUTPUT_TORCH_TYPE; triton_functions.py:142-168.  B = GROUP_SIZE at call time."""
    return _int8_matmul(a, b, state_x, state_w, bias)


def _int8_matmul(a, b, state_x, state_w, bias=None, a_store=None, w_store=None):
    """the launcher; a_store / w_store: the zero-padded buffers that a and b.t() are views of, if any"""
    block = block_linear_config.GROUP_SIZE
    out_dtype = block_linear_config.INPUT_OUTPUT_TORCH_TYPE
    a, w = _gemm_operands(a, b)
    M, K = a.shape
    N = w.shape[0]
    nblk = ceil_div(K, block)
    assert tuple(state_x.shape) == (nblk, M) and tuple(state_w.shape) == (nblk, N), "scale shapes must be [ceil(K/block), rows]"
    state_x, state_w = _scales_in(state_x), _scales_in(state_w)
    state_x, state_w, block = _halve_wide_blocks(state_x, state_w, block, M, N, K)
    a, w, state_x, state_w, K = _pad_contraction(a, w, state_x, state_w, block, a_store, w_store)
    c = torch.empty((M, N), device=a.device, dtype=out_dtype)
    bias_ptr, bias_dt = None, 0
    if bias is not None:
        assert bias.is_cuda and bias.numel() == N
        if bias.dtype not in _DT:
            bias = bias.float()
        bias = bias.contiguous()
        bias_ptr, bias_dt = bias.data_ptr(), _DT[bias.dtype]
    lib = _lib.load()
    stream = _stream(a)
    ws, ws_bytes = _workspace(lib, M, N, K, block, a.device, stream)
    with _on_device(a):
        rc = lib.bi8_gemm_nt_dequant_ws(a.data_ptr(), w.data_ptr(), state_x.data_ptr(), state_w.data_ptr(),
                                        bias_ptr, bias_dt, c.data_ptr(), _DT[out_dtype], M, N, K,
                                        _ld(a), _ld(w), max(N, 1), block, ws.data_ptr() if ws is not None else None, ws_bytes,
                                        stream)
    _lib.check(rc, "bi8_gemm_nt_dequant_ws")
    return c


_ws_need = {}                       # (M, N, K, block) -> bytes of scratch memory the library's split of K wants (0: none)
_ws_held = {}                       # (device index, stream) -> uint8 tensor, grown on demand


def _workspace(lib, M, N, K, block, device, stream):
    """Scratch memory for a GEMM of fewer output tiles than compute units (the library then splits K over the
    workgroups and sums the pieces): (tensor or None, bytes).  What a shape wants is asked once; the memory is one
    tensor per device and stream, kept for the life of the process (at most 32 MiB each) and shared by the GEMMs of
    that stream, which run one after the other.  While the stream is being captured into a graph the memory comes from
    the capture's own pool instead, so that graphs replayed side by side do not share it.
    (Up to 16 rows at blocks 64 / 128 run the one-pass decode kernels whatever they are given: not asked.)"""
    if M <= 16 and block != 32:
        return None, 0
    key = (M, N, K, block)
    need = _ws_need.get(key)
    if need is None:
        need = _ws_need[key] = lib.bi8_gemm_workspace_bytes(M, N, K, block)
    if not need:
        return None, 0
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(need, device=device, dtype=torch.uint8), need
    held = _ws_held.get((device.index, stream))
    if held is None or held.numel() < need:
        # (allocated on the current stream, which is `stream`: torch's allocator orders a later reuse of a replaced
        # tensor's memory behind the work already queued there)
        held = _ws_held[(device.index, stream)] = torch.empty(need, device=device, dtype=torch.uint8)
    return held, need


_FEW_ROWS = 2
_FEW_ROWS_LDS = 64 * 1024


def _few_rows_lds(M: int, K: int, block: int, elem_bytes: int) -> int:
    """LDS bytes of the one-launch few-row kernel: scales of the K-blocks (whole 1 KiB runs of K plus one, in multiples
    of 16) for 4 + 16 rows, the activations' codes, 1 KiB of slack, the un-quantized activations"""
    return ceil_div((ceil_div(K, 1024) + 1) * (1024 // block), 16) * 16 * 80 + (1 if M <= 1 else 2) * K + 1024 + M * K * elem_bytes


def linear_few_rows(x, W_int8, state_W, bias=None):
    """``quantize_block_rowwise(x)`` followed by ``int8_matmul_block64_rowwise_dequantize(x_int8, W_int8.t(),
    state_x, state_W, bias)`` (BlockInt8Linear.infer, block_linear.py:141-144) as ONE kernel, for the few-row case of
    token-by-token decode: x [M,K] float with 1 <= M <= 2, W_int8 [N,K] and state_W [K/B, N] the cached weights.
    Returns the same bits as the two launchers, or None when the operands are outside what the fused kernel covers
    (the caller then runs the two launchers)."""
    block = block_linear_config.GROUP_SIZE
    dtype = block_linear_config.INPUT_OUTPUT_TORCH_TYPE
    M, K = x.shape
    N = W_int8.shape[0]
    if not (1 <= M <= _FEW_ROWS and block in (64, 128) and K > 0 and K % 128 == 0 and N > 0 and x.dtype == dtype
            and x.dtype in _DT and W_int8.dtype == torch.int8 and state_W.dtype == torch.float32
            and _few_rows_lds(M, K, block, x.element_size()) <= _FEW_ROWS_LDS):
        return None
    assert x.is_cuda and W_int8.is_cuda
    assert W_int8.shape[1] == K and tuple(state_W.shape) == (K // block, N), "incompatible dimensions"
    x, w = _rows(x), _rows(W_int8)
    state_W = state_W if state_W.is_contiguous() else state_W.contiguous()
    bias_ptr, bias_dt = None, 0
    if bias is not None:
        assert bias.is_cuda and bias.numel() == N
        if bias.dtype not in _DT:
            bias = bias.float()
        bias = bias.contiguous()
        bias_ptr, bias_dt = bias.data_ptr(), _DT[bias.dtype]
    c = torch.empty((M, N), device=x.device, dtype=dtype)
    with _on_device(x):
        rc = _lib.load().bi8_linear_few_rows(x.data_ptr(), _DT[dtype], w.data_ptr(), state_W.data_ptr(), bias_ptr, bias_dt,
                                             c.data_ptr(), M, N, K, _ld(x), _ld(w), N, block, _stream(x))
    if rc == _lib.ERR_UNSUPPORTED:          # alignment of a view, for instance
        return None
    _lib.check(rc, "bi8_linear_few_rows")
    return c


def few_rows_plan(x, W_int8, state_W, bias):
    """``linear_few_rows`` with everything that does not change from call to call checked and looked up once: returns
    ``call(x) -> output or None`` for activations of x's shape and dtype against these weights under the present
    ``block_linear_config``, or None when the one-launch kernel does not cover the case.  The closure holds the
    tensors it was made from; make a new one when the weights' buffers, the bias or the configuration change."""
    block = block_linear_config.GROUP_SIZE
    dtype = block_linear_config.INPUT_OUTPUT_TORCH_TYPE
    M, K = x.shape
    N = W_int8.shape[0]
    if not (1 <= M <= _FEW_ROWS and block in (64, 128) and K > 0 and K % 128 == 0 and N > 0 and x.dtype == dtype
            and x.dtype in _DT and W_int8.dtype == torch.int8 and state_W.dtype == torch.float32 and x.is_cuda and W_int8.is_cuda
            and W_int8.shape[1] == K and tuple(state_W.shape) == (K // block, N) and state_W.is_contiguous()
            and W_int8.stride(1) == 1 and (bias is None or (bias.is_cuda and bias.numel() == N and bias.dtype in _DT and bias.is_contiguous()))
            and _few_rows_lds(M, K, block, x.element_size()) <= _FEW_ROWS_LDS):
        return None
    fn = _lib.load().bi8_linear_few_rows
    guard = _on_device(x)
    dt, ldw, dev, index = _DT[dtype], _ld(W_int8), x.device, x.device.index
    w_ptr, sw_ptr = W_int8.data_ptr(), state_W.data_ptr()
    b_ptr, b_dt = (None, 0) if bias is None else (bias.data_ptr(), _DT[bias.dtype])
    keep = (W_int8, state_W, bias)
    raw, unsupported, check, empty = _raw_stream, _lib.ERR_UNSUPPORTED, _lib.check, torch.empty

    def call(x):
        if x.stride(1) != 1:
            return None
        c = empty((M, N), device=dev, dtype=dtype)
        with guard:
            rc = fn(x.data_ptr(), dt, w_ptr, sw_ptr, b_ptr, b_dt, c.data_ptr(), M, N, K, x.stride(0) if M > 1 else K, ldw, N, block,
                    raw(index) if raw is not None else torch.cuda.current_stream(dev).cuda_stream)
        if rc:
            if rc == unsupported:                   # alignment of a view, for instance
                return None
            check(rc, "bi8_linear_few_rows")
        return c

    call.keep = keep
    return call


def int8_matmul_block_partials(a, b, fblock_size=None):
    """The GEMM kernel's int32 block partials, before any scaling: int32 [ceil(K/B), M, N]
    (what ``tl.dot`` yields at triton_functions.py:115).  Parity/debug operator."""
    block = fblock_size or block_linear_config.GROUP_SIZE
    a, w = _gemm_operands(a, b)
    M, K = a.shape
    N = w.shape[0]
    p = torch.empty((ceil_div(K, block), M, N), device=a.device, dtype=torch.int32)
    with _on_device(a):
        rc = _lib.load().bi8_gemm_nt_partials(a.data_ptr(), w.data_ptr(), p.data_ptr(), M, N, K, _ld(a), _ld(w),
                                              block, _stream(a))
    _lib.check(rc, "bi8_gemm_nt_partials")
    return p
