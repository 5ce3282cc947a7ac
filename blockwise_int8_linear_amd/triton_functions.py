"""The in-scope names of the reference's ``triton_functions`` module (triton_functions.py:142, :218, :221, :492),
so that ``from triton_functions import ...`` lines keep working once :func:`blockwise_int8_linear_amd.compat.install`
has registered this module under that name.  Everything here runs the HIP kernels of libbi8.so; nothing of the
reference's broken or dead helpers (plain ``int8_matmul``, ``groupwise_quantize``, the benchmark) is provided."""
from .ops import (  # noqa: F401
    ceil_div,
    dequantize_block_rowwise,
    int8_matmul_block64_rowwise_dequantize,
    quantize_block_rowwise,
)

__all__ = ["ceil_div", "dequantize_block_rowwise", "int8_matmul_block64_rowwise_dequantize", "quantize_block_rowwise"]
