"""MI355X-native blockwise int8 linear: HIP kernels for block quantize / dequantize / int8 GEMM with
fused dequantize behind a C ABI (libbi8.so), and the reference's Python operator and module API on top."""
from . import block_linear_config
from .block_linear import (
    BlockInt8Linear,
    BlockLinear,
    blockwise_int8_linear,
    blockwise_int8_linear_Wint8,
    quantize_weight_for_training,
    replace_linear_with_blockwise_int8,
    replace_linear_with_blockwise_int8_recursive,
)
from .ops import (
    dequantize_block_rowwise,
    int8_matmul_block64_rowwise_dequantize,
    int8_matmul_block_partials,
    linear_few_rows,
    quantize_block_dual,
    quantize_block_dual_colsum,
    quantize_block_rowwise,
    quantize_block_transposed,
)

__all__ = [
    "block_linear_config", "BlockInt8Linear", "BlockLinear", "blockwise_int8_linear",
    "blockwise_int8_linear_Wint8", "quantize_weight_for_training", "replace_linear_with_blockwise_int8_recursive",
    "replace_linear_with_blockwise_int8", "quantize_block_rowwise", "quantize_block_transposed",
    "dequantize_block_rowwise", "int8_matmul_block64_rowwise_dequantize", "int8_matmul_block_partials",
    "linear_few_rows", "quantize_block_dual", "quantize_block_dual_colsum",
]
