"""Drop-in for the reference's block_linear_config.py:3-5: three module-level globals, changed by
assignment (``block_linear_config.GROUP_SIZE = 64``).  Every operator reads them at CALL time, so a
change takes effect for the quantizer and the GEMM together (the reference freezes the GEMM's block size
at import, triton_functions.py:19, :30, :43, while the quantizer re-reads it, :222)."""
import torch

GROUP_SIZE = 128
SHARED_EXP_TORCH_TYPE = torch.float32
INPUT_OUTPUT_TORCH_TYPE = torch.bfloat16
