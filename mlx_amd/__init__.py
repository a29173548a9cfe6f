"""mlx_amd -- MLX's group-wise quantized matmul path for AMD MI355X (gfx950):
``quantize`` / ``dequantize`` / ``quantized_matmul`` / ``gather_qmm`` / ``qqmm`` /
``gather_qqmm``
(affine and the mxfp4 / mxfp8 / nvfp4 modes) with the reference's operator
names and semantics, backed by hand-written HIP
kernels through the C ABI declared in ``include/mlx_rocm_qmm.h``."""
from . import nn
from .ops import (
    dequantize, from_fp8, gather_qmm, gather_qqmm, qqmm, quantize, quantized_matmul, quantized_matmul_sb_image,
    quantized_swiglu, to_fp8,
)

__all__ = [
    "quantize", "dequantize", "quantized_matmul", "quantized_matmul_sb_image", "quantized_swiglu",
    "gather_qmm", "qqmm", "gather_qqmm", "to_fp8", "from_fp8", "nn",
]
