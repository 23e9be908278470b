"""MI355X-native FP8 quantized-collective kernels, a drop-in for torchft's
``torchft.quantization`` (and its callers in ``torchft.collectives``)."""

from .quantization import (  # noqa: F401
    fused_dequantize_from_fp8,
    fused_quantize_into_fp8,
    fused_reduce_fp8,
)

__all__ = [
    "fused_dequantize_from_fp8",
    "fused_quantize_into_fp8",
    "fused_reduce_fp8",
]
