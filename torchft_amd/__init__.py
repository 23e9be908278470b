"""MI355X-native FP8 quantized-collective kernels, a drop-in for torchft's
``torchft.quantization`` (and its callers in ``torchft.collectives``)."""

from .quantization import (  # noqa: F401
    PreparedBucket,
    fused_dequantize_from_fp8,
    fused_quantize_into_fp8,
    fused_reduce_fp8,
    prepare,
)

from .collectives import (  # noqa: F401
    allocate_reduce_scatter_output,
    allreduce_quantized,
    get_padded_sizes,
    reduce_scatter_quantized,
)

__all__ = [
    "allocate_reduce_scatter_output",
    "allreduce_quantized",
    "get_padded_sizes",
    "reduce_scatter_quantized",
    "fused_dequantize_from_fp8",
    "fused_quantize_into_fp8",
    "fused_reduce_fp8",
    "prepare",
    "PreparedBucket",
]
