"""MI355X-native block-quantized matmul path behind the ``axonml-quant`` API.

``axonml_amd.quant`` mirrors the reference crate's host API over the C ABI of
``libaxq.so`` (``include/axq.h``); ``axonml_amd.csrc`` holds the HIP sources.
"""
from ._lib import LIB_PATH, AxqError, load_library  # noqa: F401
from .quant import (  # noqa: F401
    DEFAULT_BLOCK_SIZE,
    MAX_BLOCK_SIZE,
    Context,
    DeviceWeight,
    QuantError,
    QuantizedLinear,
    QuantizedTensor,
    QuantType,
    compute_quantization_error,
    compute_quantization_stats,
    default_context,
    dequantize_block,
    dequantize_tensor,
    quantize_model,
    quantize_tensor,
    quantized_matmul,
    quantized_matmul_bf16,
)
