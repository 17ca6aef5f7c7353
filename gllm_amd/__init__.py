"""MI355X (gfx950) implementation of gllm's quantized-weight matmul path.

The product is ``libgllm_hip_quant.so`` (C ABI in ``include/gllm_hip_quant.h``);
``gllm_amd.backend.HipBackend`` mirrors the reference's ``Backend::quantized_matmul`` /
``Backend::dequantize`` on top of it.
"""
from .ggml import GgmlDType, QuantType, block_bytes, block_size, row_bytes, tensor_nbytes  # noqa: F401
