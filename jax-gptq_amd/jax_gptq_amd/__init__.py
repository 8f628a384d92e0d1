"""MI355X-native GPTQ per-layer solve and packed-int4 matmul.

Host-side mirror of ``jax_gptq`` (``gptq``, ``accumulate_H``, ``pack_matrix`` /
``unpack_matrix``, ``QuantizedMatrix``, ``quantized_matmul``) over hand-written HIP
kernels for gfx950, reached through the C ABI in ``include/gptq_hip.h``.
"""
from .gptq import (QuantizedMatrix, accumulate_H, get_col_quantize_params, get_quantize_params,
                   gptq, pack_colwise, pack_matrix, pack_rowwise, quant_matrix_shape,
                   unpack_colwise, unpack_matrix, unpack_rowwise)
from .op import quantized_matmul

__all__ = [
    "QuantizedMatrix", "accumulate_H", "get_col_quantize_params", "get_quantize_params", "gptq",
    "pack_colwise", "pack_matrix", "pack_rowwise", "quant_matrix_shape", "unpack_colwise",
    "unpack_matrix", "unpack_rowwise", "quantized_matmul",
]
