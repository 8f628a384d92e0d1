"""MI355X-native GPTQ per-layer solve and packed-int4 matmul.

Host-side mirror of ``jax_gptq`` over hand-written HIP kernels for gfx950, reached through
the C ABI in ``include/gptq_hip.h``.  As in the reference, the solve lives in the
``gptq`` submodule (``from jax_gptq_amd.gptq import gptq, accumulate_H, pack_matrix, ...``)
and the operator in ``op`` (``from jax_gptq_amd.op import quantized_matmul``); ``quantize`` and
``use_quantized`` are the callers of that path: the sequential calibration driver and the
inference-time dispatch.
"""
from . import gptq, op, utils  # noqa: F401  (submodules, as in the reference's layout)
from .gptq import QuantizedMatrix
from .quantize_interpreter import quantize
from .transform import use_quantized

__all__ = ["QuantizedMatrix", "gptq", "op", "utils", "quantize", "use_quantized"]
