"""Shape helpers: mirror of the reference's ``jax_gptq/utils.py``."""
import torch

from .gptq import QuantizedMatrix, quant_matrix_shape


def _shape_from_param(x):
    """``QuantizedMatrix`` -> an abstract array (a ``meta`` tensor) of the logical shape and of
    ``zero.dtype`` (reference ``utils.py:6-11`` returns a ``ShapedArray``)."""
    if isinstance(x, QuantizedMatrix):
        return torch.empty(quant_matrix_shape(x), dtype=x.zero.dtype, device="meta")
    return x


def quantized_params_to_shaped_arrays(params):
    """Map a nested dict/list/tuple of parameters, replacing every ``QuantizedMatrix`` by an
    abstract array of its logical shape (reference ``utils.py:13-21``)."""
    if isinstance(params, QuantizedMatrix):
        return _shape_from_param(params)
    if isinstance(params, dict):
        return {k: quantized_params_to_shaped_arrays(v) for k, v in params.items()}
    if isinstance(params, (list, tuple)):
        return type(params)(quantized_params_to_shaped_arrays(v) for v in params)
    return params
