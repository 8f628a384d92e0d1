"""Quantized-matmul operator: host-side mirror of the reference's ``jax_gptq/op.py``.

``quantized_matmul(x, quantized_matrix, transpose_b=False)`` flattens the leading
dimensions of ``x``, launches the packed-int4 HIP kernel (the counterpart of the
``jt.triton_call`` at ``op.py:46-63``) and restores the shape.  Like the reference's
``custom_vjp`` (``op.py:71-81``) it is differentiable with respect to ``x`` only: the
backward pass is the same operator with ``transpose_b`` flipped.
"""
from __future__ import annotations

import ctypes

import torch

from . import _native as N
from .gptq import _DT, _float_dev, _dev, _ptr, _stream, _ws


# The matmul workspace starts with split-K arrival counters that must be zero when a call
# starts; every call leaves them zero again.  One zero-initialised buffer per (device,
# stream) is therefore kept and only ever grown.
_WS_CACHE = {}


def _qmm_workspace(nbytes, device, stream_handle):
    key = (device.index, stream_handle)
    ws = _WS_CACHE.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        _WS_CACHE[key] = ws
    return ws


def _quantized_matmul_raw(x, int_weight, zero, scale, transpose_b, bits=4, group_size=0):
    lib = N.load()
    leading_dims = None
    if x.dim() > 2:
        leading_dims = x.shape[:-1]
        x = x.reshape(-1, x.shape[-1])
    elif x.dim() == 1:
        raise ValueError("x must have at least 2 dimensions")
    x = x.contiguous()
    M, K = x.shape
    if int_weight.dim() != 2:
        raise ValueError("quantized_matmul needs a 2-D packed matrix (contraction axis 0)")
    R, C = int_weight.shape
    Kw = R * (8 // bits)                 # logical rows of the packed matrix
    if transpose_b:
        K2, out_n = C, Kw
    else:
        K2, out_n = Kw, C
    assert K == K2, f"Inner dim mismatch: {K} != {K2}"
    if zero.dtype != scale.dtype:
        scale = scale.to(zero.dtype)
    out = torch.empty((M, out_n), dtype=x.dtype, device=x.device)
    handle = torch.cuda.current_stream(x.device).cuda_stream      # asked once per call
    stream = ctypes.c_void_p(handle)
    ws = _qmm_workspace(lib.gptq_hip_qmatmul_bits_workspace_bytes(M, R, C, int(transpose_b), _DT[x.dtype], bits),
                        x.device, handle)
    if group_size:
        zero, scale = zero.contiguous(), scale.contiguous()
        if tuple(zero.shape) != (Kw // group_size, C) or tuple(scale.shape) != (Kw // group_size, C):
            raise ValueError("grouped zero/scale must be [K / group_size, N]")
        N.check(lib.gptq_hip_qmatmul_grouped(stream, _ptr(x), _DT[x.dtype], M, _ptr(int_weight), R, C,
                                             _ptr(zero), _ptr(scale), _DT[zero.dtype], group_size, bits,
                                             int(transpose_b), _ptr(out), _ptr(ws), ws.numel()), "qmatmul")
    else:
        N.check(lib.gptq_hip_qmatmul_bits(stream, _ptr(x), _DT[x.dtype], M, _ptr(int_weight), R, C,
                                          _ptr(zero), _ptr(scale), _DT[zero.dtype], bits, int(transpose_b),
                                          _ptr(out), _ptr(ws), ws.numel()), "qmatmul")
    if leading_dims is not None:
        out = out.reshape(tuple(leading_dims) + (out_n,))
    return out


class _QuantizedMatmulFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, int_weight, zero, scale, transpose_b, bits, group_size):
        ctx.save_for_backward(int_weight, zero, scale)
        ctx.transpose_b = transpose_b
        ctx.bits = bits
        ctx.group_size = group_size
        return _quantized_matmul_raw(x, int_weight, zero, scale, transpose_b, bits, group_size)

    @staticmethod
    def backward(ctx, y_bar):
        int_weight, zero, scale = ctx.saved_tensors
        x_bar = _quantized_matmul_raw(y_bar.contiguous(), int_weight, zero, scale,
                                      not ctx.transpose_b, ctx.bits, ctx.group_size)
        return x_bar, None, None, None, None, None, None


def _quantized_matmul(x, quantized_matrix, transpose_b):
    x = _float_dev(x)
    if getattr(quantized_matrix, "contraction_axis", 0) != 0:
        raise ValueError("quantized_matmul needs contraction_axis == 0")
    iw = _dev(quantized_matrix.int_weight, torch.uint8)
    zero = _float_dev(quantized_matrix.zero)
    scale = _float_dev(quantized_matrix.scale)
    bits = int(getattr(quantized_matrix, "bits", 4))
    if bits not in (4, 8):
        raise ValueError("quantized_matmul takes 4-bit or 8-bit codes")
    group = int(getattr(quantized_matrix, "group_size", 0) or 0)
    if x.requires_grad:
        return _QuantizedMatmulFn.apply(x, iw, zero, scale, bool(transpose_b), bits, group)
    return _quantized_matmul_raw(x, iw, zero, scale, bool(transpose_b), bits, group)


def quantized_matmul(x, quantized_matrix, transpose_b=False):
    """``x @ dequant(W)`` (``transpose_b``: ``x @ dequant(W).T``), reference ``op.py:11-14``.

    fp32 accumulation; the result is rounded to fp16 and returned in ``x``'s dtype (``op.py:43,66-68``).
    fp16 and bf16 activations enter the matrix cores as they are; fp32 activations are rounded to
    fp16 precision after a per-row power-of-two scaling (the reference's Triton dot rounds them to
    TF32, which has the same mantissa width).  ``quantized_matrix.bits`` (4, the reference's width,
    unless ``pack_matrix`` was given 8-bit parameters) selects the code width."""
    return _quantized_matmul(x, quantized_matrix, transpose_b)


def qmatmul_fwd(x, quantized_matrix, transpose_b):
    return _quantized_matmul(x, quantized_matrix, transpose_b), quantized_matrix


def qmatmul_bwd(transposed, quantized_matrix, y_bar):
    return _quantized_matmul(y_bar, quantized_matrix, transpose_b=not transposed), None
