"""Inference with packed parameters: host-side counterpart of the reference's
``jax_gptq/transform.py``.

The reference re-interprets the jaxpr of ``f`` and, wherever an equation receives a
``QuantizedMatrix``, either calls the packed-int4 kernel (``x @ W`` with ``use_kernel``) or
unpacks the matrix and runs the equation as written (``transform.py:59-135``).  Here the
model is an ordinary ``torch`` function and ``QuantizedMatrix`` takes part in ``torch``'s
function-override protocol instead: every ``torch`` call that receives one lands in
:func:`quantized_torch_function`, which applies the same rule.
"""
from __future__ import annotations

import functools
import threading
import warnings

import torch

from . import _dots
from .gptq import QuantizedMatrix, unpack_matrix
from .op import quantized_matmul

KERNEL_AVAILABLE = True

_tls = threading.local()


def _config():
    return getattr(_tls, "config", (False, False))


def use_quantized(f, static_argnums=(), use_kernel=False, remat_unpack=False):
    """Wrap ``f`` so that ``QuantizedMatrix`` leaves among its arguments behave like the dense
    matrices they encode (reference ``transform.py:34-57``).

    ``use_kernel``: route ``x @ W`` to the packed-int4 HIP kernel; everything else, and
    everything when it is off, unpacks first.  ``remat_unpack``: do not keep unpacked weights
    for the backward pass, unpack again instead (the reference wraps the unpack in
    ``jax.checkpoint``).  ``static_argnums`` is accepted for signature compatibility; nothing
    is traced here, so every argument is passed through as it is.
    """
    del static_argnums

    @functools.wraps(f)
    def inner(*args, **kwargs):
        previous = _config()
        _tls.config = (bool(use_kernel), bool(remat_unpack))
        try:
            return f(*args, **kwargs)
        finally:
            _tls.config = previous

    return inner


class _UnpackedDot(torch.autograd.Function):
    """``dot(x, unpack(W))`` that keeps the packed matrix, not the dense one, for backward."""

    @staticmethod
    def forward(ctx, x, qm, dot):
        ctx.qm, ctx.dot = qm, dot
        ctx.x_shape = x.shape
        return dot.evaluate(unpack_matrix(qm).to(x.dtype), x)

    @staticmethod
    def backward(ctx, g):
        w = unpack_matrix(ctx.qm).to(g.dtype)
        x0 = torch.zeros(ctx.x_shape, dtype=g.dtype, device=g.device, requires_grad=True)
        with torch.enable_grad():
            y = ctx.dot.evaluate(w, x0)
        (gx,) = torch.autograd.grad(y, x0, g)      # the product is linear in x
        return gx, None, None


def _is_q(a):
    return isinstance(a, QuantizedMatrix)


def _unpack_all(obj):
    if _is_q(obj):
        return unpack_matrix(obj)
    if isinstance(obj, (list, tuple)):
        return type(obj)(_unpack_all(o) for o in obj)
    if isinstance(obj, dict):
        return {k: _unpack_all(v) for k, v in obj.items()}
    return obj


def _like_input(w, x):
    """The unpacked matrix in the element type of the other operand (``jnp`` would promote;
    ``torch`` refuses mixed products)."""
    return w.to(x.dtype) if isinstance(x, torch.Tensor) and x.is_floating_point() else w


def quantized_torch_function(func, args, kwargs):
    """What a ``torch`` function does when one of its arguments is a ``QuantizedMatrix``
    (reference ``eval_jaxpr_with_quantized_args`` / ``eval_with_quantized``,
    ``transform.py:59-135``)."""
    use_kernel, remat_unpack = _config()
    dot = _dots.parse_dot(func, args, kwargs, _is_q)
    if dot is not None:
        w, x = dot.w, dot.x
        if isinstance(x, torch.Tensor):
            if use_kernel:
                # only x @ W, contraction over the packed axis of a 2-D matrix (transform.py:116-120;
                # the 2-D / contraction_axis check is missing there and W would be misread)
                if (dot.w_side == 1 and dot.rhs_contract == 0 and dot.lhs_contract == x.dim() - 1
                        and w.int_weight.dim() == 2 and w.contraction_axis == 0):
                    out = quantized_matmul(x, w)
                    return dot.post(out) if dot.post is not None else out
                warnings.warn("Only X @ W for quantized W is supported, so quantized matrix will be unpacked")
            if remat_unpack and x.requires_grad:
                return _UnpackedDot.apply(x, w, dot)
            return dot.evaluate(_like_input(unpack_matrix(w), x), x)
    elif use_kernel:
        warnings.warn("Only dot products are supported by the kernel, so quantized matrix will be unpacked")
    return func(*_unpack_all(args), **_unpack_all(kwargs))


def permute_quantized(qm, perm):
    """The packed matrix of ``dense.permute(perm)`` (reference ``inverse_transpose``,
    ``quantize_interpreter.py:533-554``)."""
    perm = tuple(int(p) % len(perm) for p in perm)
    if getattr(qm, "group_size", 0):
        if perm != tuple(range(len(perm))):
            raise NotImplementedError("a matrix with grouped parameters cannot be transposed in packed form")
        return qm
    ca = qm.contraction_axis
    new_ca = perm.index(ca)
    scale_perm = [p if p < ca else p - 1 for p in perm if p != ca]

    def move(v):
        return v.permute(scale_perm) if isinstance(v, torch.Tensor) and v.dim() > 1 else v
    return QuantizedMatrix(int_weight=qm.int_weight.permute(perm), zero=move(qm.zero),
                           scale=move(qm.scale), contraction_axis=new_ca, bits=getattr(qm, "bits", 4),
                           group_size=getattr(qm, "group_size", 0))
