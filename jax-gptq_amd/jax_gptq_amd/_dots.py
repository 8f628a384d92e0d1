"""Recognition of the matrix products that can be quantised / routed to the packed kernel.

The reference inspects jaxpr equations (``dot_general`` with one contraction and no batch
dimensions, ``quantize_interpreter.py:380-392``; 1x1 ``conv_general_dilated``, ``:451-485``).
The counterpart here inspects the ``torch`` function that a model calls and reduces it to the
same canonical form: ``tensordot(lhs, rhs, ([lhs_contract], [rhs_contract]))`` followed by an
optional fix-up of the result (bias, axis order).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

_MATMULS = (torch.matmul, torch.Tensor.matmul, torch.Tensor.__matmul__, torch.mm, torch.Tensor.mm)
_RMATMULS = (torch.Tensor.__rmatmul__,)


class Dot:
    """``post(tensordot(lhs, rhs, ([lhs_contract], [rhs_contract])))`` with the weight on side
    ``w_side`` (0 = lhs, 1 = rhs)."""

    def __init__(self, lhs, rhs, lhs_contract, rhs_contract, w_side, post=None):
        self.lhs, self.rhs = lhs, rhs
        self.lhs_contract, self.rhs_contract = lhs_contract, rhs_contract
        self.w_side = w_side
        self.post = post

    @property
    def w(self):
        return self.rhs if self.w_side else self.lhs

    @property
    def x(self):
        return self.lhs if self.w_side else self.rhs

    @property
    def w_contract(self):
        return self.rhs_contract if self.w_side else self.lhs_contract

    @property
    def x_contract(self):
        return self.lhs_contract if self.w_side else self.rhs_contract

    def evaluate(self, w, x):
        lhs, rhs = (x, w) if self.w_side else (w, x)
        out = torch.tensordot(lhs, rhs, dims=([self.lhs_contract], [self.rhs_contract]))
        return self.post(out) if self.post is not None else out


def _ndim(a):
    return len(a.shape)


def _pair(a, b, is_w):
    """``a @ b`` with matmul semantics, or None when it is not a plain (unbatched) product."""
    wa, wb = is_w(a), is_w(b)
    if wa and wb:
        raise NotImplementedError("Currently only one quantize target is supported per op")
    if wb:
        if _ndim(b) != 2 or _ndim(a) < 1:
            return None
        return Dot(a, b, _ndim(a) - 1, 0, 1)
    if wa:
        if _ndim(a) != 2 or _ndim(b) not in (1, 2):
            return None      # W @ x with a batched x broadcasts: not a single dot_general
        return Dot(a, b, 1, 0, 0)
    return None


def parse_dot(func, args, kwargs, is_w):
    """``Dot`` for a call that multiplies by exactly one weight ``is_w(arg)``, else ``None``."""
    if func in _MATMULS and len(args) == 2 and not kwargs:
        return _pair(args[0], args[1], is_w)
    if func in _RMATMULS and len(args) == 2 and not kwargs:
        return _pair(args[1], args[0], is_w)
    if func is F.linear:
        x, w = args[0], args[1]
        bias = args[2] if len(args) > 2 else kwargs.get("bias")
        if is_w(x):
            return None
        if not is_w(w) or _ndim(w) != 2:
            return None
        post = (lambda out: out + bias) if bias is not None else None
        return Dot(x, w, _ndim(x) - 1, 1, 1, post)
    if func is torch.tensordot:
        a, b = args[0], args[1]
        dims = args[2] if len(args) > 2 else kwargs.get("dims", 2)
        wa, wb = is_w(a), is_w(b)
        if wa and wb:
            raise NotImplementedError("Currently only one quantize target is supported per op")
        if not (wa or wb):
            return None
        if isinstance(dims, int):
            if dims != 1:
                return None      # more than one contraction (quantize_interpreter.py:388-390)
            la, lb = [_ndim(a) - 1], [0]
        else:
            la, lb = list(dims[0]), list(dims[1])
            if len(la) != 1 or len(lb) != 1:
                return None
        return Dot(a, b, la[0] % _ndim(a), lb[0] % _ndim(b), 1 if wb else 0)
    if func is F.conv1d:
        # 1x1 convolution = a product over the input channels (quantize_interpreter.py:451-521)
        x, w = args[0], args[1]
        rest = list(args[2:]) + [None] * 5
        bias = kwargs.get("bias", rest[0])
        stride, padding = kwargs.get("stride", rest[1] or 1), kwargs.get("padding", rest[2] or 0)
        dilation, groups = kwargs.get("dilation", rest[3] or 1), kwargs.get("groups", rest[4] or 1)
        simple = all(v in (1, (1,), [1]) for v in (stride, dilation, groups)) and padding in (0, (0,), [0])
        if not is_w(w) or is_w(x) or _ndim(w) != 3 or w.shape[2] != 1 or _ndim(x) != 3 or not simple:
            return None

        def post(out):                      # [O, 1, B, S] -> [B, O, S]
            out = out.squeeze(1).permute(1, 0, 2)
            return out + bias[None, :, None] if bias is not None else out
        return Dot(w, x, 1, 1, 0, post)
    return None


def to_matrix(w, w_contract):
    """N-D weight -> ``[K, rest]`` with the contraction axis first
    (``permute_to_matrix(..., keep_first=True)``, ``quantize_interpreter.py:395-401``)."""
    return torch.movedim(w, w_contract, 0).reshape(w.shape[w_contract], -1)


def from_matrix(m, shape, w_contract):
    """Inverse of :func:`to_matrix` (``to_original_shape``, ``quantize_interpreter.py:403-408``)."""
    moved = [shape[w_contract]] + [d for i, d in enumerate(shape) if i != w_contract]
    return torch.movedim(m.reshape(moved), 0, w_contract)
