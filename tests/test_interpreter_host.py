"""Host logic of the calibration driver and of the inference dispatch (no GPU needed): the
canonical form of the products a model may contain, parameter pytrees, axis bookkeeping."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from jax_gptq_amd import _dots
from jax_gptq_amd import quantize_interpreter as QI


class W(torch.Tensor):
    """Marks an operand as the weight."""


def _w(t):
    return t.as_subclass(W)


def _is_w(a):
    return isinstance(a, W)


def _plain(a):
    return a.as_subclass(torch.Tensor) if isinstance(a, torch.Tensor) else a


CASES = [
    ("x @ w", lambda w, x: torch.matmul(x, w), (256, 64), (3, 5, 256), 0, 2),
    ("w @ x", lambda w, x: torch.matmul(w, x), (64, 256), (256, 7), 1, 0),
    ("w @ v", lambda w, x: torch.matmul(w, x), (64, 256), (256,), 1, 0),
    ("mm", lambda w, x: torch.mm(x, w), (256, 64), (5, 256), 0, 1),
    ("linear", lambda w, x: F.linear(x, w), (64, 256), (2, 5, 256), 1, 2),
    ("tensordot w first", lambda w, x: torch.tensordot(w, x, dims=([1], [0])), (47, 256, 12), (256, 32), 1, 0),
    ("tensordot x first", lambda w, x: torch.tensordot(x, w, dims=([1], [2])), (47, 12, 256), (32, 256), 2, 1),
    ("conv1d 1x1", lambda w, x: F.conv1d(x, w), (79, 32, 1), (11, 32, 13), 1, 1),
]


@pytest.mark.parametrize("name,f,wshape,xshape,wc,xc", CASES, ids=[c[0] for c in CASES])
def test_parse_dot_reproduces_the_call(name, f, wshape, xshape, wc, xc):
    g = torch.Generator().manual_seed(0)
    w = torch.randn(wshape, generator=g, dtype=torch.float64)
    x = torch.randn(xshape, generator=g, dtype=torch.float64)
    seen = {}

    class Spy(W):
        @classmethod
        def __torch_function__(cls, func, types, args=(), kwargs=None):
            with torch._C.DisableTorchFunctionSubclass():
                d = _dots.parse_dot(func, args, kwargs or {}, _is_w)
                if d is not None:
                    seen["dot"] = d
                args = tuple(_plain(a) for a in args)
                return func(*args, **(kwargs or {}))

    expected = f(w.as_subclass(Spy), x)
    d = seen["dot"]
    assert (d.w_contract, d.x_contract) == (wc, xc)
    got = d.evaluate(_plain(d.w), d.x)
    assert got.shape == expected.shape
    assert torch.allclose(got, _plain(expected), rtol=1e-12, atol=1e-12)
    # the matrix form the solve works on, and the way back
    m = _dots.to_matrix(_plain(d.w), wc)
    assert m.shape[0] == wshape[wc]
    assert torch.equal(_dots.from_matrix(m, wshape, wc), w)
    # contraction in matrix form equals the call
    xm = torch.movedim(d.x, xc, -1)
    flat = (xm.reshape(-1, xm.shape[-1]) @ m)
    assert torch.allclose(flat.sum(), _plain(expected).sum(), rtol=1e-9)


def test_parse_dot_rejects_what_the_reference_rejects():
    w = _w(torch.randn(4, 8, 8))
    x = torch.randn(4, 3, 8)
    assert _dots.parse_dot(torch.matmul, (x, w), {}, _is_w) is None           # batched product
    assert _dots.parse_dot(torch.tensordot, (x, w, 2), {}, _is_w) is None     # two contractions
    assert _dots.parse_dot(torch.add, (x, x), {}, _is_w) is None
    w2 = _w(torch.randn(8, 8))
    with pytest.raises(NotImplementedError):                                   # two targets in one op
        _dots.parse_dot(torch.matmul, (w2, w2), {}, _is_w)
    assert _dots.parse_dot(F.conv1d, (torch.randn(1, 8, 5), _w(torch.randn(8, 8, 3))), {}, _is_w) is None


def test_param_pytree_round_trip():
    tree = {"b": [1, (2, 3)], "a": {"w": 4, "v": None}}
    leaves = []
    struct = QI._flatten(tree, leaves)
    assert leaves == [None, 4, 1, 2, 3]            # keys in sorted order
    assert QI._unflatten(struct, leaves) == tree
    assert QI._unflatten(struct, [x if x is None else x * 10 for x in leaves]) == \
        {"b": [10, (20, 30)], "a": {"w": 40, "v": None}}


def test_transform_perm_bookkeeping():
    w = torch.randn(2, 3, 4)
    assert QI._transform_perm(torch.Tensor.permute, (w, 2, 0, 1), {}) == (2, 0, 1)
    assert QI._transform_perm(torch.Tensor.permute, (w, (2, 0, 1)), {}) == (2, 0, 1)
    assert QI._transform_perm(torch.transpose, (w, 0, 2), {}) == (2, 1, 0)
    assert QI._transform_perm(torch.Tensor.T.__get__, (w[0],), {}) == (1, 0)
    assert QI._transform_perm(torch.Tensor.mT.__get__, (w,), {}) == (0, 2, 1)
    assert QI._transform_perm(torch.Tensor.t, (w[0],), {}) == (1, 0)
    assert QI._transform_perm(torch.Tensor.half, (w,), {}) == (0, 1, 2)
    assert QI._transform_perm(torch.Tensor.reshape, (w, 6, 4), {}) is None
    assert QI._transform_perm(torch.Tensor.shape.__get__, (w,), {}) is None
    # composition used by the driver: transformed = leaf.permute(perm); leaf = transformed.permute(argsort(perm))
    perm = (2, 0, 1)
    inv = tuple(int(i) for i in np.argsort(perm))
    assert torch.equal(w.permute(perm).permute(inv), w)
