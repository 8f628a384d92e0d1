"""Calibration driver: host-side counterpart of the reference's
``jax_gptq/quantize_interpreter.py``.

``quantize(fn, params, inputs)`` runs ``fn(params, batch)`` on every calibration batch and
quantises, one after the other and in execution order, every parameter that ``fn`` multiplies
activations by.  As in the reference, layers are solved *sequentially*: all batches are
advanced to the next product, its inputs form the Hessian of the GPTQ solve
(:func:`jax_gptq_amd.gptq.gptq`), and (with ``use_quantized_activations``) the batches
continue with the quantised weight, so that later layers are calibrated on the activations the
quantised model really produces (``quantize_interpreter.py:151-267``).

The reference gets this control flow by interpreting the jaxpr of ``fn`` segment by segment
(``:303-378``).  ``fn`` here is an ordinary ``torch`` function, so the parameters are handed to
it as a tensor subclass that sees every ``torch`` call made on it: transposes and casts are
followed (``PARAM_TRANSFORMS``, ``:559-562``), a product with exactly one parameter operand
(``dot_general_predicate``, ``:380-392``) suspends the batch until every batch has arrived
there, and anything else just computes.  Each batch runs in a thread of its own, used as a
coroutine: exactly one of them (or the coordinator) runs at any time.
"""
from __future__ import annotations

import threading
import warnings

import numpy as np
import torch

from . import _dots
from .gptq import QuantizedMatrix, _device, accumulate_H, gptq, pack_matrix
from .transform import permute_quantized

_tls = threading.local()


# ------------------------------------------------------------------------------ pytrees
def _flatten(tree, leaves):
    """Nested dict / list / tuple -> structure with leaf indices; leaves appended in order
    (dict keys sorted, as ``jax.tree_util`` does)."""
    if isinstance(tree, dict):
        return ("dict", [(k, _flatten(tree[k], leaves)) for k in sorted(tree, key=repr)])
    if isinstance(tree, (list, tuple)) and not hasattr(tree, "_fields"):
        return (type(tree).__name__, [_flatten(v, leaves) for v in tree])
    leaves.append(tree)
    return ("leaf", len(leaves) - 1)


def _unflatten(struct, leaves):
    kind, body = struct
    if kind == "dict":
        return {k: _unflatten(v, leaves) for k, v in body}
    if kind == "list":
        return [_unflatten(v, leaves) for v in body]
    if kind == "tuple":
        return tuple(_unflatten(v, leaves) for v in body)
    return leaves[body]


def _to_device(tree, device):
    if isinstance(tree, torch.Tensor):
        return tree.to(device)
    if isinstance(tree, np.ndarray):
        return torch.from_numpy(np.ascontiguousarray(tree)).to(device)
    if isinstance(tree, dict):
        return {k: _to_device(v, device) for k, v in tree.items()}
    if isinstance(tree, (list, tuple)):
        return type(tree)(_to_device(v, device) for v in tree)
    return tree


# ------------------------------------------------------------------------------ parameters
class _Target(torch.Tensor):
    """A parameter (or a transposed / cast view of one) as ``fn`` sees it.  ``_leaf`` is its
    position among the parameter leaves, ``_perm`` the axis order relative to the leaf."""

    @staticmethod
    def __new__(cls, data, leaf, perm):
        t = torch.Tensor._make_subclass(cls, data, False)
        t._leaf, t._perm = leaf, tuple(perm)
        return t

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        return _tls.session.handle(func, args, kwargs or {})


def _plain(obj):
    if isinstance(obj, _Target):
        return obj.as_subclass(torch.Tensor)
    if isinstance(obj, (list, tuple)):
        return type(obj)(_plain(o) for o in obj)
    if isinstance(obj, dict):
        return {k: _plain(v) for k, v in obj.items()}
    return obj


def _is_target(a):
    return isinstance(a, _Target) and a.dim() > 1       # quantize_interpreter.py:315,330


_CASTS = {"float", "half", "bfloat16", "double", "to", "type", "contiguous", "detach", "clone"}


def _transform_perm(func, args, kwargs):
    """Axis permutation applied by a transform of a parameter, ``None`` for other functions."""
    w = args[0]
    n = w.dim()
    name = getattr(func, "__name__", "")
    if name == "__get__":                               # attribute getters: w.T, w.mT
        owner = getattr(func, "__self__", None)
        if owner is torch.Tensor.T:
            return tuple(reversed(range(n)))
        if owner is torch.Tensor.mT:
            name, args = "transpose", (w, -2, -1)
        else:
            return None
    if name == "t" and n == 2:
        return (1, 0)
    if name in ("transpose", "swapaxes", "swapdims") and len(args) == 3:
        perm = list(range(n))
        perm[args[1]], perm[args[2]] = perm[args[2]], perm[args[1]]
        return tuple(perm)
    if name == "permute":
        dims = args[1:] if len(args) > 1 else kwargs.get("dims")
        if len(dims) == 1 and isinstance(dims[0], (tuple, list, torch.Size)):
            dims = dims[0]
        return tuple(int(d) % n for d in dims)
    if name in _CASTS:
        return tuple(range(n))
    return None


class _Abort(BaseException):
    pass


class _Runner(threading.Thread):
    """One calibration batch, run as a coroutine on a thread."""

    def __init__(self, session, fn, params, batch, device):
        super().__init__(daemon=True)
        self.session, self.fn, self.params, self.batch, self.device = session, fn, params, batch, device
        self.go, self.back = threading.Semaphore(0), threading.Semaphore(0)
        self.request = self.reply = self.exc = None
        self.done = False

    def run(self):
        self.go.acquire()
        try:
            if not self.session.aborted:
                _tls.session, _tls.runner = self.session, self
                torch.cuda.set_device(self.device)
                with torch.no_grad():
                    self.fn(self.params, self.batch)
        except _Abort:
            pass
        except BaseException as e:      # handed to the coordinator
            self.exc = e
        finally:
            self.done = True
            self.request = None
            self.back.release()

    def resume(self):                   # coordinator side
        self.go.release()
        self.back.acquire()

    def suspend(self, request):         # batch side: wait for the coordinator's reply
        self.request = request
        self.back.release()
        self.go.acquire()
        if self.session.aborted:
            raise _Abort()
        reply, self.reply, self.request = self.reply, None, None
        return reply


class _Session:
    def __init__(self, leaves, options):
        self.leaves = leaves              # device tensors, original layout, updated in place
        self.results = {}                 # leaf -> QuantizedMatrix in the leaf's layout
        self._h_cache = None              # (signature, activations, H) of the last product
        self.options = options
        self.aborted = False

    # -------- what a torch call on a parameter does (runs on a batch thread)
    def handle(self, func, args, kwargs):
        with torch._C.DisableTorchFunctionSubclass():
            if args and isinstance(args[0], _Target) and args[0].dim() > 1:
                perm = _transform_perm(func, args, kwargs)
                if perm is not None:
                    out = func(*_plain(args), **_plain(kwargs))
                    src = args[0]
                    if isinstance(out, torch.Tensor) and out.dim() == len(perm):
                        return _Target(out, src._leaf, tuple(src._perm[p] for p in perm))
                    return out
            dot = _dots.parse_dot(func, args, kwargs, _is_target)
            if dot is not None and isinstance(dot.x, torch.Tensor):
                return self._product(dot)
            if dot is None and func in (torch.matmul, torch.Tensor.matmul, torch.Tensor.__matmul__,
                                        torch.Tensor.__rmatmul__, torch.einsum, torch.bmm) \
                    and any(_is_target(a) for a in args if isinstance(a, torch.Tensor)):
                warnings.warn(f"Operation {getattr(func, '__name__', func)} with these shapes is not "
                              "supported for quantization")
            return func(*_plain(args), **_plain(kwargs))

    def _product(self, dot):
        w = dot.w
        leaf = w._leaf
        w_plain, x = _plain(w), _plain(dot.x)
        if leaf in self.results:
            # already quantised at an earlier use; the buffer holds the quantised values
            return dot.evaluate(w_plain, x)
        reply = _tls.runner.suspend({"leaf": leaf, "perm": w._perm, "w": w_plain, "x": x,
                                     "w_contract": dot.w_contract, "x_contract": dot.x_contract})
        return dot.evaluate(reply.to(w_plain.dtype), x)

    def _shared(self, xs):
        """What ``gptq`` may reuse from the previous product (the Hessian and the factor of its
        damped inverse) when that product was applied to the very same activations (q / k / v,
        gate / up): same memory, layout and version counter, with the previous tensors kept
        alive so that the memory cannot have been handed out again."""
        sig = [(x.data_ptr(), tuple(x.shape), tuple(x.stride()), x.dtype, x._version) for x in xs]
        if self._h_cache is not None and self._h_cache[0] == sig:
            return self._h_cache[2]
        self._h_cache = None                      # release the previous activations first
        shared = {"H": accumulate_H(xs, use_fp64=self.options["use_fp64"],
                                    split_fp16=self.options["split_fp16"] and not self.options["use_fp64"])}
        self._h_cache = (sig, list(xs), shared)
        return shared

    # -------- one quantisation step (runs on the coordinator)
    def solve(self, requests):
        first = requests[0]
        key = (first["leaf"], first["perm"], first["w_contract"])
        for r in requests[1:]:
            if (r["leaf"], r["perm"], r["w_contract"]) != key:
                raise RuntimeError("the calibration batches reached different products; "
                                   "fn must take the same path for every batch")
        o = self.options
        leaf, perm, wc = key
        w = first["w"]
        W2 = _dots.to_matrix(w, wc)                                          # [K, rest]
        xs = [torch.movedim(r["x"], r["x_contract"], -1) for r in requests]   # [..., K]
        if W2.shape[0] % o["block_size"] != 0:
            raise ValueError(f"block_size={o['block_size']} must divide the contraction size "
                             f"{W2.shape[0]} of parameter {leaf}")
        Q2, qp = gptq(W=W2, xs=xs, block_size=o["block_size"], actorder=o["actorder"],
                      damping=o["damping"], use_fp64=o["use_fp64"], shared=self._shared(xs), bits=o["bits"],
                      group_size=o["group_size"])
        Qt = _dots.from_matrix(Q2, tuple(w.shape), wc)                       # layout fn sees
        if o["group_size"]:
            if w.dim() != 2 or wc != 0 or tuple(perm) != (0, 1):
                raise NotImplementedError("grouped parameters need a 2-D weight that fn contracts along axis 0")
            packed = pack_matrix(Qt.contiguous(), qp, contraction_axis=0)
        else:
            scale_shape = tuple(d for i, d in enumerate(w.shape) if i != wc)
            packed = pack_matrix(Qt.contiguous(),
                                 {"scale": qp["scale"].reshape(scale_shape),
                                  "zero": qp["zero"].reshape(scale_shape), "maxq": qp["maxq"]},
                                 contraction_axis=wc)
        inverse = tuple(int(i) for i in np.argsort(perm))
        if inverse != tuple(range(len(perm))):
            packed = permute_quantized(packed, inverse)
            packed = QuantizedMatrix(packed.int_weight.contiguous(), packed.zero.contiguous(),
                                     packed.scale.contiguous(), packed.contraction_axis, packed.bits,
                                     packed.group_size)
        self.results[leaf] = packed
        # the product is evaluated with the quantised or the original weight; every later use
        # of the parameter sees the quantised one (quantize_interpreter.py:241-243, 289-291)
        reply = Qt if o["use_quantized_activations"] else w.clone()
        self.leaves[leaf].copy_(Qt.permute(inverse).to(self.leaves[leaf].dtype))
        return reply


def quantize(fn, params, inputs, block_size=128, actorder=False, damping=0.01,
             use_quantized_activations=True, use_fp64=False, use_params_fp32=False, split_fp16=False,
             bits=4, group_size=None):
    """Run GPTQ over the parameters of ``fn`` (reference ``quantize_interpreter.py:25-80``).

    ``fn(params, batch)``: the model; ``params``: a nested dict / list / tuple of arrays;
    ``inputs``: the list of calibration batches.  Returns ``params`` with every parameter of
    two or more dimensions that ``fn`` multiplies activations by replaced by a
    :class:`QuantizedMatrix` (packed along its contraction axis, in its original layout);
    everything else is returned as it came.  Buffers of ``params`` that already live on the
    GPU are overwritten with the quantised values, so do not reuse them (the reference frees
    them, ``:42``).  ``split_fp16`` (not in the reference): see ``accumulate_H``.  ``bits`` (not in
    the reference, whose code width is fixed at 4): 4 or 8.  ``group_size`` (not in the reference): see
    ``gptq``; for 2-D weights that ``fn`` contracts along axis 0 (``x @ w``).
    """
    if int(bits) not in (4, 8):
        raise ValueError("quantize packs 4-bit or 8-bit codes")
    if not inputs:
        raise ValueError("quantize needs at least one calibration batch")
    device = _device()
    flat, struct_leaves = [], []
    struct = _flatten(params, struct_leaves)
    for leaf in struct_leaves:
        t = _to_device(leaf, device)
        if isinstance(t, torch.Tensor) and t.is_floating_point():
            if use_params_fp32:
                t = t.to(torch.float32)
            t = t.contiguous()
        flat.append(t)
    session = _Session(flat, dict(block_size=block_size, actorder=actorder, damping=damping,
                                  use_quantized_activations=use_quantized_activations,
                                  use_fp64=use_fp64, split_fp16=split_fp16, bits=int(bits),
                                  group_size=int(group_size) if group_size else None))
    wrapped = [(_Target(t, i, range(t.dim())) if isinstance(t, torch.Tensor) and t.is_floating_point()
                and t.dim() > 1 else t) for i, t in enumerate(flat)]
    fn_params = _unflatten(struct, wrapped)
    runners = [_Runner(session, fn, fn_params, _to_device(b, device), device) for b in inputs]
    for r in runners:
        r.start()
    try:
        for r in runners:
            r.resume()
        while True:
            for r in runners:
                if r.exc is not None:
                    raise r.exc
            waiting = [r for r in runners if not r.done]
            if not waiting:
                break
            if len(waiting) != len(runners):
                raise RuntimeError("some calibration batches finished while others wait at a product; "
                                   "fn must take the same path for every batch")
            reply = session.solve([r.request for r in runners])
            for r in runners:
                r.reply = reply
                r.resume()
    finally:
        session.aborted = True
        for r in runners:
            if not r.done:
                r.go.release()
        for r in runners:
            r.join(timeout=60)
    out = [session.results.get(i, leaf) for i, leaf in enumerate(struct_leaves)]
    return _unflatten(struct, out)
