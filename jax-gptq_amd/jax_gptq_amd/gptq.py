"""Host-side mirror of the reference's ``jax_gptq/gptq.py`` on top of the HIP C ABI.

Same names, argument order, defaults, return structure and error behaviour as the
reference; arrays are ``torch`` tensors on the GPU (torch is used for device memory
and streams only -- every computation is a kernel of ``libgptq_hip.so``).  NumPy
arrays and CPU tensors are accepted and moved to the device.
"""
from __future__ import annotations

import ctypes

import numpy as np
import torch

from . import _native as N

__all__ = [
    "QuantizedMatrix", "quant_matrix_shape", "accumulate_H", "get_quantize_params",
    "get_col_quantize_params", "gptq", "pack_matrix", "unpack_matrix", "pack_along_axis",
    "unpack_along_axis", "pack_rowwise", "pack_colwise", "unpack_rowwise", "unpack_colwise",
]

_DT = {torch.float32: N.F32, torch.float16: N.F16, torch.bfloat16: N.BF16}
_DT_H = {torch.float32: N.F32, torch.float64: N.F64}       # element types of H and L
_DT_X64 = {**_DT, torch.float64: N.F64}                    # batches of the fp64 Hessian


_HAVE_GPU = None       # torch.cuda.is_available(), asked once (it reads the environment on every call)


def _device():
    global _HAVE_GPU
    if _HAVE_GPU is None:
        _HAVE_GPU = bool(torch.cuda.is_available())
    if not _HAVE_GPU:
        raise RuntimeError("jax_gptq_amd needs a ROCm GPU (gfx950); there is no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


def _dev(x, dtype=None):
    """Array-like -> contiguous tensor on the current GPU."""
    if isinstance(x, torch.Tensor):
        t = x
        # the common case of the per-call operators: already in place
        if t.is_cuda and t.device.index == torch.cuda.current_device():
            if dtype is not None and t.dtype != dtype:
                t = t.to(dtype)
            return t if t.is_contiguous() else t.contiguous()
    else:
        t = torch.from_numpy(np.ascontiguousarray(np.asarray(x)))
    t = t.to(_device())
    if dtype is not None and t.dtype != dtype:
        t = t.to(dtype)
    return t.contiguous()


def _float_dev(x, keep_fp64=False):
    t = _dev(x)
    if t.dtype not in _DT and not (keep_fp64 and t.dtype == torch.float64):
        t = t.to(torch.float32)     # integer / fp64 inputs are promoted to fp32, as jnp would
    return t


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _ws(nbytes):
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=_device())


def _zeros(shape, dtype):
    """Zero-filled device tensor: torch allocates, the library's fill kernel writes."""
    t = torch.empty(shape, dtype=dtype, device=_device())
    N.check(N.load().gptq_hip_fill_zero(_stream(), _ptr(t), t.numel() * t.element_size()), "fill_zero")
    return t


def _clone(t):
    out = torch.empty_like(t)
    N.check(N.load().gptq_hip_copy(_stream(), _ptr(out), _ptr(t), t.numel() * t.element_size()), "copy")
    return out


def _to_f32_copy(t):
    """fp32 working copy of a float tensor (always a new buffer: the column loop consumes it)."""
    out = torch.empty(t.shape, dtype=torch.float32, device=t.device)
    N.check(N.load().gptq_hip_to_f32(_stream(), _ptr(t), _DT[t.dtype], t.numel(), _ptr(out)), "to_f32")
    return out


class QuantizedMatrix:
    """Packed matrix container (reference ``gptq.py:8-22``): ``int_weight`` uint8 with two
    4-bit codes per byte along ``contraction_axis``, per-channel ``zero`` and ``scale``.
    ``bits`` (not in the reference, which is fixed at 4): 8 means one code per byte.  ``group_size`` (not in
    the reference either): ``zero`` / ``scale`` are ``[K / group_size, N]`` tables of a 2-D matrix packed along
    axis 0, one row per group of ``group_size`` consecutive input features; 0 means one value per channel."""

    def __init__(self, int_weight, zero, scale, contraction_axis=0, bits=4, group_size=0):
        if bits not in (4, 8):
            raise ValueError("bits must be 4 or 8")
        if group_size and contraction_axis != 0:
            raise ValueError("grouped parameters need contraction_axis == 0")
        self.group_size = int(group_size)
        self.int_weight = int_weight
        self.zero = zero
        self.scale = scale
        self.contraction_axis = contraction_axis
        self.bits = bits

    @property
    def shape(self):
        return quant_matrix_shape(self)

    @property
    def dtype(self):
        return self.zero.dtype

    # pytree-style helpers (the reference registers the class as a pytree, gptq.py:24-32)
    def tree_flatten(self):
        plain = self.bits == 4 and not self.group_size
        aux = self.contraction_axis if plain else (self.contraction_axis, self.bits, self.group_size)
        return (self.int_weight, self.zero, self.scale), aux

    @classmethod
    def tree_unflatten(cls, aux, children):
        axis, bits, group = aux if isinstance(aux, tuple) else (aux, 4, 0)
        return cls(*children, contraction_axis=axis, bits=bits, group_size=group)

    def to(self, *args, **kwargs):
        """Move to a device.  Element-type requests are ignored: a cast of a packed parameter
        is the identity (reference ``inverse_convert_type``, ``quantize_interpreter.py:556-557``)."""
        device = kwargs.get("device")
        for a in args:
            if isinstance(a, (str, torch.device, int)):
                device = a
        if device is None:
            return self
        return QuantizedMatrix(self.int_weight.to(device), self.zero.to(device),
                               self.scale.to(device), self.contraction_axis, self.bits, self.group_size)

    # ---- array-like behaviour inside model functions.  A model written for dense weights
    # (x @ w, F.linear(x, w), w.T @ x, torch.tensordot(w, x, ...)) runs unchanged on packed ones:
    # torch hands every call that receives a QuantizedMatrix to transform.quantized_torch_function
    # (the counterpart of the reference's jaxpr re-interpretation, transform.py:59-135).
    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        from . import transform
        return transform.quantized_torch_function(func, args, kwargs or {})

    def __matmul__(self, other):
        return torch.matmul(self, other)

    def __rmatmul__(self, other):
        return torch.matmul(other, self)

    def dim(self):
        return len(self.shape)

    ndim = property(dim)

    def size(self, i=None):
        return torch.Size(self.shape) if i is None else self.shape[i]

    def permute(self, *dims):
        from . import transform
        if len(dims) == 1 and isinstance(dims[0], (tuple, list)):
            dims = tuple(dims[0])
        return transform.permute_quantized(self, dims)

    def transpose(self, dim0, dim1):
        perm = list(range(self.dim()))
        perm[dim0], perm[dim1] = perm[dim1], perm[dim0]
        return self.permute(*perm)

    def t(self):
        return self.transpose(0, 1) if self.dim() == 2 else self

    @property
    def T(self):
        return self.permute(*reversed(range(self.dim())))

    @property
    def mT(self):
        return self.transpose(-2, -1)

    def float(self):
        return self

    half = bfloat16 = double = contiguous = detach = float

    def __getattr__(self, name):
        # any other tensor method (w.sum(), w.abs(), ...): unpack, then do as written
        # (reference transform.py:74-79)
        if name.startswith("_") or name in ("int_weight", "zero", "scale", "contraction_axis", "bits", "group_size"):
            raise AttributeError(name)
        return getattr(unpack_matrix(self), name)


def quant_matrix_shape(quantized_matrix, bits=None):
    """Logical shape of a packed matrix (reference ``gptq.py:34-42``); ``bits`` defaults to the
    container's code width (the reference's 4 where it has none)."""
    if bits is None:
        bits = getattr(quantized_matrix, "bits", 4)
    mat = quantized_matrix.int_weight
    ele_width = mat.element_size() * 8 if isinstance(mat, torch.Tensor) else mat.dtype.itemsize * 8
    shape = list(mat.shape)
    shape[quantized_matrix.contraction_axis] *= ele_width // bits
    return tuple(shape)


# ------------------------------------------------------------------------------- Hessian
_MAX_BATCHES_PER_CALL = 1024


_METADATA = frozenset(("shape", "dtype", "device", "ndim", "is_cuda", "requires_grad", "layout", "names", "grad_fn"))
_METADATA_CALLS = frozenset(("dim", "size", "stride", "is_contiguous", "numel", "element_size", "nelement",
                             "storage_offset", "is_floating_point", "ndimension", "get_device"))


class _UpperH(torch.Tensor):
    """The Hessian state between two ``_accumulate_H_step`` calls.  The kernel adds a batch to the upper tiles
    only; completing the lower triangle costs a pass over the whole matrix, as much as a fifth of a 2048-row batch
    at K = 4096, so it is put off until something other than the next step looks at the values: any torch
    function (and ``data_ptr``) completes it first.  Shape and type queries do not."""

    @staticmethod
    def wrap(t):
        r = t.as_subclass(_UpperH)
        r._pending = True
        return r

    def _complete(self):
        if getattr(self, "_pending", False):
            self._pending = False
            with torch._C.DisableTorchFunctionSubclass():
                N.check(N.load().gptq_hip_hessian_finalize(_stream(), ctypes.c_void_p(self.data_ptr()),
                                                           _DT_H[self.dtype], self.shape[0], 1.0), "hessian_finalize")

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        name = getattr(func, "__name__", "")
        meta = (name in _METADATA_CALLS or
                (name == "__get__" and getattr(getattr(func, "__self__", None), "__name__", "") in _METADATA))
        if not meta:
            for a in list(args) + list(kwargs.values()):
                if isinstance(a, _UpperH):
                    a._complete()
                elif isinstance(a, (list, tuple)):
                    for b in a:
                        if isinstance(b, _UpperH):
                            b._complete()
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **kwargs)


def _accumulate_H_step(H, running_mean, n_samples, batch):
    """One batch of the Hessian accumulation (reference ``gptq.py:57-74``).

    The state differs from the reference's in representation, not in meaning: ``H`` carries the
    raw second-moment sum ``sum_b X_b^T X_b`` as a full symmetric matrix and ``running_mean`` stays
    zero, so that the reference's closing formula ``H / n + outer(mean, mean)`` (``gptq.py:100-101``)
    yields ``sum X^T X / n``, the matrix ``accumulate_H`` returns.  The kernel adds to the upper
    tiles; the mirror into the lower triangle is made when the caller looks at ``H`` (see ``_UpperH``), not after
    every step, so ``H`` is a valid state whenever the caller looks at it and a chain of steps pays for one mirror.
    """
    N.load()
    batch = _float_dev(batch, keep_fp64=(H.dtype == torch.float64))
    if batch.dim() > 2:
        batch = batch.reshape(-1, batch.shape[-1])
    elif batch.dim() == 1:
        batch = batch.reshape(1, -1)
    if batch.shape[-1] != H.shape[0]:
        raise ValueError("the batch and H disagree on the feature dimension")
    if batch.shape[0] > 0:
        with torch._C.DisableTorchFunctionSubclass():       # (taking H's address must not complete it)
            _hessian_accumulate(H, [batch.contiguous()])
        if not isinstance(H, _UpperH):
            H = _UpperH.wrap(H)
        H._pending = True
    return H, running_mean, n_samples + batch.shape[0]


def _split16_ok(H, batches):
    """Shapes that gptq_hip_hessian_accumulate_split16 takes (fp32 rows and sums, K a multiple of
    256, every batch a multiple of 32 rows and 16-byte aligned) and on which it is the faster one
    (K >= 1024: at K = 768 the fp32 kernel needs 0.8 ms for 65536 rows, the split path 1.0 ms)."""
    K = H.shape[0]
    return (H.dtype == torch.float32 and K % 256 == 0 and K >= 1024 and len(batches) > 0
            and all(b.dtype == torch.float32 and b.shape[0] % 32 == 0 and b.data_ptr() % 16 == 0 for b in batches)
            and sum(b.shape[0] for b in batches) >= 32)


def _hessian_accumulate_split16(H, batches):
    lib = N.load()
    K = H.shape[0]
    batches = [b for b in batches if b.shape[0] > 0]
    ws = _ws(lib.gptq_hip_hessian_accumulate_split16_workspace_bytes(K, max(b.shape[0] for b in batches)))
    nb = len(batches)
    ptrs = (ctypes.c_void_p * nb)(*[b.data_ptr() for b in batches])
    rows = (ctypes.c_int64 * nb)(*[b.shape[0] for b in batches])
    N.check(lib.gptq_hip_hessian_accumulate_split16(_stream(), ptrs, rows, nb, K, _ptr(H), _ptr(ws), ws.numel()),
            "hessian_accumulate_split16")


def _hessian_accumulate(H, batches):
    lib = N.load()
    K = H.shape[0]
    ws = _ws(lib.gptq_hip_hessian_accumulate_workspace_bytes(K, _DT_H[H.dtype]))
    for lo in range(0, len(batches), _MAX_BATCHES_PER_CALL):
        chunk = batches[lo:lo + _MAX_BATCHES_PER_CALL]
        dts = {b.dtype for b in chunk}
        if len(dts) != 1:
            # one launch table per element type
            for b in chunk:
                _hessian_accumulate(H, [b])
            continue
        nb = len(chunk)
        ptrs = (ctypes.c_void_p * nb)(*[b.data_ptr() for b in chunk])
        rows = (ctypes.c_int64 * nb)(*[b.shape[0] for b in chunk])
        N.check(lib.gptq_hip_hessian_accumulate(_stream(), ptrs, rows, nb, _DT_X64[chunk[0].dtype],
                                                K, _ptr(H), _DT_H[H.dtype], _ptr(ws), ws.numel()),
                "hessian_accumulate")


def accumulate_H(xs, use_fp64=False, split_fp16=False):
    """``H = sum_b X_b^T X_b / n`` over a list of calibration batches (``gptq.py:76-103``);
    fp32, or fp64 products and sums with ``use_fp64`` (``gptq.py:88``).  ``split_fp16`` (not in
    the reference) multiplies fp32 rows as pairs of fp16 numbers on the 16-bit matrix cores where
    the shapes allow it: 2.2 times faster at K = 4096, products exact to 2^-22."""
    lib = N.load()
    hdt = torch.float64 if use_fp64 else torch.float32
    batches = []
    for x in xs:
        b = _float_dev(x, keep_fp64=use_fp64)
        if b.dim() > 2:
            b = b.reshape(-1, b.shape[-1])
        elif b.dim() == 1:
            b = b.reshape(1, -1)
        batches.append(b.contiguous())
    K = batches[0].shape[-1]
    for b in batches:
        if b.shape[-1] != K:
            raise ValueError("all calibration batches must share the feature dimension")
    H = _zeros((K, K), hdt)
    if split_fp16 and _split16_ok(H, batches):
        _hessian_accumulate_split16(H, batches)
    else:
        _hessian_accumulate(H, batches)
    n = sum(b.shape[0] for b in batches)
    N.check(lib.gptq_hip_hessian_finalize(_stream(), _ptr(H), _DT_H[hdt], K, float(n)),
            "hessian_finalize")
    return H


# ------------------------------------------------------------------------------- params
def get_col_quantize_params(weight, bits=4):
    """Per-output-channel (column) min-max parameters (reference ``gptq.py:105-118``)."""
    lib = N.load()
    W = _float_dev(weight)
    if W.dim() != 2:
        raise ValueError("get_col_quantize_params expects a 2-D matrix")
    K, Nc = W.shape
    scale = torch.empty(Nc, dtype=torch.float32, device=W.device)
    zero = torch.empty(Nc, dtype=torch.float32, device=W.device)
    ws = _ws(lib.gptq_hip_col_params_workspace_bytes(K, Nc))
    N.check(lib.gptq_hip_col_params(_stream(), _ptr(W), _DT[W.dtype], K, Nc, Nc, bits, _ptr(scale),
                                    _ptr(zero), _ptr(ws), ws.numel()), "col_params")
    return {"maxq": 2 ** bits - 1, "scale": scale, "zero": zero}


def get_quantize_params(weight, bits=4):
    """Parameters of one channel: min-max over the whole array (``gptq.py:105-116``)."""
    W = _float_dev(weight).reshape(-1, 1)
    p = get_col_quantize_params(W, bits=bits)
    return {"maxq": p["maxq"], "scale": p["scale"].reshape(()), "zero": p["zero"].reshape(())}


# ------------------------------------------------------------------------------- factor
def _damp_invert(W, H, damping, fix_dead=True, want_f32=False):
    """Returns ``(L, L32, status)``: ``L`` in ``H``'s element type; ``L32`` its fp32 rounding when
    ``H`` is fp64 and ``want_f32`` is set (``L`` itself when ``H`` is fp32)."""
    lib = N.load()
    K = H.shape[0]
    Nc = 0 if W is None else W.shape[1]
    L = torch.empty((K, K), dtype=H.dtype, device=H.device)
    L32 = None
    if want_f32:
        L32 = L if H.dtype == torch.float32 else torch.empty((K, K), dtype=torch.float32,
                                                             device=H.device)
    status = _zeros((2,), torch.int32)
    hdt = _DT_H[H.dtype]
    ws = _ws(lib.gptq_hip_damp_invert_workspace_bytes(K, hdt))
    N.check(lib.gptq_hip_damp_invert(_stream(), _ptr(H), hdt, _ptr(W), K, Nc, Nc, float(damping),
                                     1 if fix_dead else 0, _ptr(L),
                                     _ptr(L32 if H.dtype == torch.float64 else None),
                                     _ptr(status), _ptr(ws), ws.numel()), "damp_invert")
    return L, L32, status


def _factor_dtype(mat):
    t = _dev(mat)
    return t if t.dtype == torch.float64 else t.to(torch.float32)


def _cholesky_inv(mat):
    """Lower Cholesky factor of ``inv(mat)`` (reference ``gptq.py:44-48``), in fp64 for an fp64
    matrix and in fp32 otherwise."""
    H = _factor_dtype(mat).clone()
    L, _, _ = _damp_invert(None, H, 0.0, fix_dead=False)
    return L


def _damp_and_invert(W, H, damping):
    """Dead-feature fix, damping, factor of the inverse (reference ``gptq.py:155-168``).
    ``W`` and ``H`` are updated in place (the reference donates both)."""
    L, _, status = _damp_invert(W, H, damping, fix_dead=True)
    any_nan = bool(status[0].item() != 0)
    return W, L, any_nan


# ------------------------------------------------------------------------------- act-order
def _permute(W, H):
    """Rows of ``W`` and rows/columns of ``H`` in descending ``diag(H)`` order (``gptq.py:170-175``)."""
    lib = N.load()
    K, Nc = W.shape
    perm = torch.argsort(torch.diagonal(H), stable=True).flip(0).contiguous()
    Wp = torch.empty_like(W)
    Hp = torch.empty_like(H)
    N.check(lib.gptq_hip_gather_rows(_stream(), _ptr(W), _ptr(Wp), W.element_size(), K, Nc,
                                     _ptr(perm)), "gather_rows")
    N.check(lib.gptq_hip_gather_sym(_stream(), _ptr(H), _ptr(Hp), H.element_size(), K, _ptr(perm)),
            "gather_sym")
    return Wp, Hp, perm


def _unpermute(Q, perm):
    """Inverse row permutation (reference ``gptq.py:177-180``)."""
    lib = N.load()
    K, Nc = Q.shape
    invperm = torch.argsort(perm, stable=True).contiguous()
    out = torch.empty_like(Q)
    N.check(lib.gptq_hip_gather_rows(_stream(), _ptr(Q), _ptr(out), Q.element_size(), K, Nc,
                                     _ptr(invperm)), "gather_rows")
    return out


# ------------------------------------------------------------------------------- loop
def _process_block(W, Hinv, start, quantize_params, block_size):
    """One block of the column loop (reference ``gptq.py:130-153``): returns
    ``(q_block, errors)``, both ``[block_size, N]`` fp32."""
    lib = N.load()
    W = _dev(W, torch.float32)
    Hinv = _dev(Hinv, torch.float32)
    K, Nc = W.shape
    if start < 0 or start + block_size > K:
        raise ValueError("block out of range")
    blk = W[start:start + block_size]
    q = torch.empty((block_size, Nc), dtype=torch.float32, device=W.device)
    err = torch.empty((block_size, Nc), dtype=torch.float32, device=W.device)
    lblk = Hinv[start:, start:]
    # named locals: the tensors must stay alive until the launch has been enqueued
    scale = _dev(quantize_params["scale"], torch.float32)
    zero = _dev(quantize_params["zero"], torch.float32)
    N.check(lib.gptq_hip_process_block(
        _stream(), _ptr(blk), Nc, ctypes.c_void_p(lblk.data_ptr()), Hinv.shape[1], block_size,
        _ptr(scale), _ptr(zero), int(quantize_params["maxq"]),
        _ptr(q), N.F32, ctypes.c_void_p(0), _ptr(err)), "process_block")
    return q, err


def _lazy_update(W, Hinv, errors, start, end):
    """The lazy batch update behind a block or a run of blocks (reference ``gptq.py:204-205``):
    ``W[end:] -= Hinv[end:, start:end] @ errors`` in place, ``errors`` ``[end - start, N]`` fp32; returns ``W``."""
    lib = N.load()
    K, Nc = W.shape
    if not (0 <= start <= end <= K) or tuple(errors.shape) != (end - start, Nc):
        raise ValueError("block out of range")
    if W.dtype != torch.float32 or Hinv.dtype != torch.float32 or errors.dtype != torch.float32 \
            or not (W.is_contiguous() and Hinv.is_contiguous() and errors.is_contiguous()):
        raise ValueError("fp32, contiguous operands")
    if end < K and end > start:
        below, panel = W[end:], Hinv[end:, start:]
        N.check(lib.gptq_hip_lazy_update(_stream(), ctypes.c_void_p(below.data_ptr()), Nc,
                                         ctypes.c_void_p(panel.data_ptr()), Hinv.shape[1], _ptr(errors),
                                         K - end, end - start), "lazy_update")
    return W


def _solve(W, L, params, block_size, out_dtype, want_codes=False):
    lib = N.load()
    K, Nc = W.shape
    Q = torch.empty((K, Nc), dtype=out_dtype, device=W.device)
    codes = torch.empty((K, Nc), dtype=torch.uint8, device=W.device) if want_codes else None
    ws = _ws(lib.gptq_hip_solve_workspace_bytes(K, Nc, block_size))
    N.check(lib.gptq_hip_solve(_stream(), _ptr(W), K, Nc, _ptr(L), _ptr(params["scale"]),
                               _ptr(params["zero"]), int(params["maxq"]), block_size, _ptr(Q),
                               _DT[out_dtype], _ptr(codes), _ptr(ws), ws.numel()), "solve")
    return Q, codes


def _solve_grouped(W, L, bits, group_size, block_size, out_dtype):
    """The column loop with one scale / zero per channel and group of ``group_size`` input features."""
    lib = N.load()
    K, Nc = W.shape
    Q = torch.empty((K, Nc), dtype=out_dtype, device=W.device)
    scale = torch.empty((K // group_size, Nc), dtype=torch.float32, device=W.device)
    zero = torch.empty((K // group_size, Nc), dtype=torch.float32, device=W.device)
    ws = _ws(lib.gptq_hip_solve_grouped_workspace_bytes(K, Nc, block_size, group_size))
    N.check(lib.gptq_hip_solve_grouped(_stream(), _ptr(W), K, Nc, _ptr(L), group_size, bits, block_size, _ptr(Q),
                                       _DT[out_dtype], _ptr(None), _ptr(scale), _ptr(zero), _ptr(ws), ws.numel()),
            "solve_grouped")
    return Q, {"maxq": 2 ** bits - 1, "scale": scale, "zero": zero, "group_size": group_size}


def gptq(W, xs, block_size=128, actorder=False, damping=0.01, use_fp64=False, H=None, shared=None,
         bits=4, split_fp16=False, group_size=None):
    """The per-layer GPTQ solve (reference ``gptq.py:182-212``).

    ``W`` is ``[K, N]`` (input features x output channels), ``xs`` a list of calibration
    batches ``[..., K]``.  Returns ``(Q, params)``: ``Q`` the dequantised matrix in ``W``'s
    dtype, ``params`` with ``scale`` / ``zero`` (fp32, one per column) and ``maxq``.

    Not in the reference, for callers that solve several matrices against the same activations
    (q / k / v of an attention block): ``H`` is the result of ``accumulate_H(xs, use_fp64)`` when
    the caller already has it (left untouched); ``shared`` is a dict that this function fills and
    reads across such calls: the Hessian, and, without ``actorder``, the factor of its damped
    inverse, which depends on ``xs`` and ``damping`` only.  The results are those of independent
    calls.  ``bits`` (1 to 8; the reference's ``gptq`` is fixed at the default of its
    ``get_quantize_params``, 4): the code width, ``maxq = 2**bits - 1``; ``pack_matrix`` stores
    4-bit results two per byte and 8-bit results one per byte.  ``split_fp16``: see
    ``accumulate_H``.  ``group_size`` (not in the reference): one scale / zero per output channel and group of
    ``group_size`` consecutive input features instead of one per channel; a group's parameters are the min-max
    parameters of its rows as they stand when the column loop reaches them.  ``params['scale']`` /
    ``['zero']`` are then ``[K / group_size, N]`` and ``params['group_size']`` is set.  Must be a multiple of
    ``block_size`` that divides ``K`` and 512; not combinable with ``actorder`` (the permutation would scatter a
    group's rows).
    """
    if group_size:
        group_size = int(group_size)
        if actorder:
            raise ValueError("group_size and actorder cannot be combined")
        if group_size % block_size or 512 % group_size or _float_dev(W).shape[0] % group_size:
            raise ValueError(f"group_size={group_size} must be a multiple of block_size={block_size} "
                             "that divides K and 512")
    Wt = _float_dev(W)
    if Wt.dim() != 2:
        raise ValueError("W must be a 2-D matrix [K, N]")
    orig_type = Wt.dtype
    K, Nc = Wt.shape
    if block_size < 1 or block_size > 128 or K % block_size != 0:
        raise ValueError(f"block_size={block_size} must divide K={K} and be at most 128")
    W32 = _to_f32_copy(Wt)            # the loop consumes its working copy
    if not 1 <= int(bits) <= 8:
        raise ValueError("bits must be between 1 and 8")
    quantize_params = get_col_quantize_params(W32, bits=int(bits))
    if H is None and shared is not None:
        H = shared.get("H")
    keep = H is not None or shared is not None      # somebody else still needs H as accumulated
    if H is None:
        H = accumulate_H(xs, use_fp64=use_fp64, split_fp16=split_fp16 and not use_fp64)
    if not isinstance(H, torch.Tensor):
        H = _dev(H)
    if H.dim() != 2 or H.shape[0] != H.shape[1] or H.dtype != (torch.float64 if use_fp64 else torch.float32):
        raise ValueError("H must be the square matrix accumulate_H(xs, use_fp64) returns")
    if H.shape[0] != K:
        raise ValueError(f"calibration feature dim {H.shape[0]} != K={K}")
    # a caller's H may be a strided view (a corner of a larger matrix) or live elsewhere: the kernels
    # take a dense [K, K] matrix on the current device
    H = _dev(H)
    if H.data_ptr() % 16:
        H = H.clone()           # a dense view that starts mid-allocation: the kernels load 16 bytes at a time
    if shared is not None:
        shared["H"] = H

    perm = None
    factor_key = ("factor", float(damping))
    Hinv = shared.get(factor_key) if (shared is not None and not actorder) else None
    if Hinv is not None:
        # same H, same damping: same factor; what is left of _damp_and_invert is the zeroing of
        # the rows of dead features (gptq.py:157-159)
        lib = N.load()
        N.check(lib.gptq_hip_zero_dead_rows(_stream(), _ptr(H), _DT_H[H.dtype], K, _ptr(W32), Nc, Nc),
                "zero_dead_rows")
    if Hinv is None:
        Hw = _clone(H) if keep else H           # the factorisation rewrites the diagonal
        if actorder:
            W32, Hw, perm = _permute(W32, Hw)
        # _damp_and_invert (gptq.py:193) and the fp32 cast of the factor (gptq.py:197) in one call
        _, Hinv, status = _damp_invert(W32, Hw, damping, fix_dead=True, want_f32=True)
    else:
        status = None

    # The column loop is enqueued before the host reads the status word back, so that the GPU
    # does not sit idle while the host waits and then launches; with a NaN factor the loop
    # computes garbage that is thrown away by the exception below (gptq.py:194-196).
    if group_size:
        Q, quantize_params = _solve_grouped(W32, Hinv, int(bits), group_size, block_size, orig_type)
    else:
        Q, _ = _solve(W32, Hinv, quantize_params, block_size, orig_type)
    if perm is not None:
        Q = _unpermute(Q, perm)
    if status is not None:
        any_nan = bool(status[0].item() != 0)
        if any_nan:
            xs_nan = any(bool(torch.isnan(_float_dev(x)).any()) for x in xs)
            raise ValueError(f"NaN when computing Hinv. Features NaN?: {xs_nan}")
        if shared is not None and not actorder:
            shared[factor_key] = Hinv
    return Q, quantize_params


# ------------------------------------------------------------------------------- codec
def _view3(shape, axis):
    if axis < 0 or axis >= len(shape):
        raise ValueError(f"Axis {axis} is out of bounds for array of dimension {len(shape)}")
    outer = int(np.prod(shape[:axis], dtype=np.int64)) if axis > 0 else 1
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64)) if axis + 1 < len(shape) else 1
    return outer, int(shape[axis]), inner


def pack_along_axis(axis, w):
    """``byte[j] = c[2j] | c[2j+1] << 4`` along ``axis`` (reference ``gptq.py:237-249, 265-283``)."""
    lib = N.load()
    w = _dev(w)
    if w.dtype not in (torch.uint8, torch.int8, torch.int32, torch.int64):
        w = w.to(torch.int32)
    outer, alen, inner = _view3(w.shape, axis)
    if alen % 2:
        raise ValueError("the packed axis must have even length")
    shape = list(w.shape)
    shape[axis] = alen // 2
    out = torch.empty(shape, dtype=torch.uint8, device=w.device)
    N.check(lib.gptq_hip_pack_int4(_stream(), _ptr(w), w.element_size(), outer, alen, inner,
                                   _ptr(out)), "pack_int4")
    return out


def unpack_along_axis(axis, w):
    """Inverse of :func:`pack_along_axis` (reference ``gptq.py:251-263, 285-286``)."""
    lib = N.load()
    w = _dev(w, torch.uint8)
    outer, plen, inner = _view3(w.shape, axis)
    shape = list(w.shape)
    shape[axis] = plen * 2
    out = torch.empty(shape, dtype=torch.uint8, device=w.device)
    N.check(lib.gptq_hip_unpack_int4(_stream(), _ptr(w), outer, plen, inner, _ptr(out)),
            "unpack_int4")
    return out


def _pack(w_int):
    assert len(w_int.shape) == 1
    return pack_along_axis(0, w_int)


def _unpack(packed):
    assert len(packed.shape) == 1
    return unpack_along_axis(0, packed)


def pack_rowwise(w):
    return pack_along_axis(1, w)


def pack_colwise(w):
    return pack_along_axis(0, w)


def unpack_rowwise(w):
    return unpack_along_axis(1, w)


def unpack_colwise(w):
    return unpack_along_axis(0, w)


def pack_matrix(Q, params, contraction_axis=0):
    """Dequantised floats -> integer codes -> packed container (reference ``gptq.py:214-228``)."""
    lib = N.load()
    maxq = int(params.get("maxq", 15))
    if maxq not in (15, 255):
        raise NotImplementedError("4-bit codes are packed two per byte (gptq.py:241), 8-bit codes are stored "
                                  "one per byte; other widths have no packed form")
    bits = 4 if maxq == 15 else 8
    Qt = _float_dev(Q)
    scale = _dev(params["scale"])
    zero = _dev(params["zero"])
    group = int(params.get("group_size", 0) or 0)
    if group:
        if Qt.dim() != 2 or contraction_axis != 0:
            raise ValueError("grouped parameters need a 2-D matrix packed along axis 0")
        K, Nc = Qt.shape
        if K % group or group % 2 or tuple(scale.shape) != (K // group, Nc) or tuple(zero.shape) != (K // group, Nc):
            raise ValueError("scale/zero must be [K / group_size, N]")
        packed = torch.empty((K // 2 if bits == 4 else K, Nc), dtype=torch.uint8, device=Qt.device)
        scale32 = scale.to(torch.float32).contiguous()
        zero32 = zero.to(torch.float32).contiguous()
        N.check(lib.gptq_hip_quantize_pack_grouped(_stream(), _ptr(Qt), _DT[Qt.dtype], K, Nc, _ptr(scale32),
                                                   _ptr(zero32), group, bits, _ptr(packed)), "quantize_pack_grouped")
        return QuantizedMatrix(int_weight=packed, zero=zero, scale=scale, contraction_axis=0, bits=bits,
                               group_size=group)
    outer, alen, inner = _view3(Qt.shape, contraction_axis)
    if bits == 4 and alen % 2:
        raise ValueError("the contraction axis must have even length")
    if scale.numel() != outer * inner or zero.numel() != outer * inner:
        raise ValueError("scale/zero must have the shape of Q without the contraction axis")
    shape = list(Qt.shape)
    shape[contraction_axis] = alen // 2 if bits == 4 else alen
    packed = torch.empty(shape, dtype=torch.uint8, device=Qt.device)
    scale32 = scale.to(torch.float32).contiguous()     # kept alive across the launch
    zero32 = zero.to(torch.float32).contiguous()
    N.check(lib.gptq_hip_quantize_pack_bits(
        _stream(), _ptr(Qt), _DT[Qt.dtype], outer, alen, inner, _ptr(scale32), _ptr(zero32), bits,
        _ptr(packed)), "quantize_pack")
    return QuantizedMatrix(int_weight=packed, zero=zero, scale=scale,
                           contraction_axis=contraction_axis, bits=bits)


def unpack_matrix(weight):
    """Dense ``(code - zero) * scale`` in ``zero.dtype`` (reference ``gptq.py:230-235``)."""
    lib = N.load()
    iw = _dev(weight.int_weight, torch.uint8)
    zero = _float_dev(weight.zero)
    scale = _float_dev(weight.scale).to(zero.dtype)
    group = int(getattr(weight, "group_size", 0) or 0)
    if group:
        bits = int(getattr(weight, "bits", 4))
        R, C = iw.shape
        out = torch.empty((R * (8 // bits), C), dtype=zero.dtype, device=iw.device)
        N.check(lib.gptq_hip_dequant_grouped(_stream(), _ptr(iw), R, C, _ptr(zero), _ptr(scale), _DT[zero.dtype],
                                             group, bits, _ptr(out)), "dequant_grouped")
        return out
    outer, plen, inner = _view3(iw.shape, weight.contraction_axis)
    if zero.numel() != outer * inner or scale.numel() != outer * inner:
        raise ValueError("scale/zero must have the shape of the matrix without the contraction axis")
    bits = int(getattr(weight, "bits", 4))
    shape = list(iw.shape)
    shape[weight.contraction_axis] = plen * (8 // bits)
    out = torch.empty(shape, dtype=zero.dtype, device=iw.device)
    N.check(lib.gptq_hip_dequant_bits(_stream(), _ptr(iw), outer, plen, inner, _ptr(zero), _ptr(scale),
                                      _DT[zero.dtype], bits, _ptr(out)), "dequant")
    return out
