"""JAX front-end over the XLA FFI handlers of ``csrc/jax_ffi.cc``: the reference's Python API
(``jax_gptq/gptq.py``, ``op.py``) on ``jax.Array`` operands, with every computation a custom call into
``libgptq_hip.so`` on XLA's stream (``jax.ffi.ffi_call``; the reference's one custom call is the
``jt.triton_call`` at ``op.py:46-63``).

Importing this module never needs JAX; using it does.  :func:`available` says whether JAX, its FFI
headers and the built shim (``libgptq_hip_jax.so``, see ``build.py``) are all there, and every public
function raises ``ImportError`` with the reason otherwise: there is no fallback to another backend.
The torch front-end (``gptq.py``, ``op.py``) binds the same C ABI through ctypes and is what runs where
JAX is not installed.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
SHIM_PATH = os.path.join(HERE, "libgptq_hip_jax.so")

# FFI target name -> handler symbol in the shim (one per XLA_FFI_DEFINE_HANDLER_SYMBOL of jax_ffi.cc)
TARGETS = {
    "gptq_col_params": "gptq_ffi_col_params",
    "gptq_hessian_accumulate": "gptq_ffi_hessian_accumulate",
    "gptq_hessian_finalize": "gptq_ffi_hessian_finalize",
    "gptq_damp_invert": "gptq_ffi_damp_invert",
    "gptq_zero_dead_rows": "gptq_ffi_zero_dead_rows",
    "gptq_solve": "gptq_ffi_solve",
    "gptq_process_block": "gptq_ffi_process_block",
    "gptq_gather_rows": "gptq_ffi_gather_rows",
    "gptq_gather_sym": "gptq_ffi_gather_sym",
    "gptq_pack_int4": "gptq_ffi_pack_int4",
    "gptq_unpack_int4": "gptq_ffi_unpack_int4",
    "gptq_quantize_pack": "gptq_ffi_quantize_pack",
    "gptq_dequant": "gptq_ffi_dequant",
    "gptq_qmatmul": "gptq_ffi_qmatmul",
}

_state = {"registered": False, "reason": None}


def _why_not():
    try:
        import jax  # noqa: F401
        import jax.ffi  # noqa: F401
    except Exception as e:  # ImportError, or an old JAX without jax.ffi
        return f"JAX with jax.ffi is not importable ({e})"
    if not os.path.exists(SHIM_PATH):
        return (f"{SHIM_PATH} is missing: run `python jax-gptq_amd/build.py --jax` on a machine whose JAX "
                "ships the XLA FFI headers (jax.ffi.include_dir())")
    return None


def available():
    """True when the JAX front-end can run here."""
    return _why_not() is None


def _register():
    if _state["registered"]:
        return
    reason = _why_not()
    if reason:
        raise ImportError("jax_gptq_amd.jax_frontend: " + reason)
    import jax
    from . import _native
    _native.load()                                   # the C ABI the shim forwards to (RTLD_GLOBAL not needed: linked)
    shim = ctypes.CDLL(SHIM_PATH)
    for target, symbol in TARGETS.items():
        jax.ffi.register_ffi_target(target, jax.ffi.pycapsule(getattr(shim, symbol)), platform="ROCM")
    _state["registered"] = True


def _lib():
    from . import _native
    return _native.load()


# ------------------------------------------------------------------------------- container
class QuantizedMatrix:
    """Reference ``gptq.py:8-32``: ``int_weight`` uint8, ``zero``, ``scale``, static ``contraction_axis``
    (and ``bits``, 4 as in the reference unless 8-bit parameters were packed); registered as a pytree."""

    def __init__(self, int_weight, zero, scale, contraction_axis=0, bits=4):
        self.int_weight, self.zero, self.scale = int_weight, zero, scale
        self.contraction_axis, self.bits = contraction_axis, bits

    @property
    def shape(self):
        shape = list(self.int_weight.shape)
        shape[self.contraction_axis] *= 8 // self.bits
        return tuple(shape)

    @property
    def dtype(self):
        return self.zero.dtype

    def tree_flatten(self):
        return (self.int_weight, self.zero, self.scale), (self.contraction_axis, self.bits)

    @classmethod
    def tree_unflatten(cls, aux, children):
        return cls(*children, contraction_axis=aux[0], bits=aux[1])


def _register_pytree():
    import jax
    try:
        jax.tree_util.register_pytree_node_class(QuantizedMatrix)
    except ValueError:
        pass                                          # already registered


# ------------------------------------------------------------------------------- helpers
def _view3(shape, axis):
    import math
    if axis < 0 or axis >= len(shape):
        raise ValueError(f"Axis {axis} is out of bounds for array of dimension {len(shape)}")
    return math.prod(shape[:axis]), int(shape[axis]), math.prod(shape[axis + 1:])


def _call(target, out_types, *args, aliases=None, **attrs):
    import jax
    _register()
    return jax.ffi.ffi_call(target, out_types, input_output_aliases=aliases or {})(*args, **attrs)


# ------------------------------------------------------------------------------- gptq.py
def get_col_quantize_params(weight, bits=4):
    """Reference ``gptq.py:105-118``."""
    import jax
    import jax.numpy as jnp
    import numpy as np
    n = weight.shape[1]
    t = jax.ShapeDtypeStruct((n,), jnp.float32)
    scale, zero = _call("gptq_col_params", (t, t), weight, bits=np.int64(bits))
    return {"maxq": 2 ** bits - 1, "scale": scale, "zero": zero}


def accumulate_H(xs, use_fp64=False):
    """Reference ``gptq.py:76-103``: all batches in one custom call, then the division by ``n``."""
    import jax
    import jax.numpy as jnp
    import numpy as np
    K = xs[0].shape[-1]
    dt = jnp.float64 if use_fp64 else jnp.float32
    H = jnp.zeros((K, K), dt)
    t = jax.ShapeDtypeStruct((K, K), dt)
    H = _call("gptq_hessian_accumulate", t, H, *xs, aliases={0: 0})
    n = sum(int(np.prod(x.shape[:-1])) for x in xs)
    return _call("gptq_hessian_finalize", t, H, aliases={0: 0}, n_samples=np.float64(n))


def gptq(W, xs, block_size=128, actorder=False, damping=0.01, use_fp64=False, bits=4):
    """Reference ``gptq.py:182-212``: returns ``(Q, {'scale', 'zero', 'maxq'})``."""
    import jax
    import jax.numpy as jnp
    import numpy as np
    K, N = W.shape
    if K % block_size or block_size > 128:
        raise ValueError(f"block_size={block_size} must divide K={K} and be at most 128")
    orig = W.dtype
    W32 = W.astype(jnp.float32)
    params = get_col_quantize_params(W32, bits=bits)
    H = accumulate_H(xs, use_fp64=use_fp64)
    perm = None
    if actorder:
        perm = jnp.argsort(jnp.diag(H), stable=True)[::-1].astype(jnp.int64)
        W32 = _call("gptq_gather_rows", jax.ShapeDtypeStruct(W32.shape, W32.dtype), W32, perm)
        H = _call("gptq_gather_sym", jax.ShapeDtypeStruct(H.shape, H.dtype), H, perm)
    f32 = lambda s: jax.ShapeDtypeStruct(s, jnp.float32)   # noqa: E731
    l32_shape = (K, K) if use_fp64 else (0,)
    H, W32, L, L32, status = _call(
        "gptq_damp_invert",
        (jax.ShapeDtypeStruct(H.shape, H.dtype), f32((K, N)), jax.ShapeDtypeStruct(H.shape, H.dtype),
         f32(l32_shape), jax.ShapeDtypeStruct((2,), jnp.int32)),
        H, W32, aliases={0: 0, 1: 1}, damping=np.float64(damping), fix_dead=True)
    Lf = L32 if use_fp64 else L
    Q, _codes, _ = _call(
        "gptq_solve", (jax.ShapeDtypeStruct((K, N), orig), jax.ShapeDtypeStruct((K, N), jnp.uint8), f32((K, N))),
        W32, Lf, params["scale"], params["zero"], aliases={0: 2}, maxq=np.int64(params["maxq"]),
        block_size=np.int64(block_size))
    if int(status[0]) != 0:
        xs_nan = any(bool(jnp.isnan(x).any()) for x in xs)
        raise ValueError(f"NaN when computing Hinv. Features NaN?: {xs_nan}")
    if perm is not None:
        inv = jnp.argsort(perm, stable=True).astype(jnp.int64)
        Q = _call("gptq_gather_rows", jax.ShapeDtypeStruct(Q.shape, Q.dtype), Q, inv)
    return Q, params


def pack_matrix(Q, params, contraction_axis=0):
    """Reference ``gptq.py:214-228`` (8-bit parameters: one code per byte)."""
    import jax
    import jax.numpy as jnp
    import numpy as np
    maxq = int(params.get("maxq", 15))
    if maxq not in (15, 255):
        raise NotImplementedError("only 4-bit and 8-bit codes have a packed form")
    bits = 4 if maxq == 15 else 8
    outer, alen, inner = _view3(Q.shape, contraction_axis)
    shape = list(Q.shape)
    shape[contraction_axis] = alen // 2 if bits == 4 else alen
    packed = _call("gptq_quantize_pack", jax.ShapeDtypeStruct(tuple(shape), jnp.uint8), Q,
                   params["scale"].astype(jnp.float32), params["zero"].astype(jnp.float32),
                   outer=np.int64(outer), axis_len=np.int64(alen), inner=np.int64(inner), bits=np.int64(bits))
    return QuantizedMatrix(packed, params["zero"], params["scale"], contraction_axis, bits)


def unpack_matrix(weight):
    """Reference ``gptq.py:230-235``."""
    import jax
    import numpy as np
    outer, plen, inner = _view3(weight.int_weight.shape, weight.contraction_axis)
    zero = weight.zero
    return _call("gptq_dequant", jax.ShapeDtypeStruct(weight.shape, zero.dtype), weight.int_weight, zero,
                 weight.scale.astype(zero.dtype), outer=np.int64(outer), packed_axis_len=np.int64(plen),
                 inner=np.int64(inner), bits=np.int64(weight.bits))


# ------------------------------------------------------------------------------- op.py
_WS = {}


def _workspace(nbytes):
    """Zero-filled workspace, kept and only ever grown: every call leaves its arrival counters zero."""
    import jax.numpy as jnp
    ws = _WS.get("ws")
    if ws is None or ws.shape[0] < nbytes:
        ws = jnp.zeros((max(int(nbytes), 256),), jnp.uint8)
    return ws


def _quantized_matmul(x, quantized_matrix, transpose_b):
    import jax
    import jax.numpy as jnp
    import numpy as np
    lead = None
    if x.ndim > 2:
        lead, x = x.shape[:-1], x.reshape(-1, x.shape[-1])
    w = quantized_matrix.int_weight
    if w.ndim != 2 or quantized_matrix.contraction_axis != 0:
        raise ValueError("quantized_matmul needs a 2-D packed matrix with contraction_axis == 0")
    R, C = w.shape
    bits = quantized_matrix.bits
    Kw = R * (8 // bits)
    out_n = Kw if transpose_b else C
    assert x.shape[1] == (C if transpose_b else Kw), "Inner dim mismatch"
    code = {jnp.dtype("float32"): 0, jnp.dtype("float16"): 1, jnp.dtype("bfloat16"): 2}[jnp.dtype(x.dtype)]
    need = _lib().gptq_hip_qmatmul_bits_workspace_bytes(x.shape[0], R, C, int(transpose_b), code, bits)
    ws = _workspace(need)
    out, ws = _call("gptq_qmatmul",
                    (jax.ShapeDtypeStruct((x.shape[0], out_n), x.dtype), jax.ShapeDtypeStruct(ws.shape, ws.dtype)),
                    x, w, quantized_matrix.zero, quantized_matrix.scale.astype(quantized_matrix.zero.dtype), ws,
                    aliases={4: 1}, transpose_b=bool(transpose_b), bits=np.int64(bits))
    _WS["ws"] = ws
    return out.reshape(lead + (out_n,)) if lead is not None else out


def quantized_matmul(x, quantized_matrix, transpose_b=False):
    """Reference ``op.py:11-14`` with its ``custom_vjp`` (``op.py:71-81``): differentiable in ``x``; the
    cotangent of the packed matrix is ``None``."""
    import jax
    _register_pytree()

    @jax.custom_vjp
    def f(x_, qm):
        return _quantized_matmul(x_, qm, transpose_b)

    def fwd(x_, qm):
        return _quantized_matmul(x_, qm, transpose_b), qm

    def bwd(qm, y_bar):
        return _quantized_matmul(y_bar, qm, not transpose_b), None

    f.defvjp(fwd, bwd)
    return f(x, quantized_matrix)
