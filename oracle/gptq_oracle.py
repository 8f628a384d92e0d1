"""CPU oracle for the per-layer GPTQ solve and its packed-int4 consumer.

TEST INFRASTRUCTURE ONLY.  This module is a NumPy/SciPy restatement of the
algorithm in the reference's ``jax_gptq/gptq.py`` and ``jax_gptq/op.py``.  It is
the checker that the HIP path is compared with; nothing in the shipped package
imports it.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  Operation order and dtypes follow the reference statement
for statement, because the solve has rounding decisions (``rint``) downstream of
almost every floating-point operation.

What pins each function (all of it runs on the CPU, in ``tests/test_oracle_*``):

* ``get_quantize_params`` / ``get_col_quantize_params``: the explicit 2x4 vector
  of the reference's ``tests.py:34-44``; closed forms for an all-positive and an
  all-zero column.
* ``accumulate_H``: closed form ``sum(x.T @ x) / n`` in fp64 (``tests.py:293-311``).
* ``cholesky_inv`` / ``damp_and_invert``: ``L @ L.T @ H == I``, lower triangular,
  positive diagonal, equality with ``scipy.linalg.cholesky(inv(H), lower=True)``;
  dead-column special case.
* ``quantize_value``: brute force over the 16 grid points.
* ``process_block`` / ``gptq``: equality with a textbook OBS elimination that keeps
  an explicit inverse Hessian (written independently in the tests), blocked ==
  unblocked, ``H = c*I`` reduces to round-to-nearest, outputs lie on the grid.
* ``permute`` / ``unpermute``: conjugation by a permutation; identity when
  ``diag(H)`` is already descending.
* ``_pack`` / ``_unpack`` / ``pack_matrix`` / ``unpack_matrix``: closed-form bit
  layout and exact round trip (``tests.py:140-156``).
* ``quantized_matmul``: ``x @ unpack_matrix(W)`` (``test_kernel.py:24``).

Parity unpinned at the bit level (no reference fixture exists and the reference
cannot be executed here, ``jax`` being absent): the tie-breaking of XLA's own
fp32 GEMM/LAPACK inside ``accumulate_H``, ``cholesky_inv`` and the lazy update of
``gptq``.  The semantics of those functions are pinned by the checks above.
"""
from __future__ import annotations

import numpy as np
import scipy.linalg

__all__ = [
    "QuantizedMatrix", "quant_matrix_shape", "cholesky_inv", "accumulate_H_step",
    "accumulate_H", "get_quantize_params", "get_col_quantize_params",
    "quantize_value", "batch_quantize", "process_block", "damp_and_invert",
    "permute", "unpermute", "gptq", "pack_matrix", "unpack_matrix", "_pack",
    "_unpack", "pack_along_axis", "unpack_along_axis", "pack_rowwise",
    "pack_colwise", "unpack_rowwise", "unpack_colwise", "quantized_matmul",
    "codes_from_q",
]


class QuantizedMatrix:
    """Container of a packed matrix (reference ``gptq.py:8-22``)."""

    def __init__(self, int_weight, zero, scale, contraction_axis=0, bits=4, group_size=0):
        self.group_size = group_size   # > 0 (an extension): zero / scale are [K / group_size, N] tables
        self.int_weight = int_weight
        self.zero = zero
        self.scale = scale
        self.contraction_axis = contraction_axis
        self.bits = bits        # 8 (an extension; the reference packs 4-bit codes only): one code per byte

    @property
    def shape(self):
        return quant_matrix_shape(self)

    @property
    def dtype(self):
        return self.zero.dtype


def quant_matrix_shape(quantized_matrix, bits=None):
    """Logical shape of a packed matrix (reference ``gptq.py:34-42``)."""
    if bits is None:
        bits = getattr(quantized_matrix, "bits", 4)
    mat = quantized_matrix.int_weight
    ele_width = mat.dtype.itemsize * 8
    shape = list(mat.shape)
    shape[quantized_matrix.contraction_axis] *= ele_width // bits
    return tuple(shape)


def cholesky_inv(mat):
    """Lower Cholesky factor of ``inv(mat)`` (reference ``gptq.py:44-48``).

    ``cho_factor`` -> ``cho_solve`` against the identity -> ``cholesky`` of the
    symmetrised inverse (``jnp.linalg.cholesky`` symmetrises its input), all in
    ``mat.dtype``.
    """
    dtype = mat.dtype
    try:
        cho, lower = scipy.linalg.cho_factor(mat, lower=False, check_finite=False)
        hinv = scipy.linalg.cho_solve((cho, lower), np.eye(mat.shape[0], dtype=dtype),
                                      check_finite=False).astype(dtype, copy=False)
        hinv = (hinv + hinv.T) / dtype.type(2)
        out = np.linalg.cholesky(hinv)
    except np.linalg.LinAlgError:
        # XLA's factorisations return NaNs instead of raising; the caller (gptq)
        # turns them into ValueError (reference gptq.py:194-196).
        out = np.full(mat.shape, np.nan, dtype=dtype)
    return out.astype(dtype, copy=False)


def accumulate_H_step(H, running_mean, n_samples, batch):
    """One running-mean update (reference ``gptq.py:57-74``)."""
    if batch.ndim > 2:
        batch = batch.reshape(-1, batch.shape[-1])
    dtype = H.dtype
    batch_size = batch.shape[0]
    new_n_samples = dtype.type(n_samples + dtype.type(batch_size))
    batch = batch.astype(dtype)
    new_mean = running_mean + np.sum(batch - running_mean, axis=0, dtype=dtype) / new_n_samples
    x_val = batch - running_mean
    y_val = batch - new_mean
    H = H + x_val.T @ y_val
    return H, new_mean.astype(dtype), new_n_samples


def accumulate_H(xs, use_fp64=False):
    """``H = sum_b X_b^T X_b / n`` by the reference's running-mean scheme (``gptq.py:76-103``)."""
    dtype = np.dtype(np.float64 if use_fp64 else np.float32)
    dim = xs[0].shape[-1]
    H = np.zeros((dim, dim), dtype=dtype)
    n_samples = dtype.type(0)
    running_mean = np.zeros(dim, dtype=dtype)
    for batch in xs:
        H, running_mean, n_samples = accumulate_H_step(H, running_mean, n_samples, np.asarray(batch))
    H = H / n_samples
    H = H + np.outer(running_mean, running_mean)
    return H.astype(dtype, copy=False)


def get_quantize_params(weight, bits=4):
    """Asymmetric min-max parameters of one channel (reference ``gptq.py:105-116``)."""
    weight = np.asarray(weight)
    dtype = weight.dtype
    maxq = 2 ** bits - 1
    xmin = np.minimum(dtype.type(0), np.min(weight))
    xmax = np.maximum(dtype.type(0), np.max(weight))
    xmin = np.where(xmin == 0, dtype.type(-1), xmin)
    xmax = np.where(xmax == 0, dtype.type(1), xmax)
    scale = ((xmax - xmin) / dtype.type(maxq)).astype(dtype)
    zero = np.round(-xmin / scale).astype(dtype)
    return {"maxq": maxq, "scale": scale, "zero": zero}


def get_col_quantize_params(weight, bits=4):
    """Per-output-channel parameters: one (scale, zero) per column (``gptq.py:118``)."""
    weight = np.asarray(weight)
    dtype = weight.dtype
    maxq = 2 ** bits - 1
    xmin = np.minimum(dtype.type(0), weight.min(axis=0))
    xmax = np.maximum(dtype.type(0), weight.max(axis=0))
    xmin = np.where(xmin == 0, dtype.type(-1), xmin).astype(dtype)
    xmax = np.where(xmax == 0, dtype.type(1), xmax).astype(dtype)
    scale = ((xmax - xmin) / dtype.type(maxq)).astype(dtype)
    zero = np.round(-xmin / scale).astype(dtype)
    return {"maxq": maxq, "scale": scale, "zero": zero}


def quantize_value(zero, scale, maxq, value):
    """Round to the grid and return the DEQUANTISED value (reference ``gptq.py:120-126``)."""
    q = np.clip(np.round(value / scale) + zero, 0, maxq)
    return scale * (q - zero)


def batch_quantize(zero, scale, maxq, value):
    """Row-wise ``quantize_value`` with per-column parameters (``gptq.py:128``)."""
    return quantize_value(zero, scale, maxq, value)


def process_block(W, Hinv, start, quantize_params, block_size):
    """Quantise ``block_size`` rows with error feedback (reference ``gptq.py:130-153``).

    Returns ``(q_block, errors)``, both ``[block_size, N]`` in ``W.dtype``.
    """
    block = np.array(W[start:start + block_size, :], copy=True)
    h_block = Hinv[start:start + block_size, start:start + block_size]
    zero, scale, maxq = quantize_params["zero"], quantize_params["scale"], quantize_params["maxq"]
    q_block = np.empty_like(block)
    errors = np.empty_like(block)
    for i in range(block.shape[0]):
        w = block[i, :].copy()
        d = h_block[i, i]
        q = batch_quantize(zero, scale, maxq, w).astype(block.dtype)
        q_block[i] = q
        error = ((w - q) / d).astype(block.dtype)
        errors[i] = error
        update = (h_block[i:, i:i + 1] * error[None, :]).astype(block.dtype)
        block[i:, :] -= update
    return q_block, errors


def damp_and_invert(W, H, damping):
    """Dead-feature fix, relative damping, factor of the inverse (``gptq.py:155-168``)."""
    dtype = H.dtype
    H = np.array(H, copy=True)
    W = np.array(W, copy=True)
    dead = np.diag(H) == 0
    idx = np.arange(H.shape[0])
    H[idx[dead], idx[dead]] = 1
    W[dead, :] = 0
    mean_diag = np.mean(np.diag(H), dtype=dtype)
    H[idx, idx] += dtype.type(mean_diag * dtype.type(damping))
    Hinv = cholesky_inv(H)
    any_nan = bool(np.any(np.isnan(Hinv)))
    return W, Hinv, any_nan


def permute(W, H):
    """Activation-order permutation (reference ``gptq.py:170-175``)."""
    perm = np.argsort(np.diag(H), kind="stable")[::-1]
    return W[perm, :], H[perm][:, perm], perm


def unpermute(Q, perm):
    """Inverse of ``permute`` on the quantised rows (``gptq.py:177-180``)."""
    return Q[np.argsort(perm, kind="stable"), :]


def gptq(W, xs, block_size=128, actorder=False, damping=0.01, use_fp64=False,
         _loop_dtype=np.float32, _H=None, _bits=4, _group_size=0):
    """The per-layer solve (reference ``gptq.py:182-212``).

    Returns ``(Q, params)``: ``Q`` is the DEQUANTISED matrix in ``W``'s dtype and
    ``params`` holds ``scale``, ``zero`` (fp32, one per column) and ``maxq``.

    ``_loop_dtype``, ``_H`` and ``_bits`` are test hooks only: the reference always runs the
    column loop in fp32 (``gptq.py:184,197``), always builds ``H`` from ``xs`` and always takes
    the default width of ``get_quantize_params`` (4 bits, ``gptq.py:105,185``).

    ``_group_size`` (an extension with no counterpart in the reference, stated here as the specification
    the HIP path is checked against): when the loop reaches a row ``r0`` that is a multiple of it, the
    parameters of rows ``[r0, r0 + group)`` are ``get_col_quantize_params`` of those rows of the working
    matrix as they then stand (every correction of the rows above applied); ``scale`` / ``zero`` come back
    as ``[K / group, N]``.  Must be a multiple of ``block_size``.
    """
    W = np.asarray(W)
    orig_type = W.dtype
    loop_dtype = np.dtype(_loop_dtype)
    W = W.astype(loop_dtype)
    quantize_params = get_col_quantize_params(W, bits=_bits)
    H = accumulate_H(xs, use_fp64=use_fp64) if _H is None else np.asarray(_H)

    perm = None
    if actorder:
        W, H, perm = permute(W, H)

    W, Hinv, any_nan = damp_and_invert(W, H, damping)
    if any_nan:
        raise ValueError("NaN when computing Hinv.")
    Hinv = Hinv.astype(loop_dtype)

    K = W.shape[0]
    blocks = []
    group_scale, group_zero = [], []
    for start in range(0, K, block_size):
        end = start + block_size
        if _group_size and start % _group_size == 0:
            quantize_params = get_col_quantize_params(W[start:start + _group_size], bits=_bits)
            group_scale.append(quantize_params["scale"])
            group_zero.append(quantize_params["zero"])
        q_block, errors = process_block(W, Hinv, start, quantize_params, block_size)
        if end < K:
            update = (Hinv[end:, start:end] @ errors).astype(W.dtype)
            W[end:, :] -= update
        blocks.append(q_block)

    Q = np.concatenate(blocks, axis=0).astype(orig_type)
    if perm is not None:
        Q = unpermute(Q, perm)
    if _group_size:
        quantize_params = {"maxq": quantize_params["maxq"], "scale": np.stack(group_scale),
                           "zero": np.stack(group_zero), "group_size": _group_size}
    return Q, quantize_params


def codes_from_q(Q, params, contraction_axis=0):
    """Integer codes of a dequantised matrix (first line of ``pack_matrix``, ``gptq.py:221``)."""
    group = int(params.get("group_size", 0) or 0)
    if group:      # [K / group, N] tables of a 2-D matrix: every row takes its group's row
        scale = np.repeat(np.asarray(params["scale"]), group, axis=0)
        zero = np.repeat(np.asarray(params["zero"]), group, axis=0)
    else:
        scale = np.expand_dims(np.asarray(params["scale"]), axis=contraction_axis)
        zero = np.expand_dims(np.asarray(params["zero"]), axis=contraction_axis)
    return np.round(np.asarray(Q) / scale + zero).astype(np.uint8)


def pack_matrix(Q, params, contraction_axis=0):
    """Floats -> codes -> nibble-packed container (reference ``gptq.py:214-228``)."""
    int_matrix = codes_from_q(Q, params, contraction_axis)
    bits = 8 if int(params.get("maxq", 15)) == 255 else 4
    # 8-bit codes (not in the reference) are the uint8 matrix itself
    packed = pack_along_axis(contraction_axis, int_matrix) if bits == 4 else int_matrix
    return QuantizedMatrix(int_weight=packed, zero=np.asarray(params["zero"]),
                           scale=np.asarray(params["scale"]), contraction_axis=contraction_axis, bits=bits,
                           group_size=int(params.get("group_size", 0) or 0))


def unpack_matrix(weight):
    """Dense ``(code - zero) * scale`` (reference ``gptq.py:230-235``)."""
    group = getattr(weight, "group_size", 0)
    if group:
        zero, scale = np.repeat(weight.zero, group, axis=0), np.repeat(weight.scale, group, axis=0)
    else:
        zero = np.expand_dims(weight.zero, axis=weight.contraction_axis)
        scale = np.expand_dims(weight.scale, axis=weight.contraction_axis)
    unpacked = (unpack_along_axis(weight.contraction_axis, weight.int_weight)
                if getattr(weight, "bits", 4) == 4 else np.asarray(weight.int_weight))
    return (unpacked.astype(zero.dtype) - zero) * scale


def _pack(w_int):
    """1-D: ``byte[j] = c[2j] | c[2j+1] << 4`` (reference ``gptq.py:237-249``)."""
    assert w_int.ndim == 1
    w_int = np.asarray(w_int)
    lo = w_int[0::2].astype(np.uint8)
    hi = (w_int[1::2] << 4).astype(np.uint8)
    return lo | hi


def _unpack(packed):
    """1-D inverse of ``_pack`` (reference ``gptq.py:251-263``)."""
    assert packed.ndim == 1
    out = np.zeros(packed.shape[0] * 2, dtype=np.uint8)
    out[0::2] = packed & 0xF
    out[1::2] = (packed >> 4) & 0xF
    return out


def pack_along_axis(axis, w):
    """Apply ``_pack`` along one axis of an N-D array (``gptq.py:265-283``)."""
    w = np.asarray(w)
    if axis >= w.ndim:
        raise ValueError(f"Axis {axis} is out of bounds for array of dimension {w.ndim}")
    return np.apply_along_axis(_pack, axis, w)


def unpack_along_axis(axis, w):
    """Apply ``_unpack`` along one axis of an N-D array (``gptq.py:265-286``)."""
    w = np.asarray(w)
    if axis >= w.ndim:
        raise ValueError(f"Axis {axis} is out of bounds for array of dimension {w.ndim}")
    return np.apply_along_axis(_unpack, axis, w)


def pack_rowwise(w):
    return pack_along_axis(1, w)


def pack_colwise(w):
    return pack_along_axis(0, w)


def unpack_rowwise(w):
    return unpack_along_axis(1, w)


def unpack_colwise(w):
    return unpack_along_axis(0, w)


def quantized_matmul(x, quantized_matrix, transpose_b=False):
    """``x @ dequant(W)`` (or ``@ dequant(W).T``), fp32 accumulate, fp16 result cast
    back to ``x.dtype`` (reference ``op.py:19-69``, ``kernel.py:73-111`` and ``:194-253``)."""
    x = np.asarray(x)
    lead = None
    if x.ndim > 2:
        lead = x.shape[:-1]
        x = x.reshape(-1, x.shape[-1])
    w = quantized_matrix.int_weight
    bits = getattr(quantized_matrix, "bits", 4)
    codes = (unpack_along_axis(0, w) if bits == 4 else np.asarray(w)).astype(np.float32)
    group = getattr(quantized_matrix, "group_size", 0)
    if group:
        dense = (codes - np.repeat(quantized_matrix.zero.astype(np.float32), group, axis=0)) * \
            np.repeat(quantized_matrix.scale.astype(np.float32), group, axis=0)
    else:
        dense = (codes - quantized_matrix.zero.astype(np.float32)[None, :]) * \
            quantized_matrix.scale.astype(np.float32)[None, :]
    K = x.shape[1]
    if transpose_b:
        assert K == w.shape[1], f"Inner dim mismatch: {K} != {w.shape[1]}"
        out = x.astype(np.float32) @ dense.T
    else:
        assert K == codes.shape[0], f"Inner dim mismatch: {K} != {codes.shape[0]}"
        out = x.astype(np.float32) @ dense
    out = out.astype(np.float16)
    if lead is not None:
        out = out.reshape(lead + (out.shape[-1],))
    return out.astype(x.dtype)
