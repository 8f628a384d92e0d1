"""Pins the CPU oracle without executing the reference.

The reference ships no stored vectors; its own tests are closed forms, round
trips and self-consistency checks (tests.py:34-44, 140-156, 293-311;
test_kernel.py:24).  Those are restated here on NumPy-seeded inputs of the same
shapes, and each remaining oracle function is checked against an independent
formulation chosen so that a dropped term, a wrong index or a transposed operand
fails.
"""
import numpy as np
import pytest
import scipy.linalg

from oracle import gptq_oracle as O


# ----------------------------------------------------------------------------- params
def test_get_quantize_params_reference_vector():
    # reference tests.py:34-44: explicit 2x4 matrix
    w = np.asarray([[0.1, 0.2, 0.3, 0.4], [-0.1, -0.1, -0.1, -0.1]], dtype=np.float32)
    p = O.get_col_quantize_params(w)
    assert p["zero"].shape == p["scale"].shape == (4,)
    assert p["maxq"] == 15
    assert np.allclose(p["scale"], (w[0, :] - w[1, :]) / 15)
    # zero = rint(-xmin/scale): 0.1/(0.2/15) = 7.5 -> 8 (half-even), 0.1/(0.3/15)=5, ...
    assert np.array_equal(p["zero"], np.round(0.1 / ((w[0] + 0.1) / 15)).astype(np.float32))


def test_get_quantize_params_edge_cases():
    w = np.zeros((8, 3), dtype=np.float32)
    w[:, 1] = np.linspace(0.5, 2.0, 8)       # all-positive column: xmin==0 -> -1
    w[:, 2] = -np.linspace(0.5, 2.0, 8)      # all-negative column: xmax==0 -> +1
    p = O.get_col_quantize_params(w)
    f = np.float32
    # all-zero column: xmin=-1, xmax=+1; in fp32 1/fl(2/15) = 7.4999995 -> 7 (7.5 -> 8 only in exact arithmetic)
    assert p["scale"][0] == f(2) / f(15) and p["zero"][0] == 7
    assert p["scale"][1] == (f(2.0) - f(-1)) / f(15)
    assert p["zero"][1] == np.round(f(1) / p["scale"][1])
    assert p["scale"][2] == (f(1) - f(-2.0)) / f(15)
    assert p["zero"][2] == np.round(f(2.0) / p["scale"][2])
    # the per-column form is the vmap of the scalar form
    for n in range(3):
        q = O.get_quantize_params(w[:, n])
        assert q["scale"] == p["scale"][n] and q["zero"] == p["zero"][n]
    assert p["scale"].dtype == np.float32 and p["zero"].dtype == np.float32


# ----------------------------------------------------------------------------- Hessian
def test_accumulate_H_closed_form_fp64():
    # reference tests.py:293-311 (20 batches of 37x256, fp64)
    rng = np.random.default_rng(9876)
    xs = [rng.standard_normal((37, 256)) for _ in range(20)]
    n = sum(x.shape[0] for x in xs)
    manual = sum(x.T @ x for x in xs) / n
    got = O.accumulate_H(xs, use_fp64=True)
    assert got.dtype == np.float64
    assert np.allclose(manual, got, atol=1e-13, rtol=0)


def test_accumulate_H_nonzero_mean_and_3d_batches():
    rng = np.random.default_rng(1)
    xs = [rng.standard_normal((3, 11, 32)) + 5.0 for _ in range(4)] + [rng.standard_normal((7, 32)) - 2.0]
    flat = np.concatenate([x.reshape(-1, 32) for x in xs])
    got = O.accumulate_H(xs, use_fp64=True)
    assert np.allclose(got, flat.T @ flat / flat.shape[0], atol=1e-12, rtol=0)
    got32 = O.accumulate_H([x.astype(np.float32) for x in xs])
    assert got32.dtype == np.float32
    assert np.allclose(got32, flat.T @ flat / flat.shape[0], rtol=2e-5, atol=1e-4)


# ----------------------------------------------------------------------------- factor
def _spd(rng, k, n):
    x = rng.standard_normal((n, k))
    return x.T @ x / n


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-10), (np.float32, 2e-3)])
def test_cholesky_inv_is_lower_factor_of_inverse(dtype, tol):
    rng = np.random.default_rng(3)
    H = (_spd(rng, 96, 400) + 0.01 * np.eye(96)).astype(dtype)
    L = O.cholesky_inv(H)
    assert L.dtype == dtype
    assert np.array_equal(L, np.tril(L)) and np.all(np.diag(L) > 0)
    H64, L64 = H.astype(np.float64), L.astype(np.float64)
    assert np.abs(L64 @ L64.T @ H64 - np.eye(96)).max() < tol
    ref = scipy.linalg.cholesky(np.linalg.inv(H64), lower=True)
    assert np.abs(ref - L64).max() < tol * np.abs(ref).max() * 10


def test_damp_and_invert_dead_column_and_damping():
    rng = np.random.default_rng(4)
    X = rng.standard_normal((300, 40))
    X[:, 7] = 0.0
    H = X.T @ X / 300
    W = rng.standard_normal((40, 5))
    W2, L, bad = O.damp_and_invert(W, H, 0.01)
    assert not bad
    assert np.all(W2[7] == 0) and np.array_equal(np.delete(W2, 7, 0), np.delete(W, 7, 0))
    Hd = H.copy()
    Hd[7, 7] = 1.0
    Hd += 0.01 * np.mean(np.diag(Hd)) * np.eye(40)
    assert np.abs(L @ L.T @ Hd - np.eye(40)).max() < 1e-10
    # inputs are not modified
    assert H[7, 7] == 0 and not np.all(W[7] == 0)


def test_damp_and_invert_not_positive_definite_flags_nan():
    H = np.array([[1.0, 2.0], [2.0, 1.0]])
    _, L, bad = O.damp_and_invert(np.ones((2, 2)), H, 0.0)
    assert bad
    with pytest.raises(ValueError):
        O.gptq(np.ones((2, 2), np.float32), None, block_size=2, damping=0.0, _H=H.astype(np.float32))


# ----------------------------------------------------------------------------- quantize
def test_quantize_value_is_nearest_grid_point():
    rng = np.random.default_rng(5)
    scale = np.float32(0.037)
    for zero in (np.float32(0), np.float32(6), np.float32(15)):
        grid = scale * (np.arange(16, dtype=np.float32) - zero)
        v = rng.uniform(grid[0] - 0.2, grid[-1] + 0.2, 4000).astype(np.float32)
        got = O.quantize_value(zero, scale, 15, v)
        dist = np.abs(v[:, None].astype(np.float64) - grid[None, :].astype(np.float64))
        best = dist.min(axis=1)
        got_dist = np.abs(v.astype(np.float64) - got.astype(np.float64))
        assert np.all(np.isin(got, grid))
        assert np.all(got_dist <= best + 1e-6 * scale)
        assert np.array_equal(O.quantize_value(zero, scale, 15, got), got)   # idempotent


def test_quantize_value_ties_half_even():
    scale, zero = np.float32(1.0), np.float32(4.0)
    v = np.array([0.5, 1.5, 2.5, -0.5, -1.5], dtype=np.float32)
    assert np.array_equal(O.quantize_value(zero, scale, 15, v), np.array([0, 2, 2, -0, -2], np.float32))


# ----------------------------------------------------------------------------- column loop
def _textbook_obs(W, H, scale, zero, maxq=15):
    """GPTQ as written in the paper: explicit inverse Hessian, one row at a time,
    Gaussian elimination of the processed row.  Independent of the Cholesky form."""
    W = W.astype(np.float64).copy()
    Hinv = np.linalg.inv(H.astype(np.float64))
    K = W.shape[0]
    Q = np.zeros_like(W)
    for i in range(K):
        w = W[i]
        q = np.clip(np.round(w / scale) + zero, 0, maxq)
        Q[i] = scale * (q - zero)
        err = (w - Q[i]) / Hinv[i, i]
        W[i:] -= np.outer(Hinv[i:, i], err)
        Hinv = Hinv - np.outer(Hinv[:, i], Hinv[i, :]) / Hinv[i, i]
    return Q


def _problem(seed, K, N, n, correlated=True):
    rng = np.random.default_rng(seed)
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    X = rng.standard_normal((n, K))
    if correlated:
        X = X @ (np.eye(K) + 0.3 * rng.standard_normal((K, K)) / np.sqrt(K))
    return W, X.astype(np.float32)


@pytest.mark.parametrize("block_size", [4, 8, 32])
def test_gptq_equals_textbook_elimination_fp64(block_size):
    K, N = 32, 24
    W, X = _problem(11, K, N, 256)
    H = (X.astype(np.float64).T @ X.astype(np.float64)) / X.shape[0]
    p = O.get_col_quantize_params(W)
    Q, params = O.gptq(W.astype(np.float64), None, block_size=block_size, damping=0.01,
                       _loop_dtype=np.float64, _H=H)
    Hd = H + 0.01 * np.mean(np.diag(H)) * np.eye(K)
    ref = _textbook_obs(W, Hd, params["scale"].astype(np.float64), params["zero"].astype(np.float64))
    assert np.allclose(params["scale"], p["scale"]) and np.array_equal(params["zero"], p["zero"])
    # identical decisions: an fp64 tie within 1e-12 does not occur on this seed
    assert np.abs(Q - ref).max() < 1e-12


def test_gptq_blocked_equals_unblocked_fp32_codes():
    K, N = 64, 48
    W, X = _problem(12, K, N, 512)
    outs = []
    for bs in (64, 16, 4):
        Q, p = O.gptq(W, [X], block_size=bs)
        outs.append(O.codes_from_q(Q, p))
    for c in outs[1:]:
        diff = c.astype(int) - outs[0].astype(int)
        assert np.mean(diff != 0) < 0.01 and np.abs(diff).max() <= 1


def test_gptq_identity_hessian_is_round_to_nearest():
    K, N = 32, 20
    rng = np.random.default_rng(13)
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    H = (3.0 * np.eye(K)).astype(np.float32)
    Q, p = O.gptq(W, None, block_size=8, _H=H)
    rtn = O.quantize_value(p["zero"], p["scale"], 15, W)
    assert np.array_equal(Q, rtn)


def test_gptq_outputs_on_grid_and_beat_rtn():
    K, N = 64, 40
    W, X = _problem(14, K, N, 300)
    Q, p = O.gptq(W, [X[:150], X[150:]], block_size=16)
    assert Q.dtype == np.float32
    codes = np.round(Q / p["scale"] + p["zero"])
    assert codes.min() >= 0 and codes.max() <= 15
    assert np.array_equal((p["scale"] * (codes - p["zero"])).astype(np.float32), Q)
    rtn = O.quantize_value(p["zero"], p["scale"], 15, W)
    X64 = X.astype(np.float64)
    e_gptq = np.linalg.norm(X64 @ (W - Q)) / np.linalg.norm(X64 @ W)
    e_rtn = np.linalg.norm(X64 @ (W - rtn)) / np.linalg.norm(X64 @ W)
    assert e_gptq < e_rtn


def test_gptq_hessian_scale_invariance():
    K, N = 32, 16
    W, X = _problem(15, K, N, 200)
    H = (X.T @ X / 200).astype(np.float32)
    Q1, _ = O.gptq(W, None, block_size=8, _H=H)
    Q2, _ = O.gptq(W, None, block_size=8, _H=(4.0 * H).astype(np.float32))   # power of two: exact
    assert np.mean(Q1 != Q2) < 0.01


def test_gptq_keeps_original_dtype_fp16():
    K, N = 32, 16
    W, X = _problem(16, K, N, 200)
    Q, p = O.gptq(W.astype(np.float16), [X], block_size=16)
    assert Q.dtype == np.float16 and p["scale"].dtype == np.float32


def test_actorder_is_conjugation_by_permutation():
    K, N = 32, 12
    W, X = _problem(17, K, N, 200)
    X = X * np.linspace(0.5, 2.0, K, dtype=np.float32)[None, :]
    H = (X.T @ X / 200).astype(np.float32)
    Wp, Hp, perm = O.permute(W, H)
    assert np.all(np.diff(np.diag(Hp)) <= 0)
    assert np.array_equal(Hp, H[np.ix_(perm, perm)]) and np.array_equal(Wp, W[perm])
    assert np.array_equal(O.unpermute(Wp, perm), W)
    Qa, p = O.gptq(W, [X], block_size=8, actorder=True)
    Qb, _ = O.gptq(Wp, None, block_size=8, _H=Hp)
    # quantisation parameters are per column, so they commute with a row permutation
    assert np.array_equal(Qa, O.unpermute(Qb, perm))
    # already descending diag -> identity permutation
    _, _, perm2 = O.permute(Wp, Hp)
    assert np.array_equal(perm2, np.arange(K))


# ----------------------------------------------------------------------------- codec
def test_pack_bit_layout_closed_form():
    codes = np.array([1, 2, 3, 15, 0, 9], dtype=np.uint8)
    assert np.array_equal(O._pack(codes), np.array([0x21, 0xF3, 0x90], dtype=np.uint8))
    assert np.array_equal(O._unpack(np.array([0x21, 0xF3, 0x90], dtype=np.uint8)), codes)


def test_pack_colwise_roundtrip():
    # reference tests.py:140-145
    rng = np.random.default_rng(0)
    w = rng.integers(0, 16, (256, 64))
    packed = O.pack_colwise(w)
    assert packed.shape == (128, 64) and packed.dtype == np.uint8
    assert np.array_equal(packed, (w[0::2] | (w[1::2] << 4)).astype(np.uint8))
    assert np.array_equal(O.unpack_colwise(packed), w)
    pr = O.pack_rowwise(w)
    assert pr.shape == (256, 32) and np.array_equal(O.unpack_rowwise(pr), w)


def test_pack_along_axis_nd_and_errors():
    rng = np.random.default_rng(1)
    w = rng.integers(0, 16, (6, 4, 10)).astype(np.uint8)
    for axis in range(3):
        p = O.pack_along_axis(axis, w)
        exp_shape = list(w.shape)
        exp_shape[axis] //= 2
        assert p.shape == tuple(exp_shape)
        assert np.array_equal(O.unpack_along_axis(axis, p), w)
    with pytest.raises(ValueError):
        O.pack_along_axis(3, w)


def test_pack_matrix_roundtrip_exact():
    # reference tests.py:147-156: W 256x64 N(0,1), integer-valued calibration, block 4
    rng = np.random.default_rng(0)
    w = rng.standard_normal((256, 64)).astype(np.float32)
    xs = [rng.integers(0, 16, (32, 256)).astype(np.float32) for _ in range(4)]
    quantized, qparams = O.gptq(w, xs, block_size=4)
    packed = O.pack_matrix(quantized, qparams)
    assert packed.int_weight.shape == (128, 64) and packed.shape == (256, 64)
    assert packed.dtype == np.float32
    assert np.array_equal(O.unpack_matrix(packed), quantized)


# ----------------------------------------------------------------------------- matmul
@pytest.mark.parametrize("transpose", [False, True])
def test_quantized_matmul_equals_dense(transpose):
    rng = np.random.default_rng(2)
    K, N, M = 64, 48, 5
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    qm = O.QuantizedMatrix(O.pack_colwise(codes), rng.integers(0, 16, N).astype(np.float32),
                           rng.uniform(0.001, 0.01, N).astype(np.float32))
    dense = O.unpack_matrix(qm)
    x = rng.standard_normal((2, M, N if transpose else K)).astype(np.float32)
    out = O.quantized_matmul(x, qm, transpose_b=transpose)
    ref = x @ (dense.T if transpose else dense)
    assert out.shape == ref.shape and out.dtype == np.float32
    assert np.allclose(out, ref, atol=1e-2, rtol=1e-3)
    with pytest.raises(AssertionError):
        O.quantized_matmul(x[..., :-2], qm, transpose_b=transpose)


# ---------------------------------------------------------------------------- grouped parameters (extension)
def test_grouped_parameters_reduce_to_the_per_channel_solve_and_to_rtn():
    """The group_size extension has no counterpart in the reference; what pins its restatement:
    (i) one group spanning all of K is the per-channel solve, bit for bit; (ii) with H = c I nothing is
    corrected, so every group is plain round-to-nearest on the min-max grid of that group's rows of the
    ORIGINAL matrix (brute force below); (iii) every output lies on its group's grid."""
    rng = np.random.default_rng(5)
    K, N, g = 256, 12, 128
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    X = rng.standard_normal((700, K)).astype(np.float32)
    Q0, p0 = O.gptq(W, [X])
    Qk, pk = O.gptq(W, [X], _group_size=K)
    assert np.array_equal(Q0, Qk) and np.array_equal(pk["scale"][0], p0["scale"]) and pk["group_size"] == K
    # (ii) orthogonal calibration columns: H = c I exactly
    Hc = 3.0 * np.eye(K, dtype=np.float32)
    Qi, pi = O.gptq(W, None, _H=Hc, _group_size=g)
    assert pi["scale"].shape == (K // g, N)
    for gi in range(K // g):
        rows = W[gi * g:(gi + 1) * g]
        ref = O.get_col_quantize_params(rows)
        assert np.array_equal(pi["scale"][gi], ref["scale"]) and np.array_equal(pi["zero"][gi], ref["zero"])
        grid = ref["scale"][None, None, :] * (np.arange(16, dtype=np.float32)[None, :, None] - ref["zero"][None, None, :])
        nearest = np.take_along_axis(grid, np.abs(rows[:, None, :] - grid).argmin(1)[:, None, :], 1)[:, 0, :]
        got = Qi[gi * g:(gi + 1) * g]
        # ties aside (none with random data), round-to-nearest-even on the grid is the nearest grid point
        assert np.allclose(got, nearest, rtol=0, atol=1e-7)
    # (iii) on the grid, and a different result from the per-channel one
    Qg, pg = O.gptq(W, [X], _group_size=g)
    codes = Qg / np.repeat(pg["scale"], g, 0) + np.repeat(pg["zero"], g, 0)
    assert np.abs(codes - np.rint(codes)).max() < 1e-3 and codes.min() > -0.5 and codes.max() < 15.5
    assert not np.array_equal(Qg, Q0)
    packed = O.pack_matrix(Qg, pg)
    assert packed.group_size == g and np.array_equal(O.unpack_matrix(packed), Qg.astype(np.float32))
