"""GPU parity of the blocked column loop and of the whole gptq() solve against the oracle.

Bars (from the task statement): scales / zeros within 1e-5 relative, at least 99.9 % of the
integer codes equal to the oracle's and the rest off by one, layer reconstruction error
within 1 % (relative) of the oracle's, packing bit-exact.
"""
import numpy as np
import pytest

from helpers import code_stats, recon_error, to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import jax_gptq_amd.gptq as g
    return g


def _problem(seed, K, N, n, wdtype=np.float32, correlated=False, wstd=0.02):
    rng = np.random.default_rng(seed)
    W = (wstd * rng.standard_normal((K, N))).astype(wdtype)
    X = rng.standard_normal((n, K))
    if correlated:
        X = X @ (np.eye(K) + 0.5 * rng.standard_normal((K, K)) / np.sqrt(K))
    return W, X.astype(np.float32)


@pytest.mark.parametrize("bs", [128, 64, 16, 8, 4, 2, 1, 24, 100])
def test_process_block_bit_exact(G, bs):
    """Given the same L and W the in-block kernel reproduces the CPU evaluation bit for bit."""
    K = 2 * bs if bs != 100 else 200
    N = 300
    W, X = _problem(20 + bs, K, N, 4 * K + 50, correlated=True)
    H = O.accumulate_H([X])
    _, L, bad = O.damp_and_invert(W, H, 0.01)
    assert not bad
    p = O.get_col_quantize_params(W)
    for start in (0, K - bs):
        q_ref, e_ref = O.process_block(W, L, start, p, bs)
        q, e = G._process_block(W, L, start, p, bs)
        assert np.array_equal(to_np(q), q_ref)
        assert np.array_equal(to_np(e), e_ref)


@pytest.mark.parametrize("bs,K,N", [(32, 96, 256), (48, 144, 260), (96, 192, 64), (112, 224, 128), (128, 384, 192),
                                    (16, 50, 130), (64, 192, 1024)])
def test_process_block_bit_exact_more_shapes(G, bs, K, N):
    """Block sizes with 2 to 8 sub-blocks of 16 rows (and of 4 rows: 50 is not a multiple of 4, so L's rows are
    not 16-byte aligned), channel counts with full and partial 64-channel tiles, blocks at the start, in the
    middle and at the end of the matrix."""
    W, X = _problem(300 + bs + N, K, N, 4 * K + 50, correlated=True)
    H = O.accumulate_H([X])
    _, L, bad = O.damp_and_invert(W, H, 0.01)
    assert not bad
    p = O.get_col_quantize_params(W)
    for start in sorted({0, ((K - bs) // 2 // 2) * 2, K - bs}):
        q_ref, e_ref = O.process_block(W, L, start, p, bs)
        q, e = G._process_block(W, L, start, p, bs)
        assert np.array_equal(to_np(q), q_ref)
        assert np.array_equal(to_np(e), e_ref)


@pytest.mark.parametrize("N", [256, 197])
@pytest.mark.parametrize("diag", ["plain", "tiny", "huge", "mixed"])
def test_process_block_bit_exact_outside_the_fast_range(G, N, diag):
    """The kernel's chain uses reciprocal forms of the two divisions where they are proven to give the bits of
    the division, and falls back to the divisions elsewhere: ties of the rounding, weights on the grid (zero
    error), extreme and denormal scales, fractional zero points, extreme diagonals of L, infinities and
    NaNs all have to come out as the CPU evaluation has them.  (One known difference is left out of the
    comparison: where the value to be quantised is a NaN, numpy's clip returns NaN and the kernel's
    fmin(fmax(., 0), maxq) returns a number; the errors are NaN in both, as long as the NaN does not come from a
    zero scale, which is therefore not among the cases.)"""
    rng = np.random.default_rng(700 + N + len(diag))
    bs, K = 32, 64
    L = np.tril(0.1 * rng.standard_normal((K, K))).astype(np.float32)
    d = rng.uniform(0.5, 2.0, K).astype(np.float32)
    if diag == "tiny":
        d *= np.float32(1e-15)
    elif diag == "huge":
        d *= np.float32(1e15)
    elif diag == "mixed":
        d[3::7] *= np.float32(1e-14)
        d[5::11] *= np.float32(1e14)
    L[np.arange(K), np.arange(K)] = d
    scale = np.full(N, 2.0 ** -6, np.float32)
    scale[1::8] = rng.uniform(0.001, 0.02, scale[1::8].shape).astype(np.float32)
    scale[2::16] = np.float32(1e-30)
    scale[3::16] = np.float32(1e30)
    scale[4::32] = np.float32(1e-40)          # denormal
    zero = rng.integers(0, 16, N).astype(np.float32)
    zero[6::16] += np.float32(0.5)
    zero[7::32] = np.float32(3e7)
    k = rng.integers(-3, 19, (K, N)).astype(np.float32)
    W = (scale[None, :] * (k - zero[None, :])).astype(np.float32)          # on the grid: zero error
    half = rng.random((K, N)) < 0.3
    W[half] += (0.5 * scale[None, :] * np.ones((K, 1), np.float32))[half]  # ties of the rounding
    noise = rng.random((K, N)) < 0.4
    W[noise] += (0.3 * scale[None, :] * rng.standard_normal((K, N)).astype(np.float32))[noise]
    W[5, 9::40] = np.inf
    W[17, 11::40] = np.nan
    W[40, 13::40] = -np.inf
    p = {"scale": scale, "zero": zero, "maxq": 15}
    with np.errstate(all="ignore"):
        for start in (0, K - bs):
            q_ref, e_ref = O.process_block(W, L, start, p, bs)
            q, e = G._process_block(W, L, start, p, bs)
            q, e = to_np(q), to_np(e)
            assert np.array_equal(e, e_ref, equal_nan=True)
            known = ~np.isnan(q_ref)
            assert np.array_equal(q[known], q_ref[known])


def _check_against_oracle(G, W, xs, X_all, **kw):
    Q, p = G.gptq(W, xs, **kw)
    Qr, pr = O.gptq(W, xs, **kw)
    Q = to_np(Q)
    assert Q.dtype == W.dtype and Q.shape == W.shape
    assert p["maxq"] == 15
    assert np.allclose(to_np(p["scale"]), pr["scale"], rtol=1e-5, atol=0)
    assert np.allclose(to_np(p["zero"]), pr["zero"], rtol=1e-5, atol=0)
    c = O.codes_from_q(Q, pr)
    cr = O.codes_from_q(Qr, pr)
    frac, mx = code_stats(c, cr)
    assert frac <= 1e-3, f"{frac:.2e} of the codes differ"
    assert mx <= 1
    e, er = recon_error(W, Q, X_all), recon_error(W, Qr, X_all)
    assert abs(e - er) <= 0.01 * er, (e, er)
    # packing of the result: bit-exact against the oracle's packing of the same Q
    packed = G.pack_matrix(Q, p)
    assert np.array_equal(to_np(packed.int_weight), O.pack_matrix(Q, pr).int_weight)
    assert np.array_equal(to_np(G.unpack_matrix(packed)).astype(W.dtype), Q)
    return frac


def test_gptq_config1_gpt2_mlp_up(G):
    """W 768x3072 fp32 ~N(0,0.02), X 2048x768 ~N(0,1), 4-bit, damp 1 %, block 128."""
    rng = np.random.default_rng(0)
    W = (0.02 * rng.standard_normal((768, 3072))).astype(np.float32)
    X = np.random.default_rng(1).standard_normal((2048, 768)).astype(np.float32)
    _check_against_oracle(G, W, [X], X)


@pytest.mark.parametrize("K,N,n,bs", [(256, 64, 128, 4), (256, 1024, 128, 16), (512, 200, 2048, 128),
                                      (192, 130, 800, 64), (384, 96, 1500, 128)])
def test_gptq_shapes_and_block_sizes(G, K, N, n, bs):
    W, X = _problem(K + N, K, N, n, correlated=True)
    xs = [X[i:i + 128] for i in range(0, n, 128)]
    _check_against_oracle(G, W, xs, X, block_size=bs)


def test_gptq_fp16_weights_and_fp16_calibration(G):
    W, X = _problem(7, 256, 320, 1024, wdtype=np.float16)
    X16 = X.astype(np.float16)
    xs = [X16[:512], X16[512:]]
    _check_against_oracle(G, W, xs, X16.astype(np.float32))


def test_gptq_actorder(G):
    W, X = _problem(8, 256, 128, 1024)
    X = (X * np.linspace(0.5, 2.0, 256, dtype=np.float32)[None, :]).astype(np.float32)
    _check_against_oracle(G, W, [X], X, actorder=True, block_size=64)


def test_gptq_dead_feature(G):
    W, X = _problem(9, 256, 64, 1024)
    X[:, 11] = 0
    Q, p = G.gptq(W, [X])
    Q = to_np(Q)
    # a dead input feature is zeroed and then quantised like any zero: dequantised 0
    qz = O.quantize_value(p_np(p)["zero"], p_np(p)["scale"], 15, np.zeros(64, np.float32))
    assert np.array_equal(Q[11], qz)
    _check_against_oracle(G, W, [X], X)


def p_np(p):
    return {"scale": to_np(p["scale"]), "zero": to_np(p["zero"]), "maxq": p["maxq"]}


def test_gptq_identity_hessian_is_round_to_nearest(G):
    """Orthogonal calibration columns: H = c I, L diagonal, no error feedback -> plain RTN."""
    K, N = 256, 96
    rng = np.random.default_rng(10)
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    X = (2.0 * np.eye(K)).astype(np.float32)
    Q, p = G.gptq(W, [X], block_size=32)
    pn = p_np(p)
    assert np.array_equal(to_np(Q), O.quantize_value(pn["zero"], pn["scale"], 15, W))


def test_gptq_pack_roundtrip_reference_case(G):
    # reference tests.py:147-156: W 256x64 N(0,1), integer calibration 4 x (32x256), block 4
    rng = np.random.default_rng(0)
    w = rng.standard_normal((256, 64)).astype(np.float32)
    xs = [rng.integers(0, 16, (32, 256)).astype(np.float32) for _ in range(4)]
    quantized, qparams = G.gptq(w, xs, block_size=4)
    packed_w = G.pack_matrix(quantized, qparams)
    unpacked_w = G.unpack_matrix(packed_w)
    assert bool((unpacked_w == quantized).all())
    assert tuple(packed_w.int_weight.shape) == (128, 64)


def test_gptq_argument_errors(G):
    W, X = _problem(11, 64, 16, 128)
    with pytest.raises(ValueError):
        G.gptq(W, [X], block_size=48)          # does not divide K
    with pytest.raises(ValueError):
        G.gptq(W, [X[:, :32]], block_size=64)  # feature dimension mismatch


@pytest.mark.parametrize("bits", [8, 3, 2])
def test_gptq_other_code_widths(G, bits):
    """``bits`` other than 4 (not in the reference's ``gptq``, whose parameters come from
    ``get_quantize_params(w, bits=4)``): same bars against the oracle run at that width, and the
    error falls with the width."""
    W, X = _problem(70 + bits, 256, 160, 1500, correlated=True)
    Q, p = G.gptq(W, [X], bits=bits)
    Qr, pr = O.gptq(W, [X], _bits=bits)
    assert p["maxq"] == 2 ** bits - 1 == pr["maxq"]
    assert np.allclose(to_np(p["scale"]), pr["scale"], rtol=1e-5, atol=0)
    assert np.allclose(to_np(p["zero"]), pr["zero"], rtol=1e-5, atol=0)
    codes = lambda q: np.rint(q.astype(np.float32) / pr["scale"][None] + pr["zero"][None]).astype(np.int32)
    c, cr = codes(to_np(Q)), codes(Qr)
    assert c.min() >= 0 and c.max() <= 2 ** bits - 1
    frac, mx = code_stats(c, cr)
    # 8-bit steps are 1/17 of the 4-bit ones: summation-order differences flip more codes
    assert frac <= (1e-3 if bits <= 4 else 2e-2) and mx <= 1, (frac, mx)
    e, er = recon_error(W, to_np(Q), X), recon_error(W, Qr, X)
    assert abs(e - er) <= 0.01 * er
    e4 = recon_error(W, to_np(G.gptq(W, [X])[0]), X)
    assert (e < e4 / 8) if bits == 8 else (e > e4)
    if bits == 8:
        # one code per byte, equal to the codes of the dequantised result
        packed = G.pack_matrix(Q, p)
        assert packed.bits == 8 and packed.shape == W.shape
        assert np.array_equal(to_np(packed.int_weight).astype(np.int32), c)
    else:
        with pytest.raises(NotImplementedError):
            G.pack_matrix(Q, p)
    with pytest.raises(ValueError):
        G.gptq(W, [X], bits=9)


@pytest.mark.parametrize("K,N,start,k", [(4096, 11008, 0, 512), (4096, 11008, 2560, 512), (4096, 11008, 3072, 512),
                                         (2048, 8192, 0, 512), (1024, 768, 0, 128), (1536, 4096, 512, 256),
                                         (4096, 4352, 1024, 512), (1000, 520, 128, 128), (11008, 4096, 512, 512)])
def test_lazy_update_against_double(K, N, start, k):
    """The lazy batch update W[end:] -= L[end:, start:end] @ errors (gptq.py:204-205) at the shapes of the column
    loop, against the product in double: the k = 512 updates of the benchmark layer (3584, 1024 and 512 rows
    below the group), k = 128 and 256 inside a group, shapes that are no multiple of the tiles.  fp32 products
    summed in fp32: 1e-5 sqrt(k) of the largest magnitude; the same bits on a second evaluation."""
    import torch
    import jax_gptq_amd.gptq as G
    g = torch.Generator(device="cuda").manual_seed(K + N + start)
    W = torch.randn((K, N), generator=g, device="cuda")
    L = torch.tril(torch.randn((K, K), generator=g, device="cuda"))
    E = torch.randn((k, N), generator=g, device="cuda")
    end = start + k
    ref = W.double()
    ref[end:] -= L[end:, start:end].double() @ E.double()
    W0 = W.clone()
    got = G._lazy_update(W, L, E, start, end)
    assert got.data_ptr() == W.data_ptr()
    assert torch.equal(got[:end], W0[:end])
    err = float((got.double() - ref).abs().max())
    assert err <= 1e-5 * float(ref.abs().max()) * (k ** 0.5), err
    # the same bits on a second evaluation
    W2 = G._lazy_update(W0.clone(), L, E, start, end)
    assert torch.equal(W2, got)
