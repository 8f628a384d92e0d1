"""GPU parity of the use_fp64 option: Hessian, factor of the inverse and the whole solve with H
and the Cholesky steps in double (reference ``gptq.py:88, 182-197``)."""
import numpy as np
import pytest
import scipy.linalg

from helpers import code_stats, recon_error, to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import jax_gptq_amd.gptq as g
    return g


def test_accumulate_H_fp64_reference_case(G):
    """The reference's own Hessian test (``tests.py:293-311``): 20 identical batches of
    37 x 256, ``accumulate_H(xs, use_fp64=True)`` against ``sum x^T x / n`` in fp64."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal((37, 256))
    xs = [x.copy() for _ in range(20)]
    H = to_np(G.accumulate_H(xs, use_fp64=True))
    assert H.dtype == np.float64 and H.shape == (256, 256)
    ref = sum(b.T @ b for b in xs) / (20 * 37)
    # a different summation order from the reference's: a few ulp of entries of O(1)
    assert np.abs(H - ref).max() < 4e-15
    assert np.array_equal(H, H.T)


@pytest.mark.parametrize("rows,K,nb,dt", [(37, 256, 20, "float64"), (512, 768, 3, "float32"),
                                          (33, 100, 4, "float64"), (5, 130, 2, "float32"),
                                          (300, 1, 1, "float64"), (200, 264, 2, "float16"),
                                          (200, 264, 2, "bfloat16")])
def test_accumulate_H_fp64_closed_form(G, rows, K, nb, dt):
    import torch
    rng = np.random.default_rng(123)
    xs_t = [torch.from_numpy(rng.standard_normal((rows, K))).to(getattr(torch, dt)) for _ in range(nb)]
    xs64 = [x.double().numpy() for x in xs_t]           # the inputs as rounded
    H = to_np(G.accumulate_H(xs_t, use_fp64=True))
    flat = np.concatenate(xs64)
    ref = flat.T @ flat / flat.shape[0]
    assert H.dtype == np.float64
    assert np.abs(H - ref).max() < 1e-13 * max(1.0, np.abs(ref).max())
    assert np.abs(H - O.accumulate_H(xs64, use_fp64=True)).max() < 1e-13 * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("K", [64, 128, 300, 37, 640, 1024])
def test_cholesky_inv_fp64_matches_lapack(G, K):
    rng = np.random.default_rng(K)
    x = rng.standard_normal((4 * K, K)) * np.linspace(0.3, 3.0, K)[None, :]
    H = x.T @ x / (4 * K)
    H += 0.01 * np.mean(np.diag(H)) * np.eye(K)
    L = to_np(G._cholesky_inv(H))
    assert L.dtype == np.float64
    assert np.array_equal(L, np.tril(L)) and np.all(np.diag(L) > 0)
    ref = scipy.linalg.cholesky(np.linalg.inv(H), lower=True)
    assert np.abs(L @ L.T @ H - np.eye(K)).max() < 1e-10
    assert np.abs(L - ref).max() < 1e-10 * np.abs(ref).max()


def test_damp_and_invert_fp64_dead_feature(G):
    import torch
    rng = np.random.default_rng(4)
    K, N = 200, 24
    X = rng.standard_normal((600, K))
    X[:, 7] = 0.0
    H = X.T @ X / 600
    W = rng.standard_normal((K, N)).astype(np.float32)
    W2, L, bad = G._damp_and_invert(torch.from_numpy(W).cuda(), torch.from_numpy(H).cuda(), 0.01)
    assert not bad and L.dtype == torch.float64
    Wr, Lr, _ = O.damp_and_invert(W, H, 0.01)
    assert np.array_equal(to_np(W2), Wr)
    assert np.abs(to_np(L) - Lr).max() < 1e-10 * np.abs(Lr).max()
    Hbad = H.copy()
    Hbad[3, 3] = -1.0
    _, _, bad = G._damp_and_invert(torch.zeros((K, 4), device="cuda"), torch.from_numpy(Hbad).cuda(), 0.0)
    assert bad


@pytest.mark.parametrize("K,N,n,actorder", [(256, 384, 1024, False), (384, 200, 1500, True)])
def test_gptq_fp64_matches_oracle(G, K, N, n, actorder):
    rng = np.random.default_rng(K + N)
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    X = rng.standard_normal((n, K)) @ (np.eye(K) + 0.5 * rng.standard_normal((K, K)) / np.sqrt(K))
    X = X.astype(np.float32)
    xs = [X[i:i + 256] for i in range(0, n, 256)]
    Q, p = G.gptq(W, xs, use_fp64=True, actorder=actorder)
    Qr, pr = O.gptq(W, xs, use_fp64=True, actorder=actorder)
    Q = to_np(Q)
    assert Q.dtype == np.float32
    assert np.allclose(to_np(p["scale"]), pr["scale"], rtol=1e-5, atol=0)
    assert np.allclose(to_np(p["zero"]), pr["zero"], rtol=1e-5, atol=0)
    frac, mx = code_stats(O.codes_from_q(Q, pr), O.codes_from_q(Qr, pr))
    assert frac <= 1e-3 and mx <= 1, (frac, mx)
    e, er = recon_error(W, Q, X), recon_error(W, Qr, X)
    assert abs(e - er) <= 0.01 * er


@pytest.mark.parametrize("use_fp64", [False, True])
def test_gptq_shared_hessian_and_factor(G, use_fp64):
    """Several matrices solved against the same activations through ``shared``: one Hessian,
    one factorisation, results bit-identical to independent calls (a dead feature included)."""
    import torch
    rng = np.random.default_rng(17)
    xs = [rng.standard_normal((96, 192)).astype(np.float32) for _ in range(4)]
    for x in xs:
        x[:, 5] = 0
    Ws = [rng.standard_normal((192, 80 + 16 * i)).astype(np.float32) for i in range(3)]
    shared = {}
    got = [G.gptq(W.copy(), xs, block_size=64, use_fp64=use_fp64, shared=shared) for W in Ws]
    assert set(shared) == {"H", ("factor", 0.01)}
    assert shared["H"].dtype == (torch.float64 if use_fp64 else torch.float32)
    for W, (Q, p) in zip(Ws, got):
        Qi, pi = G.gptq(W.copy(), xs, block_size=64, use_fp64=use_fp64)
        assert torch.equal(Q, Qi) and torch.equal(p["scale"], pi["scale"]) and torch.equal(p["zero"], pi["zero"])
        assert bool((Q[5] == 0).all())
    # another damping value gets a factor of its own; act-order never shares the factor
    G.gptq(Ws[0].copy(), xs, block_size=64, use_fp64=use_fp64, damping=0.05, shared=shared)
    assert ("factor", 0.05) in shared
    Qa, _ = G.gptq(Ws[0].copy(), xs, block_size=64, use_fp64=use_fp64, actorder=True, shared=shared)
    Qb, _ = G.gptq(Ws[0].copy(), xs, block_size=64, use_fp64=use_fp64, actorder=True)
    assert torch.equal(Qa, Qb)
