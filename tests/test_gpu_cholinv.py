"""GPU parity of the dead-feature fix, damping and the Cholesky factor of the inverse."""
import numpy as np
import pytest
import scipy.linalg

from helpers import to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import jax_gptq_amd.gptq as g
    return g


def _spd(seed, K, n, scale_cols=False):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, K))
    if scale_cols:
        x = x * np.linspace(0.3, 3.0, K)[None, :]
    return (x.T @ x / n).astype(np.float32)


@pytest.mark.parametrize("K", [128, 256, 300, 37, 640, 1024, 2240])     # 2240: 35 diagonal blocks, both forms of the step kernel
def test_cholesky_inv_matches_lapack(G, K):
    H = _spd(K, K, 4 * K, scale_cols=True)
    H += 0.01 * np.mean(np.diag(H)) * np.eye(K, dtype=np.float32)
    L = to_np(G._cholesky_inv(H)).astype(np.float64)
    assert np.array_equal(L, np.tril(L)) and np.all(np.diag(L) > 0)
    H64 = H.astype(np.float64)
    ref = scipy.linalg.cholesky(np.linalg.inv(H64), lower=True)
    # fp32 factorisation of a matrix with condition number ~1e3
    assert np.abs(L @ L.T @ H64 - np.eye(K)).max() < 2e-3
    assert np.abs(L - ref).max() < 1e-3 * np.abs(ref).max()
    # at least as close to the exact factor as the oracle's fp32 three-step route
    orc = O.cholesky_inv(H).astype(np.float64)
    assert np.abs(L - ref).max() <= 4 * np.abs(orc - ref).max() + 1e-6


def test_cholesky_inv_two_level_blocking(G):
    """K >= 6144 factorises with a second blocking level (512-row outer blocks; K = 6200 pads to
    97 diagonal blocks, so the first outer block handled is a partial one).  Reference: LAPACK
    in fp64 on the host."""
    import torch
    K = 6200
    g = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn((K + 300, K), generator=g, device="cuda", dtype=torch.float64)
    x *= torch.linspace(0.3, 3.0, K, device="cuda", dtype=torch.float64)[None, :]
    H64 = x.T @ x / x.shape[0]
    H64 += 0.01 * H64.diagonal().mean() * torch.eye(K, device="cuda", dtype=torch.float64)
    H = H64.float()
    L = G._cholesky_inv(H).double()
    assert bool((torch.triu(L, 1) == 0).all()) and bool((L.diagonal() > 0).all())
    assert float((L @ L.T @ H.double() - torch.eye(K, device="cuda", dtype=torch.float64)).abs().max()) < 5e-3
    ref = scipy.linalg.cholesky(np.linalg.inv(H.double().cpu().numpy()), lower=True)
    assert np.abs(L.cpu().numpy() - ref).max() < 1e-3 * np.abs(ref).max()


def test_damp_and_invert_dead_feature_and_damping(G):
    import torch
    rng = np.random.default_rng(4)
    K, N = 200, 24
    X = rng.standard_normal((600, K)).astype(np.float32)
    X[:, 7] = 0.0
    X[:, 150] = 0.0
    H = (X.T @ X / 600).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    Wt = torch.from_numpy(W).cuda()
    Ht = torch.from_numpy(H).cuda()
    W2, L, bad = G._damp_and_invert(Wt, Ht, 0.01)
    assert not bad
    W2 = to_np(W2)
    Wr, Lr, _ = O.damp_and_invert(W, H, 0.01)
    assert np.array_equal(W2, Wr)
    Hd = H.astype(np.float64).copy()
    Hd[7, 7] = 1.0
    Hd[150, 150] = 1.0
    Hd += 0.01 * np.mean(np.diag(Hd)) * np.eye(K)
    L = to_np(L).astype(np.float64)
    assert np.abs(L @ L.T @ Hd - np.eye(K)).max() < 2e-3
    assert np.abs(L - Lr).max() < 1e-3 * np.abs(Lr).max()


@pytest.mark.parametrize("K,idx", [(160, 3), (2240, 700)])     # the pivot fails inside a step of either form
def test_not_positive_definite_is_flagged(G, K, idx):
    import torch
    H = _spd(5, K, 4 * K)
    H[idx, idx] = -1.0
    _, _, bad = G._damp_and_invert(torch.zeros((K, 4), device="cuda"), torch.from_numpy(H).cuda(), 0.0)
    assert bad
    with pytest.raises(ValueError):
        x = np.ones((4, 8), np.float32)
        x[:, 0] = np.nan
        G.gptq(np.ones((8, 4), np.float32), [x], block_size=4)
