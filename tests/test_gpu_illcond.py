"""GPU parity of the layer solve on ill-conditioned Hessians at K = 2048 and 4096.

The other large-shape tests draw independent N(0, 1) calibration rows, whose Hessian is close to the identity.
Real calibration activations are not like that, and the reference's own kernel test is rank deficient
(``/root/reference/test_kernel.py:13-17``: one batch, far fewer rows than features, positive definite through the
damping only).  The factor of the inverse comes by another route here than in the reference (reverse Cholesky +
triangular inverse against potrf / potrs / potrf), so its error growth with the condition number is pinned here:

* outlier features: the columns of X are scaled over two decades (diag(H) spread 1e4) and share a low-rank component;
* rank-deficient calibration: n = K / 8 rows, H positive definite through the damping only;
* both with and without ``actorder``.

Bars as everywhere: scale / zero within 1e-5 relative, at least 99.9 % of the codes equal and the rest off by one,
reconstruction error within 1 % of the oracle's.  Two fp32 evaluations of an ill-conditioned solve need not agree
that closely with each other (different summation orders in H and in the factorisation move values across rounding
boundaries); where they do not, both are measured against the oracle's fp64 evaluation (``use_fp64=True``) and the
GPU result has to meet the bar against that, or be as close to it as the oracle's own fp32 evaluation is (within
a factor, stated below).
"""
import numpy as np
import pytest
import scipy.linalg

from helpers import code_stats, recon_error, to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


def _calibration(rng, K, kind):
    if kind == "outliers":
        n = 2 * K
        x = rng.standard_normal((n, K)).astype(np.float32)
        s = np.exp(rng.uniform(0.0, np.log(100.0), K)).astype(np.float32)      # diag(H) over four decades
        s[rng.choice(K, 8, replace=False)] = 100.0
        u = rng.standard_normal((n, 4)).astype(np.float32) @ rng.standard_normal((4, K)).astype(np.float32)
        x = (x + 0.5 * u) * s[None, :]
        return [x[:K], x[K:]]
    if kind == "rank_deficient":
        return [rng.standard_normal((K // 8, K)).astype(np.float32)]
    raise ValueError(kind)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("actorder", [False, True])
@pytest.mark.parametrize("kind", ["outliers", "rank_deficient"])
@pytest.mark.parametrize("K", [2048, 4096])
def test_gptq_against_the_oracle_on_ill_conditioned_hessians(K, kind, actorder):
    import jax_gptq_amd.gptq as G
    N = 256
    rng = np.random.default_rng(K + 7 * len(kind) + int(actorder))
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    xs = _calibration(rng, K, kind)
    X = np.concatenate(xs)

    Q, p = G.gptq(W, xs, actorder=actorder)
    Q = to_np(Q)
    Qr, pr = O.gptq(W, xs, actorder=actorder)
    assert np.allclose(to_np(p["scale"]), pr["scale"], rtol=1e-5, atol=0)
    assert np.allclose(to_np(p["zero"]), pr["zero"], rtol=1e-5, atol=0)
    c, cr = O.codes_from_q(Q, pr), O.codes_from_q(Qr, pr)
    frac, mx = code_stats(c, cr)
    e, er = recon_error(W, Q, X), recon_error(W, Qr, X)
    print(f"K={K} {kind} actorder={actorder}: codes differing from the fp32 oracle {frac:.2e} (max {mx}), "
          f"recon {e:.6f} vs {er:.6f}")
    if frac <= 1e-3 and mx <= 1 and abs(e - er) <= 0.01 * er:
        return
    # the two fp32 evaluations part: arbitrate against the fp64 evaluation
    Q64, p64 = O.gptq(W, xs, actorder=actorder, use_fp64=True)
    c64 = O.codes_from_q(Q64, p64)
    f_gpu, m_gpu = code_stats(c, c64)
    f_orc, m_orc = code_stats(cr, c64)
    e64 = recon_error(W, Q64, X)
    print(f"  against the fp64 oracle: GPU {f_gpu:.2e} (max {m_gpu}), fp32 oracle {f_orc:.2e} (max {m_orc}); "
          f"recon fp64 {e64:.6f}")
    # Which codes flip is a matter of the summation order (H summed in another order moved this case from 3.5e-4 to
    # 9.7e-4 against fp64 while the oracle's own fp32 evaluation stood at 1.1e-3 and 3.7e-4).  So: the usual bar
    # against the fp64 solve (99.9 % of the codes equal, none further off than the fp32 oracle's worst), or as
    # close to it as the reference arithmetic is (1.5 x the fp32 oracle's rate plus 1e-4); and a reconstruction
    # error within 1 % of the fp64 solve's or no worse than the fp32 oracle's
    assert (f_gpu <= 1e-3 and m_gpu <= max(1, m_orc)) or f_gpu <= 1.5 * f_orc + 1e-4, (f_gpu, m_gpu, f_orc, m_orc)
    assert e <= max(er, 1.01 * e64), (e, er, e64)


@pytest.mark.timeout(600)
@pytest.mark.parametrize("kind,damp,cond_min", [("outliers", 0.01, 1e4), ("outliers", 0.001, 1e5),
                                                ("rank_deficient", 0.01, 1e3)])
def test_factor_of_the_inverse_at_high_condition_number(kind, damp, cond_min):
    """L = chol(inv(H_damped)) at K = 4096 with cond(H) from 1e3 to several 1e5 (measured: 1.5e3 for the
    rank-deficient set, 5e4 and 5e5 for the outlier features at 1 % and 0.1 % damping) against LAPACK in fp64, next
    to the error of the oracle's fp32 three-step route (potrf, potrs, potrf as the reference calls them)."""
    import jax_gptq_amd.gptq as G
    K = 4096
    rng = np.random.default_rng(31 + len(kind))
    xs = _calibration(rng, K, kind)
    X = np.concatenate(xs).astype(np.float64)
    H64 = X.T @ X / X.shape[0]
    H64 += damp * np.mean(np.diag(H64)) * np.eye(K)
    H = H64.astype(np.float32)
    H64 = H.astype(np.float64)                     # the matrix both routes are given
    ev = np.linalg.eigvalsh(H64)
    cond = ev[-1] / ev[0]
    ref = scipy.linalg.cholesky(np.linalg.inv(H64), lower=True)
    L = to_np(G._cholesky_inv(H)).astype(np.float64)
    orc = O.cholesky_inv(H).astype(np.float64)
    assert np.array_equal(L, np.tril(L)) and np.all(np.diag(L) > 0)
    scale = np.abs(ref).max()
    e_gpu, e_orc = np.abs(L - ref).max() / scale, np.abs(orc - ref).max() / scale
    r_gpu = np.abs(L @ (L.T @ H64) - np.eye(K)).max()
    r_orc = np.abs(orc @ (orc.T @ H64) - np.eye(K)).max()
    print(f"{kind} damp {damp}: cond(H) = {cond:.2e}; |L - L_ref| / max|L_ref|: GPU {e_gpu:.2e}, fp32 oracle {e_orc:.2e}; "
          f"|L L^T H - I|: GPU {r_gpu:.2e}, fp32 oracle {r_orc:.2e}")
    assert cond > cond_min
    assert e_gpu <= 4 * e_orc + 1e-6
    assert r_gpu <= 4 * r_orc + 1e-5
