"""GPU parity of the Hessian accumulation (fp32 MFMA) against the closed form and the oracle."""
import numpy as np
import pytest

from helpers import to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import jax_gptq_amd.gptq as g
    return g


def _closed_form(xs):
    flat = np.concatenate([np.asarray(x, dtype=np.float64).reshape(-1, x.shape[-1]) for x in xs])
    return flat.T @ flat / flat.shape[0]


# tolerance: fp32 accumulation of n products of O(1) numbers; entries are O(1) after /n
TOL = 2e-5


@pytest.mark.parametrize("rows,K,nb", [(37, 256, 20), (2048, 768, 1), (512, 768, 3), (33, 100, 4),
                                       (5, 130, 2), (300, 1, 1), (1, 384, 1)])
def test_accumulate_H_closed_form(G, rows, K, nb):
    rng = np.random.default_rng(9876)
    xs = [rng.standard_normal((rows, K)).astype(np.float32) for _ in range(nb)]
    H = to_np(G.accumulate_H(xs))
    ref = _closed_form(xs)
    assert H.shape == (K, K) and H.dtype == np.float32
    assert np.array_equal(H, H.T)
    assert np.abs(H - ref).max() < TOL * max(1.0, np.abs(ref).max())
    orc = O.accumulate_H(xs)
    assert np.abs(H - orc).max() < 2 * TOL * max(1.0, np.abs(ref).max())


def test_accumulate_H_ragged_and_3d_batches(G):
    rng = np.random.default_rng(1)
    xs = [rng.standard_normal((3, 11, 96)).astype(np.float32),
          rng.standard_normal((7, 96)).astype(np.float32) + 2.0,
          rng.standard_normal((129, 96)).astype(np.float32)]
    H = to_np(G.accumulate_H(xs))
    ref = _closed_form(xs)
    assert np.abs(H - ref).max() < TOL * np.abs(ref).max()


@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
def test_accumulate_H_half_inputs(G, dt):
    import torch
    rng = np.random.default_rng(2)
    tdt = getattr(torch, dt)
    xs_t = [torch.from_numpy(rng.standard_normal((200, 264)).astype(np.float32)).to(tdt)
            for _ in range(3)]
    H = to_np(G.accumulate_H(xs_t))
    ref = _closed_form([x.float().numpy() for x in xs_t])   # the inputs as rounded
    assert np.abs(H - ref).max() < TOL * np.abs(ref).max()


@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
@pytest.mark.parametrize("rows,K,nb", [(37, 256, 20), (2048, 768, 2), (33, 104, 4), (5, 136, 2),
                                       (1, 384, 1), (130, 4096, 3), (64, 128, 1), (700, 520, 5),
                                       # K >= 1024: the 256 x 256-tile kernel (ragged slabs, features
                                       # past K in the last tile, more row slices than slabs)
                                       (37, 1032, 7), (1, 1024, 1), (2049, 1288, 2), (95, 2056, 40),
                                       (3, 1024, 70), (4096, 1024, 4),
                                       # K % 256 == 0 and rows % 32 == 0: loads straight into LDS
                                       # (one, two, three slabs in all; many short batches; long slices)
                                       (32, 1024, 1), (64, 1024, 1), (96, 1024, 1), (32, 1280, 37),
                                       (512, 2304, 9), (2048, 4096, 6)])
def test_accumulate_H_16bit_mfma_path(G, rows, K, nb, dt):
    """fp16 / bf16 batches with K % 8 == 0 run on the 16-bit matrix instructions: products of
    two such numbers are exact in fp32, so the result must agree with the closed form of the
    widened inputs, and with the fp32 kernel fed the widened inputs, to fp32 summation error."""
    import torch
    rng = np.random.default_rng(rows + K)
    tdt = getattr(torch, dt)
    xs_t = [torch.from_numpy(rng.standard_normal((rows, K)).astype(np.float32)).to(tdt).cuda()
            for _ in range(nb)]
    H = to_np(G.accumulate_H(xs_t))
    wide = [x.float() for x in xs_t]
    ref = _closed_form([x.cpu().numpy() for x in wide])
    assert H.dtype == np.float32 and np.array_equal(H, H.T)
    assert np.abs(H - ref).max() < TOL * max(1.0, np.abs(ref).max())
    H32 = to_np(G.accumulate_H(wide))
    assert np.abs(H - H32).max() < TOL * max(1.0, np.abs(ref).max())


def test_accumulate_H_16bit_unaligned_batch_falls_back(G):
    """A batch that is not 16-byte aligned takes the fp32 kernel; same result."""
    import torch
    rng = np.random.default_rng(77)
    base = torch.from_numpy(rng.standard_normal((64 * 264 + 1,)).astype(np.float32)).to(torch.float16).cuda()
    x = base[1:].view(64, 264)          # 2-byte aligned only
    assert x.data_ptr() % 16 != 0
    H = to_np(G.accumulate_H([x]))
    ref = _closed_form([x.float().cpu().numpy()])
    assert np.abs(H - ref).max() < TOL * np.abs(ref).max()


def test_accumulate_H_zero_feature_is_exact_zero(G):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((64, 160)).astype(np.float32)
    x[:, 5] = 0
    H = to_np(G.accumulate_H([x]))
    assert np.all(H[5] == 0) and np.all(H[:, 5] == 0)


@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
def test_accumulate_H_16bit_mixed_batch_sizes(G, dt):
    """Batches of different lengths, all multiples of 32 rows (the loads-straight-into-LDS
    kernel: row slices then start and end inside batches and cross several of them), and the
    same data with one batch shortened by a row (the register-staged kernel): both against the
    closed form."""
    import torch
    rng = np.random.default_rng(99)
    tdt = getattr(torch, dt)
    K = 1536
    sizes = [64, 96, 32, 2048, 160, 32, 32, 1024, 448, 32]
    xs_t = [torch.from_numpy(rng.standard_normal((n, K)).astype(np.float32)).to(tdt).cuda() for n in sizes]
    ref = _closed_form([x.float().cpu().numpy() for x in xs_t])
    H = to_np(G.accumulate_H(xs_t))
    assert np.array_equal(H, H.T)
    assert np.abs(H - ref).max() < TOL * max(1.0, np.abs(ref).max())
    ragged = list(xs_t)
    ragged[3] = xs_t[3][:-1]
    ref2 = _closed_form([x.float().cpu().numpy() for x in ragged])
    H2 = to_np(G.accumulate_H(ragged))
    assert np.abs(H2 - ref2).max() < TOL * max(1.0, np.abs(ref2).max())


def _split_H(G, xs):
    """accumulate_H(xs, split_fp16=True) without the wrapper's K >= 1024 rule (below that the fp32
    kernel is the faster one and the wrapper keeps it): the split entry point on any K % 256 == 0."""
    import torch
    import jax_gptq_amd._native as NV
    batches = [torch.from_numpy(x).cuda() for x in xs]
    K = batches[0].shape[1]
    H = torch.zeros((K, K), dtype=torch.float32, device="cuda")
    assert G._split16_ok(H, batches) or K < 1024
    G._hessian_accumulate_split16(H, batches)
    NV.check(NV.load().gptq_hip_hessian_finalize(G._stream(), H.data_ptr(), 0, K, float(sum(b.shape[0] for b in batches))),
             "hessian_finalize")
    return H


@pytest.mark.parametrize("rows,K,nb,scale", [(2048, 256, 2, 1.0), (512, 768, 9, 1e-4), (96, 1024, 50, 3e5),
                                             (4096, 512, 3, 1.0), (32, 256, 1, 1.0), (512, 1280, 5, 1.0)])
def test_accumulate_H_fp32_rows_as_fp16_pairs(G, rows, K, nb, scale):
    """split_fp16: x = (hi + lo) 2^e with fp16 hi and lo, X^T X from hi^T hi + hi^T lo + lo^T hi on
    the 16-bit matrix cores.  Same tolerance against the closed form as the fp32 kernel (the
    dropped lo^T lo term is 2^-22 of a product); the exponent is chosen from the data, so the
    scale of the rows (1e-4 .. 3e5 here: products far outside fp16) does not matter.  50 batches
    span two launches, whose partial tiles accumulate before the one reduction."""
    import torch
    rng = np.random.default_rng(rows + K + nb)
    xs = [(rng.standard_normal((rows, K)) * scale).astype(np.float32) for _ in range(nb)]
    # a feature 1e6 times smaller than the rest and one that is exactly zero
    for x in xs:
        x[:, 3] *= 1e-6
        x[:, 5] = 0.0
    ref = _closed_form(xs)
    Hs = to_np(_split_H(G, xs))
    if K >= 1024:
        assert np.array_equal(Hs, to_np(G.accumulate_H(xs, split_fp16=True)))
    H32 = to_np(G.accumulate_H(xs))
    assert Hs.shape == (K, K) and Hs.dtype == np.float32 and np.array_equal(Hs, Hs.T)
    top = np.abs(ref).max()
    assert np.abs(Hs - ref).max() < TOL * top
    assert np.abs(Hs - H32).max() < 2 * TOL * top
    assert np.all(Hs[5] == 0) and np.all(Hs[:, 5] == 0)
    # the small feature keeps its relative accuracy on the diagonal
    assert abs(Hs[3, 3] - ref[3, 3]) < 1e-4 * ref[3, 3]
    # through gptq(): same codes as with the fp32 Hessian up to the usual handful of ties
    if K == 1280:
        W = (0.02 * rng.standard_normal((K, 256))).astype(np.float32)
        q1, p1 = G.gptq(W, xs)
        q2, p2 = G.gptq(W, xs, split_fp16=True)
        c1 = np.rint(to_np(q1) / to_np(p1["scale"]) + to_np(p1["zero"]))
        c2 = np.rint(to_np(q2) / to_np(p2["scale"]) + to_np(p2["zero"]))
        assert np.mean(c1 == c2) >= 0.999 and np.abs(c1 - c2).max() <= 1


def test_accumulate_H_split_fp16_falls_back_on_other_shapes(G):
    """Shapes outside the split path's requirements (K % 256, rows % 32, K >= 1024, fp32 rows) run on
    the ordinary kernels and give the ordinary result."""
    rng = np.random.default_rng(3)
    for rows, K in [(40, 1024), (64, 1000), (64, 768)]:
        xs = [rng.standard_normal((rows, K)).astype(np.float32) for _ in range(3)]
        assert np.array_equal(to_np(G.accumulate_H(xs, split_fp16=True)), to_np(G.accumulate_H(xs)))
    xs = [rng.standard_normal((64, 1024)).astype(np.float16) for _ in range(3)]
    assert np.array_equal(to_np(G.accumulate_H(xs, split_fp16=True)), to_np(G.accumulate_H(xs)))


def test_accumulate_H_split_fp16_empty_and_3d_batches(G):
    """An empty batch and a [4, 64, K] batch in the list: the empty one is skipped, the 3-D one is
    256 rows; rows that are all NaN-free but contain an infinity make H non-finite, as on the fp32 path."""
    rng = np.random.default_rng(21)
    K = 1024
    xs = [rng.standard_normal((64, K)).astype(np.float32), np.zeros((0, K), np.float32),
          rng.standard_normal((4, 64, K)).astype(np.float32)]
    ref = _closed_form([xs[0], xs[2]])
    Hs = to_np(G.accumulate_H(xs, split_fp16=True))
    assert np.abs(Hs - ref).max() < TOL * np.abs(ref).max()
    assert np.abs(Hs - to_np(G.accumulate_H(xs))).max() < 2 * TOL * np.abs(ref).max()
    xs[0][3, 7] = np.inf
    assert not np.isfinite(to_np(G.accumulate_H(xs, split_fp16=True))).all()


@pytest.mark.parametrize("rows,K,nb", [(48, 1024, 5), (2048, 1280, 2), (16, 2048, 3), (4096, 1024, 1), (272, 1536, 7)])
def test_accumulate_H_fp32_wide_tile_kernel(G, rows, K, nb):
    """fp32 rows with K a multiple of 256 (from 1024 on) and batches of a multiple of 16 rows run the
    256 x 256-tile kernel that loads straight into LDS; same bars as the 128 x 128-tile kernel, and
    a batch list that breaks the row rule (one batch of 40 rows) takes that kernel and agrees."""
    rng = np.random.default_rng(rows + K + nb)
    xs = [rng.standard_normal((rows, K)).astype(np.float32) for _ in range(nb)]
    for x in xs:
        x[:, 7] = 0.0
    H = to_np(G.accumulate_H(xs))
    ref = _closed_form(xs)
    assert H.shape == (K, K) and np.array_equal(H, H.T)
    assert np.abs(H - ref).max() < TOL * max(1.0, np.abs(ref).max())
    assert np.all(H[7] == 0) and np.all(H[:, 7] == 0)
    ragged = xs + [rng.standard_normal((40, K)).astype(np.float32)]
    ragged[-1][:, 7] = 0.0
    H2 = to_np(G.accumulate_H(ragged))
    ref2 = _closed_form(ragged)
    assert np.abs(H2 - ref2).max() < TOL * max(1.0, np.abs(ref2).max())
