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


@pytest.mark.parametrize("rows,K,nb", [(2048, 4096, 1), (2048, 6144, 1), (16, 1024, 1), (32, 1024, 1), (160, 2048, 3),
                                       (1024, 1024, 2), (2048, 11008, 1), (4096, 4096, 2), (2064, 4096, 1)])
def test_accumulate_H_short_calls_in_equal_runs_of_tile_slabs(G, rows, K, nb):
    """A short call (the reference's one call per batch, gptq.py:97-98) is dealt to one round of workgroups as
    equal runs of (tile, 16-row slab) pairs: a run ends one tile, covers whole tiles and begins another.  Cases:
    136 tiles on 256 workgroups (every tile cut), 300 and 946 tiles (whole tiles inside the runs), fewer pairs than
    workgroups (one workgroup per few tiles), several batches per call, rows that are no multiple of the runs.
    Against the closed form in double, symmetric, the same bits on a second call, and a second call ADDS."""
    import torch
    rng = np.random.default_rng(rows + K + nb)
    xs = [rng.standard_normal((rows, K)).astype(np.float32) for _ in range(nb)]
    for x in xs:
        x[:, 5] = 0.0
    dev = [torch.from_numpy(x).cuda() for x in xs]
    H = to_np(G.accumulate_H(dev))
    ref = _closed_form(xs)
    assert H.shape == (K, K) and np.array_equal(H, H.T)
    assert np.abs(H - ref).max() < TOL * max(1.0, np.abs(ref).max())
    assert np.all(H[5] == 0) and np.all(H[:, 5] == 0)
    assert np.array_equal(H, to_np(G.accumulate_H(dev)))
    # two steps of the chain over the same rows: twice the sums over twice the rows
    Hs = torch.zeros((K, K), dtype=torch.float32, device="cuda")
    mean = torch.zeros((K,), dtype=torch.float32, device="cuda")
    Hs, mean, n = G._accumulate_H_step(Hs, mean, 0, dev[0])
    Hs, mean, n = G._accumulate_H_step(Hs, mean, n, dev[0])
    assert n == 2 * rows
    ref1 = _closed_form(xs[:1])
    assert np.abs(to_np(Hs) / n - ref1).max() < TOL * max(1.0, np.abs(ref1).max())


@pytest.mark.parametrize("rows,K,nb,dt", [(2048, 4096, 1, "float16"), (2048, 4096, 1, "bfloat16"), (2048, 6144, 1, "float16"),
                                          (32, 1024, 1, "float16"), (64, 1024, 1, "bfloat16"), (160, 2048, 3, "float16"),
                                          (1024, 1024, 2, "bfloat16"), (2048, 11008, 1, "float16"),
                                          (4096, 4096, 2, "float16"), (2080, 4096, 1, "bfloat16"), (512, 4096, 1, "float16")])
def test_accumulate_H_short_16bit_calls_in_equal_runs_of_tile_slabs(G, rows, K, nb, dt):
    """The same partition for fp16 / bf16 batches (32-row slabs): every tile cut, whole tiles inside the runs,
    fewer pairs than workgroups, several batches per call, slab counts that the runs do not divide.  Products of
    two 16-bit numbers are exact in fp32, so the bar is the closed form of the widened rows to fp32 summation
    error; a zero feature gives exact zeros; the same bits on a second call; a second step ADDS."""
    import torch
    rng = np.random.default_rng(rows + K + nb)
    tdt = getattr(torch, dt)
    dev = [torch.from_numpy(rng.standard_normal((rows, K)).astype(np.float32)).to(tdt).cuda() for _ in range(nb)]
    for x in dev:
        x[:, 5] = 0.0
    xs = [x.float().cpu().numpy() for x in dev]
    H = to_np(G.accumulate_H(dev))
    ref = _closed_form(xs)
    assert H.shape == (K, K) and np.array_equal(H, H.T)
    assert np.abs(H - ref).max() < TOL * max(1.0, np.abs(ref).max())
    assert np.all(H[5] == 0) and np.all(H[:, 5] == 0)
    assert np.array_equal(H, to_np(G.accumulate_H(dev)))
    Hs = torch.zeros((K, K), dtype=torch.float32, device="cuda")
    mean = torch.zeros((K,), dtype=torch.float32, device="cuda")
    Hs, mean, n = G._accumulate_H_step(Hs, mean, 0, dev[0])
    Hs, mean, n = G._accumulate_H_step(Hs, mean, n, dev[0])
    assert n == 2 * rows
    ref1 = _closed_form(xs[:1])
    assert np.abs(to_np(Hs) / n - ref1).max() < TOL * max(1.0, np.abs(ref1).max())


@pytest.mark.parametrize("rows,K,nb,dt", [(64, 384, 5, "float32"), (37, 200, 4, "float32"), (256, 1024, 6, "float32"),
                                          (2048, 4096, 3, "float32"), (96, 1280, 4, "float16"),
                                          (50, 520, 3, "bfloat16")])
def test_accumulate_H_step_chain_equals_accumulate_H(G, rows, K, nb, dt):
    """The reference's streaming use (gptq.py:97-101): one `_accumulate_H_step` per batch, then the
    closing formula H / n + outer(mean, mean).  After every step the state must be a full symmetric
    matrix (K > one tile: the kernels add to the upper tiles only), the closed state must equal
    what `accumulate_H` returns for the list, and the factor computed from it the one-shot factor."""
    import torch
    rng = np.random.default_rng(rows + K + nb)
    tdt = getattr(torch, dt)
    xs = [torch.from_numpy(rng.standard_normal((rows, K)).astype(np.float32)).to(tdt).cuda() for _ in range(nb)]
    H = torch.zeros((K, K), dtype=torch.float32, device="cuda")
    mean = torch.zeros(K, dtype=torch.float32, device="cuda")
    n = 0
    seen = []
    for x in xs:
        H, mean, n = G._accumulate_H_step(H, mean, n, x)
        seen.append(x.float().cpu().numpy())
        part = np.concatenate(seen)
        raw = part.astype(np.float64).T @ part.astype(np.float64)
        Hn = to_np(H)
        assert np.array_equal(Hn, Hn.T), "the state is not symmetric after a step"
        assert np.abs(Hn - raw).max() < TOL * max(1.0, np.abs(raw).max())
    assert n == rows * nb
    closed = H / n + torch.outer(mean, mean)          # gptq.py:100-101
    one_shot = G.accumulate_H(xs)
    ref = _closed_form([x.float().cpu().numpy() for x in xs])
    assert np.abs(to_np(closed) - ref).max() < TOL * max(1.0, np.abs(ref).max())
    assert np.abs(to_np(closed) - to_np(one_shot)).max() < TOL * max(1.0, np.abs(ref).max())
    if rows * nb >= K:
        # the streamed matrix is as good an input to the factorisation as the one-shot matrix
        _, L1, bad1 = G._damp_and_invert(torch.zeros((K, 8), device="cuda"), closed.clone(), 0.01)
        _, L2, bad2 = G._damp_and_invert(torch.zeros((K, 8), device="cuda"), one_shot.clone(), 0.01)
        assert not bad1 and not bad2
        assert float((L1 - L2).abs().max()) < 1e-3 * float(L2.abs().max())


def test_accumulate_H_step_completes_the_lower_triangle_when_it_is_looked_at(G):
    """A chain of steps pays for ONE mirror into the lower triangle: the state a step returns completes itself when
    anything but the next step looks at its values (a torch function, the address handed to a kernel), and shape
    or type queries do not count as looking."""
    import torch
    K, rows = 1024, 256
    g = torch.Generator(device="cuda").manual_seed(3)
    xs = [torch.randn((rows, K), device="cuda", generator=g) for _ in range(4)]
    ref = sum(x.double().T @ x.double() for x in xs)

    def chain():
        H = torch.zeros((K, K), device="cuda")
        m, n = torch.zeros(K, device="cuda"), 0
        for x in xs:
            H, m, n = G._accumulate_H_step(H, m, n, x)
        return H, n

    H, n = chain()
    assert n == 4 * rows and tuple(H.shape) == (K, K) and H.dtype == torch.float32 and H.dim() == 2 and H.is_cuda
    assert H._pending                                   # nothing above looked at the values
    full = H.clone()                                    # a torch function: completes first
    assert not H._pending and type(full) is torch.Tensor
    assert torch.equal(full, full.T)
    assert float((full.double() - ref).abs().max()) < 2e-5 * float(ref.abs().max())
    # the address (what the library's own entry points take) completes as well
    H2, _ = chain()
    assert H2._pending
    H2.data_ptr()
    assert not H2._pending
    torch.cuda.synchronize()
    assert torch.equal(H2.clone(), full)
    # a further step after a look, and the closing formula and solve on a state nobody looked at
    H3, n3 = chain()
    Q1, _ = G.gptq(torch.randn((K, 64), device="cuda", generator=g) * 0.02, None, H=H3 / n3)
    H4, _ = chain()
    H4.sum()
    H4, _, n4 = G._accumulate_H_step(H4, torch.zeros(K, device="cuda"), n, xs[0])
    assert H4._pending and n4 == 5 * rows
    ref5 = ref + xs[0].double().T @ xs[0].double()
    assert float((H4.double() - ref5).abs().max()) < 2e-5 * float(ref5.abs().max())
    assert torch.equal(H4.clone(), H4.clone().T)


def test_accumulate_H_step_takes_3d_and_empty_batches(G):
    import torch
    rng = np.random.default_rng(5)
    K = 256
    a = rng.standard_normal((3, 11, K)).astype(np.float32)
    H = torch.zeros((K, K), dtype=torch.float32, device="cuda")
    H, m, n = G._accumulate_H_step(H, torch.zeros(K, device="cuda"), 0, a)
    H, m, n = G._accumulate_H_step(H, m, n, np.zeros((0, K), np.float32))
    assert n == 33
    flat = a.reshape(-1, K).astype(np.float64)
    assert np.abs(to_np(H) - flat.T @ flat).max() < TOL * np.abs(flat.T @ flat).max()
    with pytest.raises(ValueError):
        G._accumulate_H_step(H, m, n, np.zeros((4, K + 1), np.float32))


@pytest.mark.parametrize("nb,rows,K", [(300, 16, 256), (1100, 4, 136), (260, 32, 1024)])
def test_accumulate_H_long_batch_lists(G, nb, rows, K):
    """More batches than one launch table holds (128) and than one call of the binding passes
    (1024): the list is cut into several launches that add into the same H."""
    rng = np.random.default_rng(nb)
    xs = [rng.standard_normal((rows, K)).astype(np.float32) for _ in range(nb)]
    H = to_np(G.accumulate_H(xs))
    ref = _closed_form(xs)
    assert np.array_equal(H, H.T)
    assert np.abs(H - ref).max() < TOL * max(1.0, np.abs(ref).max())


def test_accumulate_H_mixed_dtype_batch_list(G):
    """fp32, fp16 and bf16 batches in one list (one launch table holds one element type, so the
    binding falls back to a launch per batch); the closed form is taken of the values as stored."""
    import torch
    rng = np.random.default_rng(31)
    K = 1024
    dts = [torch.float32, torch.float16, torch.float32, torch.bfloat16, torch.float16]
    xs = [torch.from_numpy(rng.standard_normal((64 + 32 * i, K)).astype(np.float32)).to(dt).cuda()
          for i, dt in enumerate(dts)]
    H = to_np(G.accumulate_H(xs))
    ref = _closed_form([x.float().cpu().numpy() for x in xs])
    assert np.array_equal(H, H.T)
    assert np.abs(H - ref).max() < TOL * max(1.0, np.abs(ref).max())


def test_accumulate_H_full_calibration_set_of_the_benchmark_layer(G):
    """The launch the benchmark times: 128 batches of [2048, 4096] fp32 rows (262144 tokens, the
    full 128-entry pointer table, every row slice) against a double-precision product of the same
    rows formed on the device batch by batch (test-only: torch's fp64 matmul)."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(4096)
    K, nb, rows = 4096, 128, 2048
    xs = [torch.randn((rows, K), generator=g, device="cuda") for _ in range(nb)]
    H = G.accumulate_H(xs)
    ref = torch.zeros((K, K), dtype=torch.float64, device="cuda")
    for x in xs:
        xd = x.double()
        ref.addmm_(xd.T, xd)
    ref /= nb * rows
    assert bool((H == H.T).all())
    top = float(ref.abs().max())
    assert float((H.double() - ref).abs().max()) < TOL * max(1.0, top)
    # fp16 copies of the same rows on the 16-bit kernel, against the product of the rounded rows
    xs16 = [x.to(torch.float16) for x in xs]
    del xs
    H16 = G.accumulate_H(xs16)
    ref.zero_()
    for x in xs16:
        xd = x.double()
        ref.addmm_(xd.T, xd)
    ref /= nb * rows
    assert float((H16.double() - ref).abs().max()) < TOL * max(1.0, top)
