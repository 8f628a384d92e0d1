"""Grouped scales / zero points (an extension with no counterpart in the reference, specified by the oracle's
``_group_size`` option, which tests/test_oracle.py pins): solve, packing and the packed matmul in both
directions against the oracle.  Tolerances as for the per-channel path."""
import numpy as np
import pytest

from helpers import code_stats, recon_error, to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 1e-3


@pytest.fixture(scope="module")
def G():
    import jax_gptq_amd.gptq as g
    return g


@pytest.fixture(scope="module")
def OP():
    import jax_gptq_amd.op as op
    return op


@pytest.mark.parametrize("K,N,g,bits", [(512, 320, 128, 4), (1024, 200, 256, 4), (1024, 136, 512, 4),
                                         (256, 160, 128, 8), (768, 3072, 128, 4)])
def test_gptq_grouped_against_the_oracle(G, K, N, g, bits):
    rng = np.random.default_rng(K + N + g)
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    X = (rng.standard_normal((2048, K)) * (1.0 + rng.random(K))).astype(np.float32)
    Q, p = G.gptq(W, [X], group_size=g, bits=bits)
    Qr, pr = O.gptq(W, [X], _group_size=g, _bits=bits)
    assert p["group_size"] == g and tuple(p["scale"].shape) == (K // g, N)
    # group 0 sees the original rows: exact; later groups see rows corrected in a different summation order
    assert np.array_equal(to_np(p["scale"])[0], pr["scale"][0]) and np.array_equal(to_np(p["zero"])[0], pr["zero"][0])
    # a code that differs from the oracle's (one in a thousand) moves the corrected rows below it in its column,
    # and with them that column's later group ranges: a few columns deviate, none by much
    sc, scr = to_np(p["scale"]), pr["scale"]
    assert np.mean(~np.isclose(sc, scr, rtol=1e-5)) <= 0.02 and np.max(np.abs(sc - scr) / scr) <= 0.1
    assert np.mean(to_np(p["zero"]) != pr["zero"]) <= 5e-3
    packed = G.pack_matrix(Q, p)
    assert packed.group_size == g and packed.bits == bits and packed.shape == (K, N)
    ref_packed = O.pack_matrix(Qr, pr)
    if bits == 4:
        c = O.unpack_colwise(to_np(packed.int_weight)).astype(np.int32)
        cr = O.unpack_colwise(ref_packed.int_weight).astype(np.int32)
    else:
        c, cr = to_np(packed.int_weight).astype(np.int32), ref_packed.int_weight.astype(np.int32)
    same_grid = np.repeat(to_np(p["zero"]) == pr["zero"], g, 0) & np.repeat(to_np(p["scale"]) == pr["scale"], g, 0)
    frac, mx = code_stats(c[same_grid], cr[same_grid])
    assert frac <= (1e-3 if bits == 4 else 2e-2) and mx <= 1, (frac, mx)
    e, er = recon_error(W, to_np(Q), X), recon_error(W, Qr, X)
    assert abs(e - er) <= 0.01 * er
    # pack -> unpack returns the solve's output
    assert np.array_equal(to_np(G.unpack_matrix(packed)), to_np(Q))
    # grouped parameters fit at least as well as per-channel ones on this data
    e0 = recon_error(W, to_np(G.gptq(W, [X], bits=bits)[0]), X)
    assert e < e0


def test_gptq_grouped_argument_checks(G):
    rng = np.random.default_rng(0)
    W = rng.standard_normal((256, 32)).astype(np.float32)
    X = rng.standard_normal((512, 256)).astype(np.float32)
    with pytest.raises(ValueError):
        G.gptq(W, [X], group_size=96)
    with pytest.raises(ValueError):
        G.gptq(W, [X], group_size=128, actorder=True)
    with pytest.raises(ValueError):
        G.gptq(W, [X], group_size=1024)


def _grouped_matrix(seed, K, N, g, bits, zs="float32", frac=False):
    import torch
    import jax_gptq_amd.gptq as Gm
    rng = np.random.default_rng(seed)
    top = 16 if bits == 4 else 256
    codes = rng.integers(0, top, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.001, 0.01, (K // g, N)).astype(np.float32) / (1 if bits == 4 else 16)).to(tdt)
    zero = torch.from_numpy((rng.uniform(0, top - 1, (K // g, N)) if frac else rng.integers(0, top, (K // g, N)))
                            .astype(np.float32)).to(tdt)
    iw = O.pack_colwise(codes) if bits == 4 else codes
    ref = O.QuantizedMatrix(iw, zero.float().numpy(), scale.float().numpy(), bits=bits, group_size=g)
    qm = Gm.QuantizedMatrix(torch.from_numpy(iw).cuda(), zero.cuda(), scale.cuda(), bits=bits, group_size=g)
    dense = (codes.astype(np.float64) - np.repeat(zero.double().numpy(), g, 0)) * np.repeat(scale.double().numpy(), g, 0)
    return qm, ref, dense


def _check(got, ref, atol=ATOL, rtol=RTOL):
    got = to_np(got).astype(np.float64)
    assert got.shape == ref.shape
    err = np.abs(got - ref)
    bad = err > atol + rtol * np.abs(ref)
    assert not bad.any(), f"{bad.sum()} of {bad.size} off, max err {err.max():.3e}, first {np.argwhere(bad)[0]}"


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("xdt", ["float16", "bfloat16", "float32"])
@pytest.mark.parametrize("M,N,K,g,bits", [(1, 4096, 4096, 128, 4), (16, 1024, 2048, 128, 4), (100, 909, 512, 128, 4),
                                           (300, 2304, 768, 256, 4), (5, 1000, 520 * 0 + 512, 64, 4),
                                           (40, 640, 1024, 128, 8), (3, 4, 64, 32, 4), (70, 200, 96, 32, 4)])
def test_qmatmul_grouped(OP, M, N, K, g, bits, xdt, transpose):
    import torch
    qm, ref, dense = _grouped_matrix(M + N + K + g, K, N, g, bits, frac=(M % 2 == 0))
    rng = np.random.default_rng(3)
    x32 = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0)).astype(np.float32)
    x = torch.from_numpy(x32).to(getattr(torch, xdt))
    got = OP.quantized_matmul(x, qm, transpose_b=transpose)
    assert got.dtype == x.dtype
    want = x.double().numpy() @ (dense.T if transpose else dense)
    # the grouped kernels form (code - zero) * scale in the activations' 16-bit type before the product
    rtol = {"float16": 2 * RTOL, "float32": 3 * RTOL, "bfloat16": 2.0 ** -7}[xdt]
    if xdt == "bfloat16" and not transpose:
        # bf16 weights carry 8 bits (as a dense bf16 matrix would): every term is off by up to 2^-9, random in
        # sign, so an output's error has standard deviation 2^-9 / sqrt(3) * ||x * w||_2; eight of them allowed
        xd = x.double().numpy()
        sigma = 2.0 ** -9 / np.sqrt(3.0) * np.sqrt((xd ** 2) @ (dense ** 2))
        err = np.abs(to_np(got).astype(np.float64) - want)
        assert np.all(err <= ATOL + rtol * np.abs(want) + 8 * sigma), float((err - 8 * sigma).max())
    else:
        _check(got, want, rtol=rtol)
    # and agree with the dense product of unpack_matrix
    import jax_gptq_amd.gptq as Gm
    assert np.allclose(to_np(Gm.unpack_matrix(qm)), dense, rtol=1e-5, atol=1e-7)


def test_qmatmul_grouped_gradient_and_zs_types(OP):
    import torch
    for zs in ("float16", "bfloat16"):
        qm, ref, dense = _grouped_matrix(11, 512, 384, 128, 4, zs=zs)
        x = torch.randn((20, 512), device="cuda", dtype=torch.float16, requires_grad=True)
        y = OP.quantized_matmul(x, qm)
        _check(y.detach(), x.detach().double().cpu().numpy() @ dense, rtol=2 * RTOL)
        w = torch.randn_like(y) * 0.05
        (y * w).sum().backward()
        _check(x.grad, w.double().cpu().numpy() @ dense.T, rtol=2 * RTOL)


def test_quantize_driver_with_groups(G, OP):
    """quantize(..., group_size=128) on a two-layer function equals the chain of grouped gptq() calls."""
    import torch
    from jax_gptq_amd import quantize, use_quantized
    rng = np.random.default_rng(2)
    w1 = (0.05 * rng.standard_normal((256, 384))).astype(np.float32)
    w2 = (0.05 * rng.standard_normal((384, 128))).astype(np.float32)
    xs = [rng.standard_normal((64, 256)).astype(np.float32) for _ in range(4)]

    def fn(params, x):
        return torch.relu(x @ params["w1"]) @ params["w2"]

    out = quantize(fn, {"w1": w1, "w2": w2}, xs, group_size=128)
    Q1, p1 = G.gptq(w1, xs, group_size=128)
    hs = [torch.relu(torch.from_numpy(x).cuda() @ Q1) for x in xs]
    Q2, p2 = G.gptq(w2, hs, group_size=128)
    assert out["w1"].group_size == 128 and out["w2"].group_size == 128
    assert np.array_equal(to_np(out["w1"].int_weight), to_np(G.pack_matrix(Q1, p1).int_weight))
    assert np.array_equal(to_np(out["w2"].int_weight), to_np(G.pack_matrix(Q2, p2).int_weight))
    x = torch.from_numpy(xs[0]).cuda().half()
    y = use_quantized(fn, use_kernel=True)(out, x)
    y_ref = torch.relu(x.float() @ Q1) @ Q2
    assert torch.allclose(y.float(), y_ref, atol=2e-2, rtol=1e-2)
