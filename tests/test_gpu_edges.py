"""Edge cases of the path on the GPU: degenerate shapes, empty inputs, rank-deficient
calibration, all-zero weights; each against the oracle or a closed form."""
import numpy as np
import pytest

from helpers import code_stats, to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import jax_gptq_amd.gptq as g
    return g


@pytest.fixture(scope="module")
def OP():
    import jax_gptq_amd.op as op
    return op


def test_single_output_channel_and_single_block(G):
    rng = np.random.default_rng(0)
    W = rng.standard_normal((128, 1)).astype(np.float32)
    X = rng.standard_normal((512, 128)).astype(np.float32)
    Q, p = G.gptq(W, [X])
    Qr, pr = O.gptq(W, [X])
    frac, mx = code_stats(O.codes_from_q(to_np(Q), pr), O.codes_from_q(Qr, pr))
    assert frac <= 0.02 and mx <= 1          # 128 codes in all
    assert np.allclose(to_np(p["scale"]), pr["scale"], rtol=1e-6)


def test_smallest_matrix(G):
    W = np.array([[0.3, -0.2], [-0.7, 0.9]], np.float32)
    X = np.array([[1.0, 0.5], [0.25, -1.0], [2.0, 1.0]], np.float32)
    Q, p = G.gptq(W, [X], block_size=2)
    Qr, pr = O.gptq(W, [X], block_size=2)
    assert np.allclose(to_np(Q), Qr, atol=1e-6)
    packed = G.pack_matrix(Q, p)
    assert tuple(packed.int_weight.shape) == (1, 2)
    assert np.array_equal(to_np(G.unpack_matrix(packed)), to_np(Q))


def test_rank_deficient_calibration_needs_the_damping(G):
    """Fewer calibration rows than features: H is singular, the damping makes it invertible."""
    rng = np.random.default_rng(1)
    W = (0.02 * rng.standard_normal((256, 64))).astype(np.float32)
    X = rng.standard_normal((8, 256)).astype(np.float32)
    Q, p = G.gptq(W, [X])
    Qr, pr = O.gptq(W, [X])
    frac, mx = code_stats(O.codes_from_q(to_np(Q), pr), O.codes_from_q(Qr, pr))
    assert frac <= 5e-3 and mx <= 1
    with pytest.raises(ValueError):
        G.gptq(W, [X], damping=0.0)          # singular without damping: NaN -> ValueError (gptq.py:194-196)


def test_all_zero_weights_and_all_zero_calibration(G):
    W = np.zeros((128, 32), np.float32)
    X = np.random.default_rng(2).standard_normal((64, 128)).astype(np.float32)
    Q, p = G.gptq(W, [X])
    assert np.all(to_np(Q) == O.gptq(W, [X])[0])
    # every feature dead: H becomes the identity, W rows are zeroed, nothing fails (gptq.py:157-159)
    W2 = np.random.default_rng(3).standard_normal((128, 32)).astype(np.float32)
    Q2, p2 = G.gptq(W2, [np.zeros((16, 128), np.float32)])
    Qr2, pr2 = O.gptq(W2, [np.zeros((16, 128), np.float32)])
    assert np.array_equal(to_np(Q2), Qr2)


def test_empty_and_ragged_calibration_lists(G):
    W = np.ones((64, 8), np.float32)
    with pytest.raises((ValueError, IndexError)):
        G.gptq(W, [], block_size=64)
    rng = np.random.default_rng(4)
    xs = [rng.standard_normal((n, 64)).astype(np.float32) for n in (1, 0, 7, 130, 0, 3)]
    H = to_np(G.accumulate_H(xs))
    flat = np.concatenate(xs).astype(np.float64)
    assert np.abs(H - flat.T @ flat / flat.shape[0]).max() < 2e-5
    assert np.abs(H - O.accumulate_H(xs)).max() < 4e-5


def test_matmul_with_no_rows_and_one_packed_row(OP, G):
    import torch
    codes = np.random.default_rng(5).integers(0, 16, (2, 48)).astype(np.uint8)
    qm = O.QuantizedMatrix(O.pack_colwise(codes), np.full(48, 8, np.float16), np.full(48, 0.5, np.float16))
    x0 = torch.zeros((0, 2), dtype=torch.float16)
    y0 = OP.quantized_matmul(x0, qm)
    assert tuple(y0.shape) == (0, 48)
    x = np.array([[1.0, -2.0]], np.float16)
    y = to_np(OP.quantized_matmul(x, qm)).astype(np.float32)
    ref = x.astype(np.float32) @ ((codes.astype(np.float32) - 8.0) * 0.5)
    assert np.allclose(y, ref, atol=1e-2)


def test_pack_unpack_maximum_codes_and_odd_axis_error(G):
    codes = np.full((6, 5), 15, np.uint8)
    packed = to_np(G.pack_colwise(codes))
    assert packed.shape == (3, 5) and np.all(packed == 0xFF)
    assert np.array_equal(to_np(G.unpack_colwise(packed)), codes)
    with pytest.raises(ValueError):
        G.pack_colwise(np.zeros((5, 4), np.uint8))
    assert to_np(G.pack_colwise(np.zeros((0, 4), np.uint8))).shape == (0, 4)


def test_qmatmul_split_sum_range():
    """The decode path sums the splits of the contraction in 64-bit fixed-point cells: a PARTIAL result beyond
    +-65536 poisons its cell and the output is NaN, also where the partial sums would cancel (the reference's fp32
    accumulation would give the finite sum there, and +-inf where the result itself leaves the fp16 range).  Partials
    just inside the range are summed exactly."""
    import torch
    import jax_gptq_amd.gptq as G
    from jax_gptq_amd.op import quantized_matmul
    from jax_gptq_amd import _native as N
    K, C = 4096, 512
    plan = N.qmatmul_plan(1, K // 2, C)
    assert plan["kernel"] == "qmm_fwd_dec_kernel" and plan["splits"] > 1
    pk = torch.full((K // 2, C), 0x88, dtype=torch.uint8, device="cuda")          # every code 8
    zero = torch.zeros(C, device="cuda")
    scale = torch.ones(C, device="cuda")
    qm = G.QuantizedMatrix(pk, zero, scale)
    # first half of the contraction +v, second half -v: a split's partial is +-8 v times its K / S columns, the sum 0
    half = K // 2
    for v, poisoned in ((4.0, False), (64.0, True)):
        x = torch.cat([torch.full((1, half), v), torch.full((1, half), -v)], dim=1).to(torch.float16).cuda()
        y = quantized_matmul(x, qm).float()
        if poisoned:
            assert 8 * v * (K // plan["splits"]) > 65536 * 0.9
            assert bool(torch.isnan(y).all())
        else:
            assert 8 * v * (K // plan["splits"]) < 65536
            assert bool((y == 0).all())
    # a further call on the same (cached) workspace finds clean cells
    x = torch.ones((1, K), dtype=torch.float16, device="cuda") / 64
    y = quantized_matmul(x, qm).float()
    assert bool((y == 8.0 * K / 64).all())
