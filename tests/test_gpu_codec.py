"""GPU parity of the int4 codec, dequantisation and column parameters: bit-exact."""
import numpy as np
import pytest

from helpers import to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import jax_gptq_amd.gptq as g
    return g


@pytest.mark.parametrize("shape,axis", [((256, 64), 0), ((256, 64), 1), ((6, 4, 10), 0),
                                        ((6, 4, 10), 1), ((6, 4, 10), 2), ((2, 1000, 3), 1),
                                        ((4096, 1), 0), ((2, 37), 0)])
def test_pack_unpack_bit_exact(G, shape, axis):
    rng = np.random.default_rng(0)
    w = rng.integers(0, 16, shape)
    for dt in (np.uint8, np.int32, np.int64):
        packed = to_np(G.pack_along_axis(axis, w.astype(dt)))
        ref = O.pack_along_axis(axis, w.astype(np.uint8))
        assert packed.dtype == np.uint8 and packed.shape == ref.shape
        assert np.array_equal(packed, ref)
    assert np.array_equal(to_np(G.unpack_along_axis(axis, ref)), w)


def test_pack_colwise_rowwise_reference_case(G):
    # reference tests.py:140-145
    rng = np.random.default_rng(0)
    w = rng.integers(0, 16, (256, 64))
    packed = G.pack_colwise(w)
    assert tuple(packed.shape) == (128, 64)
    assert np.array_equal(to_np(G.unpack_colwise(packed)), w)
    assert np.array_equal(to_np(G.unpack_rowwise(G.pack_rowwise(w))), w)
    assert np.array_equal(to_np(packed), O.pack_colwise(w))


def test_pack_errors(G):
    with pytest.raises(ValueError):
        G.pack_along_axis(2, np.zeros((4, 4), np.uint8))
    with pytest.raises(ValueError):
        G.pack_along_axis(0, np.zeros((3, 4), np.uint8))
    assert tuple(G.pack_along_axis(0, np.zeros((0, 4), np.uint8)).shape) == (0, 4)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("K,N", [(256, 64), (768, 3072), (130, 77)])
def test_col_params_bit_exact(G, dtype, K, N):
    rng = np.random.default_rng(1)
    w = (0.02 * rng.standard_normal((K, N))).astype(dtype)
    w[:, 0] = 0
    w[:, 1] = np.abs(w[:, 1]) + dtype(0.001)
    w[:, 2] = -np.abs(w[:, 2]) - dtype(0.001)
    got = G.get_col_quantize_params(w)
    ref = O.get_col_quantize_params(w.astype(np.float32))
    assert got["maxq"] == 15
    assert np.array_equal(to_np(got["scale"]), ref["scale"])
    assert np.array_equal(to_np(got["zero"]), ref["zero"])


def test_get_quantize_params_reference_vector(G):
    # reference tests.py:34-44
    w = np.asarray([[0.1, 0.2, 0.3, 0.4], [-0.1, -0.1, -0.1, -0.1]], dtype=np.float32)
    p = G.get_col_quantize_params(w)
    assert tuple(p["zero"].shape) == tuple(p["scale"].shape) == (4,)
    assert np.allclose(to_np(p["scale"]), (w[0, :] - w[1, :]) / 15)
    s = G.get_quantize_params(w[:, 3])
    r = O.get_quantize_params(w[:, 3])
    assert float(s["scale"]) == float(r["scale"]) and float(s["zero"]) == float(r["zero"])


@pytest.mark.parametrize("qdtype", [np.float32, np.float16])
def test_pack_matrix_and_unpack_matrix_bit_exact(G, qdtype):
    rng = np.random.default_rng(2)
    K, N = 256, 96
    w = rng.standard_normal((K, N)).astype(np.float32)
    p = O.get_col_quantize_params(w)
    q = O.quantize_value(p["zero"], p["scale"], 15, w).astype(qdtype)
    ref = O.pack_matrix(q, p)
    got = G.pack_matrix(q, p)
    assert got.contraction_axis == 0 and got.shape == (K, N)
    assert np.array_equal(to_np(got.int_weight), ref.int_weight)
    dense = to_np(G.unpack_matrix(got))
    assert dense.dtype == np.float32
    assert np.array_equal(dense, O.unpack_matrix(ref))
    if qdtype == np.float32:
        assert np.array_equal(dense, q)          # reference tests.py:147-156


def test_pack_matrix_other_axis_and_fp16_params(G):
    rng = np.random.default_rng(3)
    codes = rng.integers(0, 16, (5, 64, 7)).astype(np.uint8)
    scale = rng.uniform(0.001, 0.01, (5, 7)).astype(np.float32)
    zero = rng.integers(0, 16, (5, 7)).astype(np.float32)
    q = (scale[:, None, :] * (codes.astype(np.float32) - zero[:, None, :])).astype(np.float32)
    got = G.pack_matrix(q, {"scale": scale, "zero": zero}, contraction_axis=1)
    ref = O.pack_matrix(q, {"scale": scale, "zero": zero}, contraction_axis=1)
    assert np.array_equal(to_np(got.int_weight), ref.int_weight)
    assert np.array_equal(to_np(G.unpack_matrix(got)), O.unpack_matrix(ref))
    # fp16 scale/zero: the dense matrix is computed in fp16, as the reference does
    qm16 = O.QuantizedMatrix(ref.int_weight, zero.astype(np.float16), scale.astype(np.float16), 1)
    assert np.array_equal(to_np(G.unpack_matrix(qm16)), O.unpack_matrix(qm16))
