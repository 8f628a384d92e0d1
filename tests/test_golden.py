"""The fixtures under tests/golden: known-answer content of the reference's own tests (data only)
and one small layer solved by the oracle.  CPU part: the oracle reproduces both files exactly.
GPU part: the HIP path against the same files (codes, packed bytes and parameters to the bars the
other parity tests use)."""
import json
import os

import numpy as np
import pytest

from oracle import gptq_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def vectors():
    with open(os.path.join(GOLD, "reference_test_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def layer():
    with np.load(os.path.join(GOLD, "oracle_small_layer.npz")) as z:
        return {k: z[k] for k in z.files}


def test_oracle_reproduces_reference_test_vectors(vectors):
    v = vectors["get_col_quantize_params"]
    p = O.get_col_quantize_params(np.asarray(v["w"], dtype=np.float32))
    assert np.allclose(p["scale"], v["scale"], rtol=1e-7, atol=0)
    assert np.array_equal(np.asarray(p["zero"]), np.asarray(v["zero"], dtype=np.float32))
    v = vectors["pack_colwise"]
    codes = np.asarray(v["codes"], dtype=np.uint8)
    packed = np.asarray(O.pack_colwise(codes))
    assert np.array_equal(packed, np.asarray(v["packed"], dtype=np.uint8))
    assert np.array_equal(np.asarray(O.unpack_colwise(packed)), codes)
    v = vectors["quantize_value"]
    vals = np.asarray(v["v"], dtype=np.float32)
    deq = O.quantize_value(np.float32(v["zero"]), np.float32(v["scale"]), 15, vals)
    assert np.array_equal(np.asarray(deq), np.float32(v["scale"]) * (np.asarray(v["q"], dtype=np.float32) - np.float32(v["zero"])))


def test_oracle_reproduces_small_layer_fixture(layer):
    xs = [layer["x0"], layer["x1"]]
    p = O.get_col_quantize_params(layer["W"])
    assert np.array_equal(np.asarray(p["scale"]), layer["scale"]) and np.array_equal(np.asarray(p["zero"]), layer["zero"])
    assert np.allclose(np.asarray(O.accumulate_H(xs)), layer["H"], rtol=1e-6, atol=1e-7)
    Q, pp = O.gptq(layer["W"], xs, block_size=int(layer["block_size"]))
    assert np.array_equal(O.codes_from_q(Q, pp).astype(np.uint8), layer["codes"])
    assert np.array_equal(np.asarray(O.pack_matrix(Q, pp).int_weight), layer["packed"])
    # the fixture is self-consistent: packed bytes are the codes, codes are on the grid of Q
    assert np.array_equal(np.asarray(O.unpack_colwise(layer["packed"])), layer["codes"])
    assert np.allclose(layer["Q"], layer["scale"][None] * (layer["codes"].astype(np.float32) - layer["zero"][None]),
                       rtol=0, atol=1e-7)


@pytest.mark.gpu
def test_hip_path_against_reference_test_vectors(vectors):
    import jax_gptq_amd.gptq as G
    from helpers import to_np
    v = vectors["get_col_quantize_params"]
    p = G.get_col_quantize_params(np.asarray(v["w"], dtype=np.float32))
    assert np.allclose(to_np(p["scale"]), v["scale"], rtol=1e-7, atol=0)
    assert np.array_equal(to_np(p["zero"]), np.asarray(v["zero"], dtype=np.float32))
    v = vectors["pack_colwise"]
    codes = np.asarray(v["codes"], dtype=np.uint8)
    packed = to_np(G.pack_colwise(codes))
    assert np.array_equal(packed, np.asarray(v["packed"], dtype=np.uint8))
    assert np.array_equal(to_np(G.unpack_colwise(packed)), codes)


@pytest.mark.gpu
def test_hip_path_against_small_layer_fixture(layer):
    import jax_gptq_amd.gptq as G
    from helpers import to_np
    xs = [layer["x0"], layer["x1"]]
    p = G.get_col_quantize_params(layer["W"])
    assert np.allclose(to_np(p["scale"]), layer["scale"], rtol=1e-5, atol=0)
    assert np.array_equal(to_np(p["zero"]), layer["zero"])
    H = to_np(G.accumulate_H(xs))
    assert np.abs(H - layer["H"]).max() < 2e-5 * np.abs(layer["H"]).max()
    Q, pp = G.gptq(layer["W"], xs, block_size=int(layer["block_size"]))
    packed = G.pack_matrix(Q, pp)
    codes = to_np(G.unpack_colwise(packed.int_weight))
    diff = codes.astype(np.int32) - layer["codes"].astype(np.int32)
    assert np.mean(diff != 0) <= 1e-3 and np.abs(diff).max() <= 1
    # packing is exact: the bytes are the codes the solve produced
    assert np.array_equal(to_np(packed.int_weight), np.asarray(O.pack_colwise(codes)))
