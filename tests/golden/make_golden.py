"""Writes the fixtures of this folder.  Run from the repository root: python tests/golden/make_golden.py

reference_test_vectors.json  known-answer content of the reference's own tests, transcribed as data
                             (inputs and the values its assertions fix), with the lines it comes from;
oracle_small_layer.npz       one small seeded layer solved by the oracle (oracle/gptq_oracle.py): inputs and
                             every intermediate the parity tests compare (scale, zero, Hessian, codes, packed
                             bytes), so that a change of the oracle or of a kernel shows up against a fixed file.
Nothing here imports or runs the reference.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle import gptq_oracle as O   # noqa: E402


def reference_vectors():
    w = np.array([[0.1, 0.2, 0.3, 0.4], [-0.1, -0.1, -0.1, -0.1]], dtype=np.float32)
    scale = (w[0] - w[1]) / np.float32(15)                       # the assertion of tests.py:44
    return {
        "get_col_quantize_params": {
            "source": "tests.py:35-44 (w and the asserted scale); zero follows gptq.py:114-116",
            "w": w.tolist(),
            "scale": [float(v) for v in scale],
            "zero": [float(v) for v in np.rint(np.float32(0.1) / scale)],
        },
        "pack_colwise": {
            "source": "gptq.py:247 (byte = c[2j] | c[2j+1] << 4), read back in that order by kernel.py:92-104; "
                      "round trip asserted by tests.py:140-145",
            "codes": [[1, 15, 0], [2, 0, 7], [15, 15, 9], [0, 1, 8]],
            "packed": [[0x21, 0x0F, 0x70], [0x0F, 0x1F, 0x89]],
        },
        "quantize_value": {
            "source": "gptq.py:120-128: clip(rint(v / scale) + zero, 0, 15), dequantised scale * (q - zero); "
                      "ties to even",
            "scale": 0.5, "zero": 3.0,
            "v": [-10.0, -1.5, -1.25, -0.75, -0.25, 0.0, 0.25, 0.75, 1.25, 5.9, 6.0, 100.0],
            "q": [0, 0, 1, 1, 3, 3, 3, 5, 5, 15, 15, 15],
        },
        "kernel_shapes": {"source": "test_kernel.py:13", "M_N_K": [[137, 909, 256], [32, 1024, 2048], [37, 32000, 5120]]},
    }


def small_layer():
    rng = np.random.default_rng(20240229)
    K, N, n = 64, 24, 160
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    mix = (np.eye(K) + 0.3 * rng.standard_normal((K, K)) / np.sqrt(K)).astype(np.float32)
    xs = [(rng.standard_normal((n // 2, K)).astype(np.float32) @ mix) for _ in range(2)]
    params = O.get_col_quantize_params(W)
    H = O.accumulate_H(xs)
    Q, p = O.gptq(W, xs, block_size=16)
    codes = O.codes_from_q(Q, p)
    packed = O.pack_matrix(Q, p)
    return dict(W=W, x0=xs[0], x1=xs[1], scale=np.asarray(params["scale"]), zero=np.asarray(params["zero"]),
                H=np.asarray(H), Q=np.asarray(Q), codes=codes.astype(np.uint8),
                packed=np.ascontiguousarray(packed.int_weight), block_size=np.int64(16))


if __name__ == "__main__":
    with open(os.path.join(HERE, "reference_test_vectors.json"), "w") as f:
        json.dump(reference_vectors(), f, indent=1)
    np.savez_compressed(os.path.join(HERE, "oracle_small_layer.npz"), **small_layer())
    print("written")
