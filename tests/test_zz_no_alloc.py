"""The packed-int4 matmul entry point that allocates nothing (``gptq_hip_qmatmul_static``).

It must give what ``gptq_hip_qmatmul`` gives (same kernels on a workspace inside the library, so
bit for bit), on calls in a row that share the one array: a larger problem first, then a smaller
one, then the larger again.  The fp64 dense product of the same operands bounds the result as in
the other matmul tests (atol 1e-2, rtol 1e-3; 2^-8 for a bf16 result).  Problems beyond the fixed array are refused.
"""
import numpy as np
import pytest

from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 1e-3


def _problem(seed, M, K, N, x_dtype, transpose):
    import torch
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    scale = rng.uniform(0.001, 0.01, N).astype(np.float16)
    zero = rng.integers(0, 16, N).astype(np.float16)
    packed = np.ascontiguousarray(O.pack_colwise(codes), dtype=np.uint8)
    x = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0)).astype(np.float32)
    dense = (codes.astype(np.float64) - zero.astype(np.float64)[None]) * scale.astype(np.float64)[None]
    dev = torch.device("cuda:0")
    xt = torch.from_numpy(x).to(dev).to(x_dtype)
    ref = xt.double().cpu().numpy() @ (dense.T if transpose else dense)
    return dict(M=M, R=K // 2, C=N, transpose=int(transpose), x=xt,
                packed=torch.from_numpy(packed).to(dev), zero=torch.from_numpy(zero).to(dev),
                scale=torch.from_numpy(scale).to(dev), ref=ref,
                out_cols=K if transpose else N)


def _run(lib, N, p, static):
    import torch
    from jax_gptq_amd.gptq import _DT, _ptr, _stream
    out = torch.full((p["M"], p["out_cols"]), float("nan"), dtype=p["x"].dtype, device=p["x"].device)
    args = (_stream(), _ptr(p["x"]), _DT[p["x"].dtype], p["M"], _ptr(p["packed"]), p["R"], p["C"],
            _ptr(p["zero"]), _ptr(p["scale"]), _DT[p["zero"].dtype], p["transpose"], _ptr(out))
    if static:
        rc = lib.gptq_hip_qmatmul_static(*args)
    else:
        nbytes = lib.gptq_hip_qmatmul_workspace_bytes_x(p["M"], p["R"], p["C"], p["transpose"], _DT[p["x"].dtype])
        ws = torch.zeros(max(int(nbytes), 256), dtype=torch.uint8, device=out.device)
        rc = lib.gptq_hip_qmatmul(*args, _ptr(ws), ws.numel())
    assert rc == 0, lib.gptq_hip_error_string(rc)
    torch.cuda.synchronize()
    return out


def _check_oracle(out, p):
    import torch
    got = out.double().cpu().numpy()
    err = np.abs(got - p["ref"])
    # a bf16 result is rounded to bf16 (2^-9 relative), the bar the other bf16 matmul tests use
    rtol = 2.0 ** -8 if out.dtype == torch.bfloat16 else RTOL
    assert np.all(err <= ATOL + rtol * np.abs(p["ref"])), f"max err {err.max():.3e}"


# (M, K, N, dtype name, transposed): split-K decode shapes, the tiled kernel with split-K, fp32
# activations through the fp16 staging buffers, the transposed product, a shape on the plain kernels
SEQUENCES = [
    [(16, 4096, 11008, "float16", False), (1, 4096, 4096, "float16", False)],
    [(128, 11008, 4096, "float16", False), (3, 1024, 2048, "bfloat16", False)],
    [(16, 7168, 28672, "float16", False), (1, 4096, 11008, "float16", False)],
    [(64, 4096, 4096, "float32", False), (5, 512, 768, "float32", False)],
    [(48, 2048, 4096, "float16", True), (7, 512, 256, "float16", True)],
    [(37, 256, 909, "float16", False), (2, 64, 30, "float16", False)],
]


@pytest.mark.parametrize("seq", SEQUENCES)
def test_static_entry_matches_workspace_entry(seq):
    import torch
    from jax_gptq_amd import _native as N
    lib = N.load()
    probs = [_problem(11 + i, M, K, Nc, getattr(torch, dt), tr) for i, (M, K, Nc, dt, tr) in enumerate(seq)]
    expect = [_run(lib, N, p, static=False) for p in probs]
    # larger, smaller, larger again: every call finds what the one before it left in the array
    for i in (0, 1, 0, 1):
        got = _run(lib, N, probs[i], static=True)
        assert torch.equal(got, expect[i]), f"call {i} of {seq} differs from gptq_hip_qmatmul"
        _check_oracle(got, probs[i])


def test_static_entry_refuses_what_does_not_fit():
    import torch
    from jax_gptq_amd import _native as N
    from jax_gptq_amd.gptq import _DT
    lib = N.load()
    M, K, Nc = 2048, 4096, 11008
    assert lib.gptq_hip_qmatmul_workspace_bytes_x(M, K // 2, Nc, 0, _DT[torch.float16]) > N.QMATMUL_STATIC_BYTES
    p = _problem(3, 4, 64, 32, torch.float16, False)
    p.update(M=M, R=K // 2, C=Nc)       # sizes only: the call must return before it touches a pointer
    from jax_gptq_amd.gptq import _ptr, _stream
    rc = lib.gptq_hip_qmatmul_static(_stream(), _ptr(p["x"]), _DT[torch.float16], M, _ptr(p["packed"]), K // 2, Nc,
                                     _ptr(p["zero"]), _ptr(p["scale"]), _DT[torch.float16], 0, _ptr(p["x"]))
    assert rc == N.ETOOBIG
    assert b"scratch" in lib.gptq_hip_error_string(rc)
    torch.cuda.synchronize()
    # and the entry point still works afterwards
    q = _problem(4, 2, 256, 128, torch.float16, False)
    assert torch.equal(_run(lib, N, q, static=True), _run(lib, N, q, static=False))


@pytest.mark.parametrize("M,K,Nc,dt", [(1, 4096, 11008, "float16"), (16, 4096, 11008, "float16"),
                                        (64, 4096, 4096, "float16"), (4, 4096, 4096, "float32")])
def test_static_entry_in_a_captured_graph(M, K, Nc, dt):
    """What the entry point is for: after one eager call of the same shape (the warm-up the header asks for) the call
    is captured into a HIP graph; every replay, with eager work and new input contents in between, gives bit for bit
    what gptq_hip_qmatmul gives for the input contents of that moment."""
    import torch
    from jax_gptq_amd import _native as N
    from jax_gptq_amd.gptq import _DT, _ptr
    import ctypes
    lib = N.load()
    p = _problem(21, M, K, Nc, getattr(torch, dt), False)
    _run(lib, N, p, static=True)                          # warm-up, eager
    out = torch.full((M, Nc), float("nan"), dtype=p["x"].dtype, device=p["x"].device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.gptq_hip_qmatmul_static(st, _ptr(p["x"]), _DT[p["x"].dtype], M, _ptr(p["packed"]), p["R"], p["C"],
                                         _ptr(p["zero"]), _ptr(p["scale"]), _DT[p["zero"].dtype], 0, _ptr(out))
    assert rc == 0
    g = torch.Generator(device="cuda").manual_seed(5)
    for rep in range(3):
        graph.replay()
        torch.cuda.synchronize()
        expect = _run(lib, N, p, static=False)
        assert torch.equal(out, expect), rep
        # eager work on the same array and new input contents between the replays
        _run(lib, N, p, static=True)
        p["x"].copy_(torch.randn(p["x"].shape, device="cuda", generator=g).to(p["x"].dtype))
        torch.cuda.synchronize()
