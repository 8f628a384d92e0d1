"""Size-independent properties of the solve at the full benchmark shapes.

The CPU evaluation needs minutes at these sizes, so the checks here are ones that hold
for any correct implementation: H symmetric; L lower triangular with a positive diagonal
and L L^T the inverse of the damped H (applied to random vectors); every quantised weight
on its column's grid; pack -> unpack returns the quantised weights bit for bit; the layer
reconstruction error below round-to-nearest's on the same grid; and the packed matmul
agreeing with a dense product of the dequantised weights.
"""
import pytest

pytestmark = pytest.mark.gpu

SHAPES = [
    (4096, 11008, 4),    # LLaMA-7B gate/up projection, the benchmark layer
    (11008, 4096, 4),    # LLaMA-7B down projection
    (7168, 28672, 2),    # OPT-30B fc1
    (28672, 7168, 16),   # OPT-30B fc2: H is 28672^2 fp32 (rows >= K keeps H well conditioned)
]


@pytest.mark.parametrize("K,N,nb", SHAPES)
def test_layer_properties(K, N, nb):
    import torch
    import jax_gptq_amd.gptq as G
    from jax_gptq_amd.op import quantized_matmul

    g = torch.Generator(device="cuda")
    g.manual_seed(K + N)
    W = (0.02 * torch.randn((K, N), generator=g, device="cuda")).to(torch.float16)
    xs = [torch.randn((2048, K), generator=g, device="cuda") for _ in range(nb)]

    W32 = W.float()
    params = G.get_col_quantize_params(W32)
    H = G.accumulate_H(xs)
    assert bool((H == H.T).all())
    Hd = H.clone()
    Hd.diagonal().add_(0.01 * float(H.diagonal().mean()))
    W32, L, bad = G._damp_and_invert(W32, H, 0.01)
    assert not bad
    assert bool((torch.triu(L, 1) == 0).all())
    assert bool((L.diagonal() > 0).all())
    v = torch.randn((K, 4), generator=g, device="cuda")
    r = L @ (L.T @ (Hd @ v)) - v
    assert float(r.norm() / v.norm()) < 2e-4      # fp32 factorisation, cond(H) is small here
    del Hd, H

    Q, _ = G._solve(W32.clone(), L, params, 128, torch.float16)
    del L
    sc, z = params["scale"], params["zero"]
    codes = Q.float() / sc + z
    assert float((codes - codes.round()).abs().max()) < 2e-2   # fp16 rounding of scale*(c-z)
    assert float(codes.round().min()) >= 0 and float(codes.round().max()) <= 15

    packed = G.pack_matrix(Q, params)
    assert packed.int_weight.shape == (K // 2, N) and packed.int_weight.dtype == torch.uint8
    assert bool((G.unpack_matrix(packed).to(torch.float16) == Q).all())

    X = xs[0]
    Wf = W.float()
    rtn = sc * (torch.clamp(torch.round(Wf / sc) + z, 0, 15) - z)
    ref = (X @ Wf).norm()
    e_gptq = float((X @ (Wf - Q.float())).norm() / ref)
    e_rtn = float((X @ (Wf - rtn)).norm() / ref)
    assert e_gptq < 0.98 * e_rtn, (e_gptq, e_rtn)

    x16 = X[:40].to(torch.float16)
    y = quantized_matmul(x16, packed).float()
    y_ref = x16.float() @ Q.float()
    assert torch.allclose(y, y_ref, atol=1e-2 * float(y_ref.abs().max()), rtol=1e-3)
