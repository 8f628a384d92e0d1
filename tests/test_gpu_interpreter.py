"""GPU tests of the callers of the hot path: ``quantize`` (sequential calibration driver) and
``use_quantized`` (inference dispatch).  They restate the reference's behavioural tests
(``tests.py:46-138, 158-291``) for ``torch`` model functions, and add what pins the driver:
its result must equal the layer-by-layer chain of ``gptq`` calls written out by hand."""
import numpy as np
import pytest

from helpers import to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    import torch
    return torch


@pytest.fixture(scope="module")
def J():
    import jax_gptq_amd
    return jax_gptq_amd


def _randn(T, seed, *shape, dtype=None):
    g = T.Generator(device="cuda")
    g.manual_seed(seed)
    return T.randn(shape, generator=g, device="cuda", dtype=dtype or T.float32)


def test_single(T, J):
    """reference test_single (tests.py:46-73) + equality with the direct solve."""
    G = J.gptq
    w = _randn(T, 0, 256, 64)
    orig_w = w.clone()
    xs = [_randn(T, 1 + i, 32, 256) for i in range(4)]
    f = lambda w, x: x @ w
    orig_output = f(orig_w, xs[0])
    quantized = J.quantize(f, w, xs, block_size=16)
    assert isinstance(quantized, J.QuantizedMatrix)
    assert tuple(quantized.int_weight.shape) == (128, 64) and quantized.contraction_axis == 0
    de_quantized = G.unpack_matrix(quantized)
    Q, p = G.gptq(orig_w.clone(), xs, block_size=16)
    assert T.equal(de_quantized, Q)                                   # the driver adds nothing
    assert T.equal(quantized.int_weight, G.pack_matrix(Q, p).int_weight)
    new_output = f(de_quantized, xs[0])
    assert float((orig_output - new_output).abs().mean() / orig_output.abs().mean()) < 0.15
    assert T.equal(w, Q)          # the parameter buffer now holds the quantised values


@pytest.mark.parametrize("use_quantized_activations", [True, False])
def test_three_linear_layers_are_solved_sequentially(T, J, use_quantized_activations):
    """reference test_hk (tests.py:75-116): three bias-free fp16 linear layers 256 -> 1024 ->
    1024 -> 1024, 64 batches of 32."""
    G = J.gptq
    dims = [256, 1024, 1024, 1024]
    params = {f"linear_{i}": {"w": (_randn(T, 10 + i, dims[i], dims[i + 1]) / np.sqrt(dims[i])).half()}
              for i in range(3)}
    originals = {k: v["w"].clone() for k, v in params.items()}
    xs = [_randn(T, 100 + i, 32, 256).half() for i in range(64)]

    def f(p, x):
        for i in range(3):
            x = x @ p[f"linear_{i}"]["w"]
        return x

    quantized_params = J.quantize(f, params, xs, use_quantized_activations=use_quantized_activations)
    # the same chain by hand: layer i is calibrated on what the layers before it produce
    acts = list(xs)
    for i in range(3):
        W = originals[f"linear_{i}"]
        Q, p = G.gptq(W.clone(), acts)
        got = quantized_params[f"linear_{i}"]["w"]
        assert isinstance(got, J.QuantizedMatrix)
        assert T.equal(got.int_weight, G.pack_matrix(Q, p).int_weight), f"layer {i}"
        acts = [a @ (Q if use_quantized_activations else W) for a in acts]

    manual_result = xs[0]
    for i in range(3):
        manual_result = manual_result @ G.unpack_matrix(quantized_params[f"linear_{i}"]["w"]).half()
    new_output = J.use_quantized(f)(quantized_params, xs[0])
    assert T.allclose(manual_result.float(), new_output.float(), atol=3e-3, rtol=0)
    kernel_output = J.use_quantized(f, use_kernel=True)(quantized_params, xs[0])
    assert T.allclose(manual_result.float(), kernel_output.float(), atol=3e-2, rtol=1e-2)


def test_products_on_the_same_activations_share_one_hessian(T, J, monkeypatch):
    """q / k / v style: three matrices applied to the same activations are solved with one
    Hessian accumulation and one factorisation; a product on other activations of the same shape
    gets its own.  The results are those of independent ``gptq`` calls, including the zeroed
    rows of a feature that is dead in the first set of activations only."""
    G = J.gptq
    import jax_gptq_amd.quantize_interpreter as QI
    calls = []
    real = QI.accumulate_H
    monkeypatch.setattr(QI, "accumulate_H", lambda xs, **kw: (calls.append(len(xs)), real(xs, **kw))[1])
    factorisations = []
    real_di = G._damp_invert
    monkeypatch.setattr(G, "_damp_invert", lambda *a, **k: (factorisations.append(1), real_di(*a, **k))[1])
    params = {n: _randn(T, 20 + i, 256, 384) / 16 for i, n in enumerate(("q", "k", "v", "o"))}
    originals = {k: v.clone() for k, v in params.items()}
    xs = [_randn(T, 200 + i, 48, 256) for i in range(6)]
    for x in xs:
        x[:, 7] = 0                              # dead for q / k / v; 1.0 in the activations of o

    def f(p, x):
        h = x * 1.5
        a = (h @ p["q"]) + (h @ p["k"]) + (h @ p["v"])
        h2 = x * 0.5 + 1.0                      # same shape, other values
        return a + h2 @ p["o"]

    out = J.quantize(f, params, xs, block_size=64)
    assert calls == [6, 6] and len(factorisations) == 2          # one each for q/k/v, one for o
    factorisations.clear()
    for n in ("q", "k", "v", "o"):
        acts = [x * 1.5 for x in xs] if n != "o" else [x * 0.5 + 1.0 for x in xs]
        Q, p = G.gptq(originals[n].clone(), acts, block_size=64)
        assert T.equal(out[n].int_weight, G.pack_matrix(Q, p).int_weight), n
        assert bool((Q[7] == 0).all()) == (n != "o")
    assert len(factorisations) == 4
    # gptq leaves a Hessian that it is given untouched
    H = G.accumulate_H(xs)
    H0 = H.clone()
    Q1, _ = G.gptq(originals["q"].clone(), xs, block_size=64, H=H)
    Q2, _ = G.gptq(originals["q"].clone(), xs, block_size=64)
    assert T.equal(H, H0) and T.equal(Q1, Q2)
    with pytest.raises(ValueError):
        G.gptq(originals["q"].clone(), xs, block_size=64, H=H[:, :-1])
    # a Hessian handed over as a strided view (the corner of a larger matrix), and one that starts
    # in the middle of an allocation, are the same matrix to gptq
    big = T.zeros((300, 300), dtype=H.dtype, device=H.device)
    big[:256, :256] = H
    Q3, _ = G.gptq(originals["q"].clone(), xs, block_size=64, H=big[:256, :256])
    flat = T.zeros(256 * 256 + 1, dtype=H.dtype, device=H.device)
    flat[1:] = H.reshape(-1)
    Q4, _ = G.gptq(originals["q"].clone(), xs, block_size=64, H=flat[1:].view(256, 256))
    assert T.equal(Q3, Q1) and T.equal(Q4, Q1)


def test_transform(T, J):
    """reference test_transform (tests.py:118-138), 1024 x 1024."""
    G = J.gptq
    w = _randn(T, 0, 1024, 1024)
    xs = [_randn(T, i, 32, 1024) for i in range(16)]
    f = lambda w, x: x @ w
    quantized_params = J.quantize(f, w, xs, block_size=16)
    unpacked_matrix = G.unpack_matrix(quantized_params)
    manual_result = xs[0] @ unpacked_matrix
    transform_result = J.use_quantized(f)(quantized_params, xs[0])
    assert T.allclose(manual_result, transform_result, atol=1e-4, rtol=0)


@pytest.fixture(scope="module")
def simple_model(T, J):
    w = _randn(T, 0, 256, 64)
    xs = [_randn(T, 1 + i, 32, 256) for i in range(4)]
    f = lambda w, x: x @ w
    w_q = J.quantize(f, w.clone(), xs, block_size=4)
    return f, w, w_q, xs


def test_remat(T, J, simple_model):
    """reference test_remat (tests.py:158-168)."""
    f, _, w_q, xs = simple_model
    x = xs[0].half()
    expected = x.float() @ J.gptq.unpack_matrix(w_q)
    result = J.use_quantized(f, use_kernel=True, remat_unpack=True)(w_q, x)
    assert T.allclose(result.float(), expected, atol=0.03, rtol=0)


@pytest.mark.parametrize("use_kernel,remat_unpack", [(True, False), (False, True), (False, False)])
def test_grad(T, J, simple_model, use_kernel, remat_unpack):
    """reference test_grad (tests.py:170-186): gradient with respect to x through the packed matrix."""
    _, _, w_q, xs = simple_model
    f = lambda x, w: (x @ w)[3].sum()
    unpacked = J.gptq.unpack_matrix(w_q)
    x = xs[0].clone().requires_grad_(True)
    J.use_quantized(f, use_kernel=use_kernel, remat_unpack=remat_unpack)(x, w_q).backward()
    x2 = xs[0].clone().requires_grad_(True)
    f(x2, unpacked).backward()
    assert T.allclose(x.grad, x2.grad, atol=1e-1, rtol=0)
    assert float(x.grad[3].abs().sum()) > 0 and float(x.grad[0].abs().sum()) == 0


@pytest.mark.parametrize("w_contract", range(3))
@pytest.mark.parametrize("x_contract", range(2))
def test_weird_dots(T, J, w_contract, x_contract):
    """reference test_weird_dots (tests.py:188-217): a 3-D weight contracted along any axis."""
    w_shape, x_shape = [47, 768], [32]
    w_shape.insert(w_contract, 256)
    x_shape.insert(x_contract, 256)
    w = _randn(T, 9999, *w_shape)
    xs = [_randn(T, 10 * i, *x_shape) for i in range(10)]
    f = lambda w, x: T.tensordot(w, x, dims=([w_contract], [x_contract]))
    expected_output = f(w.clone(), xs[0])
    quantized_params = J.quantize(f, w, xs, block_size=16)
    assert isinstance(quantized_params, J.QuantizedMatrix)
    assert quantized_params.contraction_axis == w_contract and tuple(quantized_params.shape) == tuple(w_shape)
    quantized_output = J.use_quantized(f)(quantized_params, xs[0])
    mean_error = (expected_output - quantized_output).abs().mean()
    assert float(mean_error / expected_output.abs().mean()) < 0.1


def test_conv(T, J):
    """reference test_conv (tests.py:219-254): a 1x1 convolution is the same product."""
    import torch.nn.functional as F
    w = _randn(T, 0, 79, 32)
    xs = [_randn(T, i, 11, 32, 13) for i in range(1, 20)]
    matmul_f = lambda w, x: T.tensordot(w, x, dims=([1], [1]))
    conv_f = lambda w, x: F.conv1d(x, w)
    quantized_params = J.quantize(matmul_f, w.clone(), xs, block_size=16)
    quantized_output = J.use_quantized(matmul_f)(quantized_params, xs[0])
    conv_quantized = J.quantize(conv_f, w.clone()[:, :, None], xs, block_size=16)
    unpacked_w = J.gptq.unpack_matrix(quantized_params)
    unpacked_kernel = J.gptq.unpack_matrix(conv_quantized)
    assert int((unpacked_w != unpacked_kernel[:, :, 0]).sum()) < 10
    quantized_conv_output = J.use_quantized(conv_f)(conv_quantized, xs[0]).permute(1, 0, 2)
    assert float((quantized_output - quantized_conv_output).abs().max()) < 1e-4


def test_transpose(T, J):
    """reference test_transpose (tests.py:256-278): the parameter is transposed before use."""
    w = _randn(T, 9999, 256, 1024)
    w_copy = w.clone()
    xs = [_randn(T, i, 256, 32) for i in range(10)]
    f = lambda w, x: w.T @ x
    quantized_params = J.quantize(f, w, xs, block_size=16)
    assert isinstance(quantized_params, J.QuantizedMatrix)
    assert tuple(quantized_params.shape) == (256, 1024) and quantized_params.contraction_axis == 0
    quantized_output = J.use_quantized(f)(quantized_params, xs[0])
    unpacked = J.gptq.unpack_matrix(quantized_params)
    manual_result = unpacked.T @ xs[0]
    assert float((unpacked - w_copy).abs().mean()) < 0.15
    assert T.allclose(manual_result, quantized_output, atol=1e-4)
    # same codes as solving the [K, N] matrix directly
    Q, p = J.gptq.gptq(w_copy.clone(), [x.T for x in xs], block_size=16)
    assert T.equal(unpacked, Q)


def test_reuse(T, J, simple_model):
    """reference test_reuse (tests.py:280-291): other uses of a parameter do not confuse the driver."""
    _, w, _, xs = simple_model

    def f(w, x):
        intermediate = w.T       # noqa: F841  (unused on purpose)
        answer = w.T @ x.T
        answer = answer + w.sum()
        return answer

    quantized_params = J.quantize(f, w.clone(), xs, block_size=16)
    assert isinstance(quantized_params, J.QuantizedMatrix)
    quantized_output = J.use_quantized(f)(quantized_params, xs[0])
    dense = J.gptq.unpack_matrix(quantized_params)
    assert T.allclose(quantized_output, dense.T @ xs[0].T + dense.sum(), atol=1e-3)


def test_parameter_used_by_two_products_is_quantized_once(T, J):
    w = _randn(T, 3, 128, 128)
    xs = [_randn(T, i, 16, 128) for i in range(4)]
    f = lambda w, x: (x @ w) @ w
    q = J.quantize(f, w.clone(), xs, block_size=16)
    Q, p = J.gptq.gptq(w.clone(), xs, block_size=16)
    assert T.equal(J.gptq.unpack_matrix(q), Q)


def test_other_leaves_pass_through_and_errors(T, J):
    params = {"w": _randn(T, 0, 64, 32), "b": _randn(T, 1, 32), "n": 3, "unused": _randn(T, 2, 8, 8)}
    xs = [_randn(T, i, 8, 64) for i in range(3)]
    f = lambda p, x: (x @ p["w"] + p["b"]) * p["n"]
    out = J.quantize(f, params, xs, block_size=16)
    assert isinstance(out["w"], J.QuantizedMatrix)
    assert out["b"] is params["b"] and out["n"] == 3 and out["unused"] is params["unused"]
    with pytest.raises(NotImplementedError):
        J.quantize(lambda p, x: p["w"].T @ p["w"], {"w": _randn(T, 0, 64, 32)}, xs, block_size=16)
    with pytest.raises(ValueError):
        J.quantize(f, {"w": _randn(T, 0, 64, 32), "b": params["b"], "n": 1}, xs, block_size=48)
    with pytest.raises(ZeroDivisionError):
        J.quantize(lambda p, x: x @ p["w"] / 0 if False else 1 // 0, params, xs)


def _gpt2_params(T, d, n_layer, vocab, n_ctx, seed=0):
    g = T.Generator(device="cuda")
    g.manual_seed(seed)
    n = lambda *s: 0.02 * T.randn(s, generator=g, device="cuda")
    p = {"wte": n(vocab, d), "wpe": n(n_ctx, d), "ln_f": {"g": T.ones(d, device="cuda"), "b": T.zeros(d, device="cuda")},
         "h": []}
    for _ in range(n_layer):
        p["h"].append({
            "ln_1": {"g": T.ones(d, device="cuda"), "b": T.zeros(d, device="cuda")},
            "ln_2": {"g": T.ones(d, device="cuda"), "b": T.zeros(d, device="cuda")},
            "attn": {"c_attn": {"w": n(d, 3 * d), "b": T.zeros(3 * d, device="cuda")},
                     "c_proj": {"w": n(d, d), "b": T.zeros(d, device="cuda")}},
            "mlp": {"c_fc": {"w": n(d, 4 * d), "b": T.zeros(4 * d, device="cuda")},
                    "c_proj": {"w": n(4 * d, d), "b": T.zeros(d, device="cuda")}}})
    return p


def _gpt2(n_head):
    import torch
    import torch.nn.functional as F

    def forward(p, tokens):
        B, S = tokens.shape
        d = p["wte"].shape[1]
        x = F.embedding(tokens, p["wte"]) + p["wpe"][:S]
        mask = torch.ones(S, S, dtype=torch.bool, device=tokens.device).tril()
        for blk in p["h"]:
            h = F.layer_norm(x, (d,), blk["ln_1"]["g"], blk["ln_1"]["b"])
            qkv = h @ blk["attn"]["c_attn"]["w"] + blk["attn"]["c_attn"]["b"]
            q, k, v = (t.reshape(B, S, n_head, d // n_head).transpose(1, 2) for t in qkv.split(d, dim=-1))
            att = (q @ k.transpose(-1, -2)) / (d // n_head) ** 0.5
            att = att.masked_fill(~mask, float("-inf")).softmax(-1)
            a = (att @ v).transpose(1, 2).reshape(B, S, d)
            x = x + a @ blk["attn"]["c_proj"]["w"] + blk["attn"]["c_proj"]["b"]
            h = F.layer_norm(x, (d,), blk["ln_2"]["g"], blk["ln_2"]["b"])
            h = F.gelu(h @ blk["mlp"]["c_fc"]["w"] + blk["mlp"]["c_fc"]["b"])
            x = x + h @ blk["mlp"]["c_proj"]["w"] + blk["mlp"]["c_proj"]["b"]
        x = F.layer_norm(x, (d,), p["ln_f"]["g"], p["ln_f"]["b"])
        return x @ p["wte"].T          # tied output head
    return forward


def test_gpt2_shaped_model_through_the_driver(T, J):
    """A GPT-2-shaped decoder (random init N(0, 0.02), uniform random tokens) through
    ``quantize`` and back through ``use_quantized``: every Linear weight and the tied
    embedding / output matrix are packed, nothing else is touched, and the packed model
    reproduces the dense one."""
    d, n_layer, vocab, n_ctx, n_head = 128, 2, 512, 64, 4
    params = _gpt2_params(T, d, n_layer, vocab, n_ctx)
    import copy
    dense = copy.deepcopy(params)
    g = T.Generator(device="cuda")
    g.manual_seed(5)
    batches = [T.randint(0, vocab, (4, n_ctx), generator=g, device="cuda") for _ in range(8)]
    f = _gpt2(n_head)
    ref = f(dense, batches[0])
    q = J.quantize(f, params, batches, block_size=64)
    for blk in q["h"]:
        for name, sub in (("attn", "c_attn"), ("attn", "c_proj"), ("mlp", "c_fc"), ("mlp", "c_proj")):
            assert isinstance(blk[name][sub]["w"], J.QuantizedMatrix)
            assert isinstance(blk[name][sub]["b"], T.Tensor)
        assert isinstance(blk["ln_1"]["g"], T.Tensor)
    assert isinstance(q["wte"], J.QuantizedMatrix)
    assert tuple(q["wte"].shape) == (vocab, d) and q["wte"].contraction_axis == 1   # used as wte.T
    assert isinstance(q["wpe"], T.Tensor)
    out = J.use_quantized(f)(q, batches[0])
    out_k = J.use_quantized(f, use_kernel=True)(q, batches[0])
    rel = float((out - ref).norm() / ref.norm())
    assert rel < 0.25, rel
    assert float((out_k - out).norm() / out.norm()) < 2e-2


def test_quantize_with_split_fp16_hessians(T, J):
    """``quantize(..., split_fp16=True)``: fp32 activations of a GPT-2-shaped model (d = 256, so
    every Linear input has a multiple of 256 features) go through the fp16-pair Hessian.  The
    first product sees identical inputs: its codes agree up to a handful of ties.  Every flipped
    tie changes the activations that later products are calibrated on, and the error feedback of
    the column loop turns such a change into many different (equally good) codes, so for the
    model as a whole the check is the distance to the dense model."""
    import copy
    d, n_layer, vocab, n_ctx, n_head = 256, 1, 512, 64, 4
    params = _gpt2_params(T, d, n_layer, vocab, n_ctx)
    dense = copy.deepcopy(params)
    params2 = copy.deepcopy(params)
    g = T.Generator(device="cuda")
    g.manual_seed(6)
    batches = [T.randint(0, vocab, (4, n_ctx), generator=g, device="cuda") for _ in range(8)]
    f = _gpt2(n_head)
    ref = f(dense, batches[0])
    q1 = J.quantize(f, params, batches, block_size=64)
    q2 = J.quantize(f, params2, batches, block_size=64, split_fp16=True)
    a, b = q1["h"][0]["attn"]["c_attn"]["w"].int_weight, q2["h"][0]["attn"]["c_attn"]["w"].int_weight
    same = ((a & 15) == (b & 15)).float().mean() + ((a >> 4) == (b >> 4)).float().mean()
    assert float(same) / 2 >= 0.999, float(same) / 2
    e1 = float((J.use_quantized(f)(q1, batches[0]) - ref).norm() / ref.norm())
    e2 = float((J.use_quantized(f)(q2, batches[0]) - ref).norm() / ref.norm())
    assert e2 < 1.1 * e1 + 1e-3, (e1, e2)


def test_gpt2_small_full_shape(T, J):
    """GPT-2-small-shaped model at full size (12 layers, d = 768, 12 heads, MLP 3072, vocab
    50257), 128 sequences x 512 uniform random tokens in 16 batches: all 48 Linear weights and
    the tied embedding matrix are packed; the packed model tracks the dense one and the kernel
    path tracks the unpack path."""
    import copy
    d, n_layer, vocab, n_ctx, n_head = 768, 12, 50257, 512, 12
    params = _gpt2_params(T, d, n_layer, vocab, n_ctx)
    dense = copy.deepcopy(params)
    g = T.Generator(device="cuda")
    g.manual_seed(5)
    batches = [T.randint(0, vocab, (8, n_ctx), generator=g, device="cuda") for _ in range(16)]
    f = _gpt2(n_head)
    with T.no_grad():
        ref = f(dense, batches[0])
        q = J.quantize(f, params, batches)
        packed = [blk[m][s]["w"] for blk in q["h"] for m, s in
                  (("attn", "c_attn"), ("attn", "c_proj"), ("mlp", "c_fc"), ("mlp", "c_proj"))]
        assert len(packed) == 48 and all(isinstance(w, J.QuantizedMatrix) for w in packed)
        assert isinstance(q["wte"], J.QuantizedMatrix) and tuple(q["wte"].int_weight.shape) == (vocab, d // 2)
        out = J.use_quantized(f)(q, batches[0])
        assert float((out - ref).norm() / ref.norm()) < 0.3
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")      # the embedding lookup is not a product: it unpacks
            out_k = J.use_quantized(f, use_kernel=True)(q, batches[0])
        assert float((out_k - out).norm() / out.norm()) < 5e-3


def _llama_block_params(T, d, d_ff, seed=0, dtype=None):
    g = T.Generator(device="cuda")
    g.manual_seed(seed)
    dtype = dtype or T.float16
    n = lambda *s: (0.02 * T.randn(s, generator=g, device="cuda")).to(dtype)
    return {"ln_1": T.ones(d, device="cuda", dtype=dtype), "ln_2": T.ones(d, device="cuda", dtype=dtype),
            "q": n(d, d), "k": n(d, d), "v": n(d, d), "o": n(d, d),
            "gate": n(d, d_ff), "up": n(d, d_ff), "down": n(d_ff, d)}


def _llama_block(n_head):
    import torch
    import torch.nn.functional as F

    def rms(x, w):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).to(x.dtype) * w

    def forward(p, x):                       # x: [B, S, d] hidden states
        B, S, d = x.shape
        h = rms(x, p["ln_1"])
        q, k, v = ((h @ p[n]).reshape(B, S, n_head, d // n_head).transpose(1, 2) for n in ("q", "k", "v"))
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B, S, d)
        x = x + a @ p["o"]
        h = rms(x, p["ln_2"])
        return x + (F.silu(h @ p["gate"]) * (h @ p["up"])) @ p["down"]
    return forward


def test_llama7b_shaped_decoder_block(T, J):
    """One Llama-7B-shaped decoder block (q/k/v/o 4096 x 4096, gate/up 4096 x 11008, down
    11008 x 4096, fp16 weights N(0, 0.02)) on fp16 hidden states N(0, 1), 16 sequences of 2048
    tokens: all seven matrices are solved in calling order on the activations of the already
    quantised part, packed, and the packed block tracks the dense one."""
    import copy
    d, d_ff, n_head, S = 4096, 11008, 32, 2048
    params = _llama_block_params(T, d, d_ff)
    dense = copy.deepcopy(params)
    g = T.Generator(device="cuda")
    g.manual_seed(9)
    batches = [T.randn((2, S, d), generator=g, device="cuda").half() for _ in range(8)]
    f = _llama_block(n_head)
    with T.no_grad():
        ref = f(dense, batches[0])
        q = J.quantize(f, params, batches)
        for name, shape in (("q", (d, d)), ("k", (d, d)), ("v", (d, d)), ("o", (d, d)),
                            ("gate", (d, d_ff)), ("up", (d, d_ff)), ("down", (d_ff, d))):
            assert isinstance(q[name], J.QuantizedMatrix), name
            assert tuple(q[name].shape) == shape and tuple(q[name].int_weight.shape) == (shape[0] // 2, shape[1])
        assert isinstance(q["ln_1"], T.Tensor)
        out = J.use_quantized(f)(q, batches[0])
        out_k = J.use_quantized(f, use_kernel=True)(q, batches[0])
    # the block's own contribution (output minus the residual input) is what quantisation perturbs
    dref = (ref - batches[0]).float()
    # (4-bit codes of Gaussian weights: ~0.28 relative, measured; round-to-nearest gives the same order)
    assert float(((out - batches[0]).float() - dref).norm() / dref.norm()) < 0.35
    assert float((out_k.float() - out.float()).norm() / out.float().norm()) < 5e-3


def test_three_layer_chain_against_the_oracle_chain(T, J):
    """`quantize` over three fp32 linear layers against the same chain run by the CPU oracle:
    layer 0 sees identical inputs on both sides, so its codes must match to the solve's bar
    (>= 99.9 % equal, the rest off by one); later layers are calibrated on what the (nearly
    identical) quantised layers before them produce, so they are compared through their layer
    reconstruction error, within 1 % of the oracle's."""
    from helpers import code_stats, recon_error
    from oracle import gptq_oracle as O
    G = J.gptq
    dims = [256, 512, 384, 320]
    rng = np.random.default_rng(42)
    Ws = [(rng.standard_normal((dims[i], dims[i + 1])) / np.sqrt(dims[i])).astype(np.float32) for i in range(3)]
    xs = [rng.standard_normal((64, 256)).astype(np.float32) for _ in range(16)]
    params = {f"l{i}": T.from_numpy(Ws[i].copy()).cuda() for i in range(3)}

    def f(p, x):
        for i in range(3):
            x = x @ p[f"l{i}"]
        return x

    qp = J.quantize(f, params, [T.from_numpy(x).cuda() for x in xs])
    acts = list(xs)                      # the oracle's chain, fed by its own quantised layers
    for i in range(3):
        Qr, pr = O.gptq(Ws[i], acts)
        got = qp[f"l{i}"]
        Qg = to_np(G.unpack_matrix(got))
        assert np.allclose(to_np(got.scale), pr["scale"], rtol=1e-5) and np.allclose(to_np(got.zero), pr["zero"], rtol=1e-5)
        X = np.concatenate(acts)
        e, er = recon_error(Ws[i], Qg, X), recon_error(Ws[i], Qr, X)
        assert abs(e - er) <= 0.01 * er, (i, e, er)
        if i == 0:
            frac, mx = code_stats(to_np(G.unpack_colwise(got.int_weight)), O.codes_from_q(Qr, pr))
            assert frac <= 1e-3 and mx <= 1, (frac, mx)
        acts = [a @ Qr for a in acts]


def test_shape_helpers_of_utils(T, J):
    """reference utils.py:6-21: a QuantizedMatrix maps to an abstract array of its logical shape and
    of zero's dtype, anything else maps to itself, containers keep their structure."""
    from jax_gptq_amd import utils as U
    G = J.gptq
    qm = G.QuantizedMatrix(T.zeros((64, 48), dtype=T.uint8, device="cuda"), T.zeros(48, dtype=T.float16, device="cuda"),
                           T.ones(48, dtype=T.float16, device="cuda"), contraction_axis=0)
    a = U._shape_from_param(qm)
    assert tuple(a.shape) == (128, 48) and a.dtype == T.float16 and a.device.type == "meta"
    qm1 = G.QuantizedMatrix(T.zeros((5, 30, 7), dtype=T.uint8, device="cuda"), T.zeros((5, 7), device="cuda"),
                            T.ones((5, 7), device="cuda"), contraction_axis=1)
    assert tuple(U._shape_from_param(qm1).shape) == (5, 60, 7) and U._shape_from_param(qm1).dtype == T.float32
    assert tuple(G.quant_matrix_shape(qm1)) == (5, 60, 7) and tuple(qm1.shape) == (5, 60, 7)
    plain = T.ones(3, device="cuda")
    assert U._shape_from_param(plain) is plain
    tree = {"a": qm, "b": [plain, (qm1, 4)], "c": None}
    out = U.quantized_params_to_shaped_arrays(tree)
    assert set(out) == {"a", "b", "c"} and out["c"] is None
    assert tuple(out["a"].shape) == (128, 48)
    assert isinstance(out["b"], list) and out["b"][0] is plain
    assert isinstance(out["b"][1], tuple) and tuple(out["b"][1][0].shape) == (5, 60, 7) and out["b"][1][1] == 4
    assert tuple(U.quantized_params_to_shaped_arrays(qm).shape) == (128, 48)
