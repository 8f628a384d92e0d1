"""8-bit codes (an extension: the reference packs and multiplies 4-bit codes only): packing, unpacking and
the packed matmul in both directions against the oracle, and 4-bit shapes that only the register-operand
kernels serve (rows that are not multiples of 16 channels, unaligned operands).

Tolerance of the products (task statement): atol 1e-2, rtol 1e-3 against the fp64 dense product."""
import numpy as np
import pytest

from helpers import to_np
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 1e-3


@pytest.fixture(scope="module")
def OP():
    import jax_gptq_amd.op as op
    return op


def _matrix8(seed, K, N, zs_dtype=np.float32, frac=False):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 256, (K, N)).astype(np.uint8)
    scale = rng.uniform(0.0001, 0.001, N).astype(zs_dtype)
    zero = (rng.uniform(0, 255, N) if frac else rng.integers(0, 256, N)).astype(zs_dtype)
    return O.QuantizedMatrix(codes, zero, scale, bits=8)


def _matrix4(seed, K, N, zs_dtype=np.float32):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    scale = rng.uniform(0.001, 0.01, N).astype(zs_dtype)
    zero = rng.integers(0, 16, N).astype(zs_dtype)
    return O.QuantizedMatrix(O.pack_colwise(codes), zero, scale)


def _dense(qm):
    codes = qm.int_weight if qm.bits == 8 else O.unpack_colwise(qm.int_weight)
    return (codes.astype(np.float64) - qm.zero.astype(np.float64)[None]) * qm.scale.astype(np.float64)[None]


def _check(got, x, qm, transpose, atol=ATOL, rtol=RTOL):
    dense = _dense(qm)
    ref = x.astype(np.float64) @ (dense.T if transpose else dense)
    got = to_np(got).astype(np.float64)
    assert got.shape == ref.shape
    err = np.abs(got - ref)
    tol = atol + rtol * np.abs(ref)
    bad = err > tol
    assert not bad.any(), (f"{bad.sum()} of {bad.size} off, max err {err.max():.3e} at |ref|="
                           f"{np.abs(ref).flat[err.argmax()]:.3e}, first bad index {np.argwhere(bad)[0]}")


SHAPES8 = [(1, 4096, 4096), (5, 1024, 2048), (16, 11008, 4096), (37, 5120, 1280), (128, 4096, 1024),
           (200, 2304, 768), (300, 909, 256), (3, 130, 66), (70, 8, 8), (1, 50257, 768), (2, 24, 1000),
           (17, 136, 40), (64, 128, 33)]


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("M,N,K", SHAPES8)
def test_qmatmul_8bit_fp16(OP, M, N, K, transpose):
    qm = _matrix8(M + N + K, K, N, np.float16)
    assert qm.shape == (K, N)
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0)).astype(np.float16)
    got = OP.quantized_matmul(x, qm, transpose_b=transpose)
    assert to_np(got).dtype == np.float16
    _check(got, x.astype(np.float32), qm, transpose)


@pytest.mark.parametrize("K,N", [(64, 256), (256, 512), (1024, 16), (4096, 1024), (2048, 8192), (8192, 2048),
                                 (520, 272)])
@pytest.mark.parametrize("M", [1, 2, 4, 5, 8, 9, 16])
def test_qmatmul_8bit_decode_kernel_instantiations(OP, M, K, N):
    """Up to 16 fp16 rows against aligned 8-bit matrices run on the decode kernel: one, four or sixteen rows of
    the tile kept, one to four k-steps per wavefront, 8 or 16 wavefronts, with and without a split over K
    (atomic sum or partial tiles).  Each case three times on the same workspace (the sum's cells must be left
    zero), with fractional zero points."""
    qm = _matrix8(11 * M + K + N, K, N, np.float16, frac=True)
    rng = np.random.default_rng(M + K)
    for rep in range(3):
        x = rng.standard_normal((M, K)).astype(np.float16)
        got = OP.quantized_matmul(x, qm, transpose_b=False)
        _check(got, x.astype(np.float32), qm, False)


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("zs", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("xdt", ["float16", "bfloat16", "float32"])
@pytest.mark.parametrize("M,N,K", [(1, 2048, 1024), (40, 1000, 520), (130, 1024, 512)])
def test_qmatmul_8bit_dtypes_and_fractional_zero_points(OP, M, N, K, xdt, zs, transpose):
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 256, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.0001, 0.001, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 255.0, N).astype(np.float32)).to(tdt)
    qm_ref = O.QuantizedMatrix(codes, zero.float().numpy(), scale.float().numpy(), bits=8)
    qm = G.QuantizedMatrix(torch.from_numpy(codes).cuda(), zero.cuda(), scale.cuda(), bits=8)
    x32 = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0)).astype(np.float32)
    x = torch.from_numpy(x32).to(getattr(torch, xdt))
    got = OP.quantized_matmul(x, qm, transpose_b=transpose)
    assert got.dtype == x.dtype
    xr = x.double().numpy()
    if xdt == "float32":
        # the operator rounds fp32 activations to fp16 precision (the reference's dot: TF32) and the result to fp16
        _check(got, xr, qm_ref, transpose, atol=ATOL, rtol=2 * RTOL)
    elif xdt == "bfloat16":
        _check(got, xr, qm_ref, transpose, atol=ATOL, rtol=2.0 ** -8)      # result rounded to bf16
    else:
        _check(got, xr, qm_ref, transpose)


RAGGED4 = [(137, 909, 256), (1, 50257, 768), (16, 909, 256), (5, 1000, 64), (300, 72, 136), (33, 24, 40),
           (64, 909, 66), (2, 8, 8)]


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("xdt", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K", RAGGED4)
def test_qmatmul_4bit_rows_that_are_not_multiples_of_16_channels(OP, M, N, K, xdt, transpose):
    """test_kernel.py:13 of the reference holds (137, 909, 256); a vocabulary-sized N is the other common case."""
    import torch
    qm = _matrix4(M + N + K, K, N, np.float32)
    rng = np.random.default_rng(7)
    x32 = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0)).astype(np.float32)
    x = torch.from_numpy(x32).to(getattr(torch, xdt))
    got = OP.quantized_matmul(x, qm, transpose_b=transpose)
    _check(got, x.double().numpy(), qm, transpose, rtol=RTOL if xdt == "float16" else 2.0 ** -8)


def test_qmatmul_4bit_unaligned_operands(OP):
    """Views that start in the middle of an allocation: 2-byte aligned activations, 1-byte aligned weights."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(3)
    for (M, N, K) in ((4, 512, 256), (48, 640, 320), (48, 200, 96)):
        qm = _matrix4(N, K, N, np.float16)
        buf = torch.zeros(qm.int_weight.size + 3, dtype=torch.uint8, device="cuda")
        iw = buf[3:].view(K // 2, N)
        iw.copy_(torch.from_numpy(qm.int_weight))
        xb = torch.zeros(M * K + 1, dtype=torch.float16, device="cuda")
        x = xb[1:].view(M, K)
        x32 = rng.standard_normal((M, K)).astype(np.float16)
        x.copy_(torch.from_numpy(x32))
        g = G.QuantizedMatrix(iw, torch.from_numpy(qm.zero).cuda(), torch.from_numpy(qm.scale).cuda())
        got = OP.quantized_matmul(x, g)
        _check(got, x32.astype(np.float64), qm, False)
        yb = torch.zeros(M * N + 1, dtype=torch.float16, device="cuda")
        y = yb[1:].view(M, N)
        y32 = (0.05 * rng.standard_normal((M, N))).astype(np.float16)
        y.copy_(torch.from_numpy(y32))
        got = OP.quantized_matmul(y, g, transpose_b=True)
        _check(got, y32.astype(np.float64), qm, True)


def test_pack_unpack_8bit_against_the_oracle():
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(11)
    for shape, axis in (((64, 48), 0), ((5, 30, 7), 1), ((33, 3), 0), ((4, 6, 10), 2)):
        pshape = tuple(d for i, d in enumerate(shape) if i != axis)
        scale = rng.uniform(0.001, 0.01, pshape).astype(np.float32)
        zero = rng.integers(0, 256, pshape).astype(np.float32)
        codes = rng.integers(0, 256, shape).astype(np.uint8)
        Q = ((codes.astype(np.float32) - np.expand_dims(zero, axis)) * np.expand_dims(scale, axis)).astype(np.float32)
        params = {"scale": scale, "zero": zero, "maxq": 255}
        ref = O.pack_matrix(Q, params, contraction_axis=axis)
        got = G.pack_matrix(Q, params, contraction_axis=axis)
        assert got.bits == 8 and ref.bits == 8 and got.shape == tuple(shape)
        assert np.array_equal(to_np(got.int_weight), ref.int_weight)
        assert np.array_equal(ref.int_weight, codes)
        assert np.array_equal(to_np(G.unpack_matrix(got)), O.unpack_matrix(ref))


def test_gptq_8bit_solve_pack_matmul_against_the_oracle(OP):
    """bits = 8 through the whole path: solve, pack (one code per byte), product."""
    import jax_gptq_amd.gptq as G
    from helpers import code_stats, recon_error
    rng = np.random.default_rng(21)
    K, N, n = 256, 320, 1024
    W = (0.02 * rng.standard_normal((K, N))).astype(np.float32)
    X = rng.standard_normal((n, K)).astype(np.float32)
    Q, params = G.gptq(W, [X], bits=8)
    Qr, pr = O.gptq(W, [X], _bits=8)
    assert np.allclose(to_np(params["scale"]), pr["scale"], rtol=1e-5) and params["maxq"] == 255
    packed = G.pack_matrix(Q, params)
    pr_packed = O.pack_matrix(Qr, pr)
    frac, mx = code_stats(to_np(packed.int_weight), pr_packed.int_weight)
    assert frac <= 1e-3 and mx <= 1
    e, er = recon_error(W, to_np(Q), X), recon_error(W, Qr, X)
    assert abs(e - er) <= 0.01 * er
    x = rng.standard_normal((4, K)).astype(np.float16)
    qm_ref = O.QuantizedMatrix(to_np(packed.int_weight), to_np(params["zero"]), to_np(params["scale"]), bits=8)
    _check(OP.quantized_matmul(x, packed), x.astype(np.float32), qm_ref, False)


def test_qmatmul_8bit_gradient_wrt_x(OP):
    import torch
    import jax_gptq_amd.gptq as G
    qm = _matrix8(9, 256, 192, np.float32)
    g = G.QuantizedMatrix(torch.from_numpy(qm.int_weight).cuda(), torch.from_numpy(qm.zero).cuda(),
                          torch.from_numpy(qm.scale).cuda(), bits=8)
    x = torch.randn((6, 256), device="cuda", dtype=torch.float16, requires_grad=True)
    y = OP.quantized_matmul(x, g)
    w = torch.randn_like(y) * 0.05
    (y * w).sum().backward()
    ref = w.double().cpu().numpy() @ _dense(qm).T
    err = np.abs(x.grad.double().cpu().numpy() - ref)
    assert np.all(err <= ATOL + RTOL * np.abs(ref))


@pytest.mark.parametrize("xdt,zs", [("float16", "float32"), ("float16", "float16"), ("float32", "float32"),
                                    ("bfloat16", "float32")])
@pytest.mark.parametrize("M,N,K", [(3500, 4480, 512), (2048, 11008, 1024), (4096, 4096, 576), (2000, 4224, 1088)])
def test_qmatmul_8bit_many_rows_128x512_tiles(OP, M, N, K, xdt, zs):
    """8-bit codes, many fp16 (or fp32) rows: the leading columns that fill whole rounds of workgroups run on the
    128 x 512 tiles (the shapes of the 4-bit test: 8 x 512 + 384 columns, 16 tiles + 22 x 128 columns, a ragged
    last row tile, an odd number of 64-k stages, 128 x 256 tiles where the wide ones are under a round), whose
    8-bit form pairs the bytes of two rows as fp16 subnormals; bf16 rows stay on the 128-row tiles.  Fractional
    zero points leave through the row sums."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 256, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.0001, 0.001, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 255.0, N).astype(np.float32)).to(tdt)
    qm = G.QuantizedMatrix(torch.from_numpy(codes).cuda(), zero.cuda(), scale.cuda(), bits=8)
    rowscale = np.array([1.0, 1e-3, 3e4])[np.arange(M) % 3][:, None] if xdt == "float32" else np.ones((M, 1))
    x = torch.from_numpy((rng.standard_normal((M, K)) * rowscale).astype(np.float32)).to(getattr(torch, xdt))
    got = OP.quantized_matmul(x, qm)
    assert got.dtype == getattr(torch, xdt) and tuple(got.shape) == (M, N)
    dense = (codes.astype(np.float64) - zero.double().numpy()[None]) * scale.double().numpy()[None]
    ref = x.double().numpy() @ dense
    err = np.abs(to_np(got).astype(np.float64) - ref)
    rel = 2.0 ** -8 if xdt == "bfloat16" else RTOL
    tol = (ATOL + rel * np.abs(ref / rowscale)) * rowscale
    assert np.all(err <= tol), float((err / tol).max())


@pytest.mark.parametrize("xdt,zs", [("float16", "float32"), ("float16", "float16"), ("float32", "bfloat16"),
                                    ("bfloat16", "float32")])
@pytest.mark.parametrize("M,N,K", [(3500, 512, 4480), (2048, 1024, 11008), (4096, 576, 4096), (1800, 20480, 4096),
                                   (2000, 1088, 4224)])
def test_qmatmul_8bit_many_rows_128x512_tiles_transposed(OP, M, N, K, xdt, zs):
    """The transposed product of many fp16 (or fp32) rows against 8-bit codes on the 128 x 512 tiles: a packed row
    is one output column, 512 of them per workgroup, the contraction along the channels in stages of 64 (an odd
    number of stages, 20480 channels, 128 x 256 tiles where the wide ones are under a round, columns left over for
    the 128-row tiles); bf16 rows stay on the 128-row tiles."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 256, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.0001, 0.001, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 255.0, N).astype(np.float32)).to(tdt)
    qm = G.QuantizedMatrix(torch.from_numpy(codes).cuda(), zero.cuda(), scale.cuda(), bits=8)
    rowscale = np.array([1.0, 1e-3, 3e4])[np.arange(M) % 3][:, None] if xdt == "float32" else np.ones((M, 1))
    x = torch.from_numpy((0.05 * rng.standard_normal((M, N)) * rowscale).astype(np.float32)).to(getattr(torch, xdt))
    got = OP.quantized_matmul(x, qm, transpose_b=True)
    assert got.dtype == getattr(torch, xdt) and tuple(got.shape) == (M, K)
    dense = (codes.astype(np.float64) - zero.double().numpy()[None]) * scale.double().numpy()[None]
    ref = x.double().numpy() @ dense.T
    err = np.abs(to_np(got).astype(np.float64) - ref)
    rel = 2.0 ** -8 if xdt == "bfloat16" else RTOL
    tol = (ATOL + rel * np.abs(ref / rowscale)) * rowscale
    assert np.all(err <= tol), float((err / tol).max())


@pytest.mark.parametrize("xdt", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K", [(17, 1024, 4096), (64, 11008, 512), (100, 2048, 1000), (200, 4096, 1064),
                                   (256, 1152, 2048), (33, 8192, 8192)])
def test_qmatmul_4bit_few_rows_against_a_whole_matrix(OP, M, N, K, xdt):
    """16 < M <= 256 on aligned shapes: the register-operand kernel with and without a split of the
    contraction, full and ragged last k-steps (K % 32 != 0), fractional zero points."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    scale = rng.uniform(0.001, 0.01, N).astype(np.float32)
    zero = rng.uniform(0.0, 15.0, N).astype(np.float32)
    qm_ref = O.QuantizedMatrix(O.pack_colwise(codes), zero, scale)
    qm = G.QuantizedMatrix(torch.from_numpy(qm_ref.int_weight).cuda(), torch.from_numpy(zero).cuda(),
                           torch.from_numpy(scale).cuda())
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(getattr(torch, xdt))
    for rep in range(2):                       # the second call finds the arrival counters as the first left them
        got = OP.quantized_matmul(x, qm)
        _check(got, x.double().numpy(), qm_ref, False, rtol=RTOL if xdt == "float16" else 2.0 ** -8)


def test_qmatmul_more_rows_than_a_grid_dimension_on_the_plain_kernels(OP):
    """Shapes no matrix-core kernel takes (fewer than 8 channels) with M > 65535: several launches."""
    import torch
    qm = _matrix4(5, 16, 4, np.float32)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((70000, 16)).astype(np.float16)
    got = OP.quantized_matmul(x, qm)
    _check(got, x.astype(np.float64), qm, False)
    y = (0.05 * rng.standard_normal((70000, 4))).astype(np.float16)
    _check(OP.quantized_matmul(y, qm, transpose_b=True), y.astype(np.float64), qm, True)
