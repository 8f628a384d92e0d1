"""GPU parity of the packed-int4 matmul (forward and transposed) against the oracle.

Tolerance (task statement): atol 1e-2, rtol 1e-3 against the fp32 dense product.
"""
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


def _matrix(seed, K, N, zs_dtype=np.float32):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    scale = rng.uniform(0.001, 0.01, N).astype(zs_dtype)
    zero = rng.integers(0, 16, N).astype(zs_dtype)
    return O.QuantizedMatrix(O.pack_colwise(codes), zero, scale)


def _check(got, x, qm, transpose):
    dense = ((O.unpack_colwise(qm.int_weight).astype(np.float64) - qm.zero.astype(np.float64)[None])
             * qm.scale.astype(np.float64)[None])
    ref = x.astype(np.float64) @ (dense.T if transpose else dense)
    got = to_np(got).astype(np.float64)
    assert got.shape == ref.shape
    err = np.abs(got - ref)
    # fp16 rounding of the result (2^-11 relative) is part of the operator's definition
    tol = ATOL + RTOL * np.abs(ref)
    assert np.all(err <= tol), f"max err {err.max():.3e} at |ref|={np.abs(ref).flat[err.argmax()]:.3e}"


# shapes of the reference's test_kernel.py:13 plus the decode shapes of the benchmark config
SHAPES = [(137, 909, 256), (32, 1024, 2048), (37, 32000, 5120), (1, 11008, 4096), (16, 4096, 11008),
          (128, 11008, 4096), (128, 4096, 11008), (70, 2304, 768), (3, 130, 66), (1, 64, 2)]


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_qmatmul_fp16(OP, M, N, K, transpose):
    qm = _matrix(M + N + K, K, N, np.float16)
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0)).astype(np.float16)
    got = OP.quantized_matmul(x, qm, transpose_b=transpose)
    assert to_np(got).dtype == np.float16
    _check(got, x.astype(np.float32), qm, transpose)
    ref = O.quantized_matmul(x, qm, transpose_b=transpose)
    assert np.allclose(to_np(got).astype(np.float32), ref.astype(np.float32), atol=ATOL, rtol=2 * RTOL)


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("M,N,K", [(137, 909, 256), (32, 1024, 2048), (5, 192, 384)])
def test_qmatmul_fp32_x_and_params(OP, M, N, K, transpose):
    qm = _matrix(M * 3 + N, K, N, np.float32)
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0)).astype(np.float32)
    got = OP.quantized_matmul(x, qm, transpose_b=transpose)
    assert to_np(got).dtype == np.float32
    _check(got, x, qm, transpose)


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 11008, 4096), (16, 4096, 11008), (200, 5120, 256), (2048, 4096, 1024),
                                   (9000, 256, 128)])
def test_qmatmul_fp32_x_on_the_matrix_core_kernels(OP, M, N, K, transpose):
    """fp32 activations with C % 16 == 0 are rounded to fp16 precision (the reference's dot rounds
    them to TF32: same mantissa width) after a per-row power-of-two scaling and run on the fp16
    kernels.  Rows of very different magnitude (1e-20 to 1e20, far outside fp16) check the scaling;
    M = 9000 spans two row chunks.  With the workspace of the 16-bit query the same call stays on the
    unrounded kernels."""
    import torch
    import jax_gptq_amd._native as NV
    qm = _matrix(M + N + K, K, N, np.float32)
    rng = np.random.default_rng(11)
    rowscale = np.array([1.0, 1e-3, 3e4, 1e20, 1e-20])[np.arange(M) % 5][:, None]
    x = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0) * rowscale).astype(np.float32)
    got = to_np(OP.quantized_matmul(x, qm, transpose_b=transpose)).astype(np.float64)
    assert got.dtype == np.float64 and to_np(OP.quantized_matmul(x, qm, transpose_b=transpose)).dtype == np.float32
    dense = ((O.unpack_colwise(qm.int_weight).astype(np.float64) - qm.zero.astype(np.float64)[None])
             * qm.scale.astype(np.float64)[None])
    ref = x.astype(np.float64) @ (dense.T if transpose else dense)
    tol = (ATOL + RTOL * np.abs(ref / rowscale)) * rowscale       # relative to the row's magnitude
    err = np.abs(got - ref)
    assert np.all(err <= tol), float((err / tol).max())
    if M > 200:
        return
    # the same call with the smaller workspace: plain kernels, fp32 activations unrounded
    lib = NV.load()
    xt = torch.from_numpy(x).cuda()
    pk = torch.from_numpy(np.ascontiguousarray(qm.int_weight)).cuda()
    zero, scale = torch.from_numpy(qm.zero).cuda(), torch.from_numpy(qm.scale).cuda()
    R, C = pk.shape
    out = torch.empty((M, 2 * R if transpose else C), dtype=torch.float32, device="cuda")
    nb = lib.gptq_hip_qmatmul_workspace_bytes(M, R, C, int(transpose))
    assert nb < lib.gptq_hip_qmatmul_workspace_bytes_x(M, R, C, int(transpose), 0)
    ws = torch.zeros(max(nb, 256), dtype=torch.uint8, device="cuda")
    rc = lib.gptq_hip_qmatmul(OP._stream(), xt.data_ptr(), 0, M, pk.data_ptr(), R, C, zero.data_ptr(), scale.data_ptr(),
                              0, int(transpose), out.data_ptr(), ws.data_ptr(), nb)
    assert rc == 0
    torch.cuda.synchronize()
    # (rows whose results leave the fp16 range become infinite there, as in the reference: op.py:43)
    small = (rowscale <= 1.0)[:, 0]
    err = np.abs(out.cpu().numpy().astype(np.float64) - ref)[small]
    assert np.all(err <= 1e-4 + 2.0 ** -10 * np.abs(ref[small]))


@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("zs", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("M", [1, 16, 200])
def test_qmatmul_fractional_zero_points_and_param_dtypes(OP, M, zs, transpose):
    """Zero points need not be integers (the reference subtracts them in fp32, kernel.py:98);
    every kernel of the dispatch table (GEMV, chunked, tiled, transposed) has to honour that."""
    import torch
    import jax_gptq_amd.gptq as G
    K, N = 256, 5120
    rng = np.random.default_rng(M)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.001, 0.01, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 15.0, N).astype(np.float32)).to(tdt)
    qm_ref = O.QuantizedMatrix(O.pack_colwise(codes), zero.float().numpy(), scale.float().numpy())
    qm = G.QuantizedMatrix(torch.from_numpy(qm_ref.int_weight).cuda(), zero.cuda(), scale.cuda())
    x = (rng.standard_normal((M, N if transpose else K)) * (0.05 if transpose else 1.0)).astype(np.float16)
    got = OP.quantized_matmul(x, qm, transpose_b=transpose)
    _check(got, x.astype(np.float32), qm_ref, transpose)


def test_qmatmul_bf16_x(OP):
    import torch
    qm = _matrix(77, 512, 384, np.float32)
    x = torch.randn((9, 512), generator=torch.Generator().manual_seed(0)).to(torch.bfloat16)
    got = OP.quantized_matmul(x, qm)
    assert got.dtype == torch.bfloat16
    dense = O.unpack_matrix(qm)
    ref = x.float().numpy() @ dense
    assert np.allclose(to_np(got), ref, atol=3e-2, rtol=1e-2)    # bf16 result: 2^-8 relative


@pytest.mark.parametrize("zs", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,N,K", [(1, 11008, 4096), (3, 4096, 11008), (16, 4096, 11008), (128, 4096, 1024),
                                   (70, 2304, 768), (5, 48, 96), (200, 5120, 256), (300, 11008, 512)])
def test_qmatmul_bf16_x_mfma_path(OP, M, N, K, zs):
    """bf16 activations on the 16-bit MFMA kernel (both nibbles dequantise to 128 + code, which
    bf16 holds exactly); the result is rounded once, to bf16 (2^-9 relative)."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.001, 0.01, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 15.0, N).astype(np.float32)).to(tdt)      # fractional, too
    qm = G.QuantizedMatrix(torch.from_numpy(O.pack_colwise(codes)).cuda(), zero.cuda(), scale.cuda())
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16)
    got = OP.quantized_matmul(x, qm)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (M, N)
    dense = (codes.astype(np.float64) - zero.double().numpy()[None]) * scale.double().numpy()[None]
    ref = x.double().numpy() @ dense
    err = np.abs(to_np(got).astype(np.float64) - ref)
    assert np.all(err <= 1e-2 + 2.0 ** -8 * np.abs(ref)), err.max()


@pytest.mark.parametrize("xdt,zs", [("float16", "float32"), ("float16", "float16"), ("bfloat16", "float32"),
                                    ("bfloat16", "bfloat16"), ("float32", "float32")])
@pytest.mark.parametrize("M,N,K", [(3500, 4480, 512), (2048, 11008, 1024), (4096, 4096, 576), (2000, 4224, 1088)])
def test_qmatmul_many_rows_128x512_tiles(OP, M, N, K, xdt, zs):
    """Forward products of many rows: the leading columns that fill whole rounds of workgroups run on
    128 x 512 tiles whose wavefronts share the activations through LDS, the rest on the 128- and 64-row
    tiles (4480 = 8 x 512 + 384 columns; 11008: 16 tiles + 22 x 128 columns; M = 3500 leaves a ragged
    last row tile; K = 576 has an odd number of 64-k stages; 2000 x 4224: the 512-channel tiles are
    under one round of workgroups, so 128 x 256 tiles of four 64 x 128 wavefronts take 16 x 256 columns).
    Fractional zero points exercise the row sums that the wavefronts exchange; fp32 rows the scaled
    fp32 store."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.001, 0.01, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 15.0, N).astype(np.float32)).to(tdt)
    qm = G.QuantizedMatrix(torch.from_numpy(O.pack_colwise(codes)).cuda(), zero.cuda(), scale.cuda())
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


@pytest.mark.parametrize("xdt,zs", [("float16", "float32"), ("float16", "float16"), ("float16", "bfloat16"),
                                    ("float32", "float32"), ("bfloat16", "float32"), ("bfloat16", "bfloat16")])
@pytest.mark.parametrize("M,N,K", [(17, 11008, 4096), (32, 11008, 4096), (33, 4096, 11008), (64, 11008, 4096),
                                   (50, 80, 2304), (128, 4096, 4096), (100, 1104, 1024), (256, 3072, 768),
                                   (40, 64, 256)])
def test_qmatmul_few_dozen_rows_tall_narrow_tiles(OP, M, N, K, xdt, zs):
    """17 to a few dozen fp16 rows (up to 128 / 256 on small matrices), K a multiple of 256, C of 16: 32- or 64-row
    tiles of 64 channels whose eight wavefronts split the contraction and share the activations through LDS
    (4096 x 11008: 172 workgroups over all of K; 11008 x 4096 and 4096 x 4096: 64 column tiles x 4 splits, partial
    tiles through the workspace; 80 and 1104 channels: a last tile of 16 channels; M = 33, 50, 100: ragged row
    tiles; 2304 = 9 stages and 256 = 1 stage: the loop's remainder).  The weight operands are formed as
    (code - zero) 2^-9 in fp16, so a fractional zero point costs fp16's relative precision and no more; fp32 rows
    of very different magnitudes go through the scaled fp16 staging and the tiles' own fp32 store; bf16 rows multiply
    128 + code and the term in 128 + zero leaves through row sums that one more MFMA per row block accumulates
    (two passes of the final reduction for 64-row tiles; a split applies the term to its own partial sums)."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.001, 0.01, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 15.0, N).astype(np.float32)).to(tdt)      # fractional, too
    if xdt == "float32":
        zero = zero.round()     # (the rounding of fp32 rows to fp16 uses up the tolerance at K = 11008 by itself)
    qm = G.QuantizedMatrix(torch.from_numpy(O.pack_colwise(codes)).cuda(), zero.cuda(), scale.cuda())
    rowscale = np.array([1.0, 1e-3, 3e4])[np.arange(M) % 3][:, None] if xdt == "float32" else np.ones((M, 1))
    x = torch.from_numpy((rng.standard_normal((M, K)) * rowscale).astype(np.float32)).to(getattr(torch, xdt))
    dense = (codes.astype(np.float64) - zero.double().numpy()[None]) * scale.double().numpy()[None]
    ref = x.double().numpy() @ dense
    tol = (ATOL + (2.0 ** -8 if xdt == "bfloat16" else RTOL) * np.abs(ref / rowscale)) * rowscale
    first = None
    for rep in range(3):            # the split sums leave their counters as they found them
        got = OP.quantized_matmul(x, qm)
        assert got.dtype == getattr(torch, xdt) and tuple(got.shape) == (M, N)
        err = np.abs(to_np(got).astype(np.float64) - ref)
        assert np.all(err <= tol), float((err / tol).max())
        first = got.clone() if first is None else first
        assert torch.equal(got, first)          # and are summed in split order: the same bits every time


@pytest.mark.parametrize("xdt,zs", [("float16", "float32"), ("float16", "float16"), ("float32", "bfloat16"),
                                    ("bfloat16", "float32"), ("bfloat16", "bfloat16")])
@pytest.mark.parametrize("M,N,K", [(3500, 512, 4480), (2048, 1024, 11008), (4096, 576, 4096), (1800, 20480, 8192),
                                   (2000, 1088, 4224)])      # (4224 output columns: 128 x 256 tiles, as forward)
def test_qmatmul_many_rows_128x512_tiles_transposed(OP, M, N, K, xdt, zs):
    """The transposed product of many fp16 (or fp32) rows on the same tiling: 512 output columns per
    workgroup, contraction along the channels in stages of 64 (N = 576: an odd number of stages;
    N = 20480 channels: more than the other kernel's LDS holds constants for, so its tiles split the
    contraction while these do not).  bf16 rows (up to 16384 channels): the scale multiplies the rows on their
    way into LDS, the weights enter as 128 + code and the term in 128 + zero leaves through a ninth tile that the
    wavefronts share out (fractional zero points included); 20480 channels stay on the 128-row tiles."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.001, 0.01, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 15.0, N).astype(np.float32)).to(tdt)
    qm = G.QuantizedMatrix(torch.from_numpy(O.pack_colwise(codes)).cuda(), zero.cuda(), scale.cuda())
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


@pytest.mark.parametrize("zs", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K", [(1, 4096, 11008), (16, 11008, 4096), (128, 4096, 1024), (70, 2304, 768),
                                   (5, 48, 96), (200, 5120, 256), (300, 1008, 514), (2048, 4096, 512)])
def test_qmatmul_bf16_x_transposed_mfma_path(OP, M, N, K, zs):
    """Transposed product with bf16 activations: the scale multiplies the activations (rounded
    once to bf16, which is their own precision), the weights enter as 128 + code, and the term in
    128 + zero leaves through fp32 row sums; the result is rounded once, to bf16."""
    import torch
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(M + N + K)
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    tdt = getattr(torch, zs)
    scale = torch.from_numpy(rng.uniform(0.001, 0.01, N).astype(np.float32)).to(tdt)
    zero = torch.from_numpy(rng.uniform(0.0, 15.0, N).astype(np.float32)).to(tdt)      # fractional, too
    qm = G.QuantizedMatrix(torch.from_numpy(O.pack_colwise(codes)).cuda(), zero.cuda(), scale.cuda())
    x = torch.from_numpy((0.05 * rng.standard_normal((M, N))).astype(np.float32)).to(torch.bfloat16)
    got = OP.quantized_matmul(x, qm, transpose_b=True)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (M, K)
    dense = (codes.astype(np.float64) - zero.double().numpy()[None]) * scale.double().numpy()[None]
    ref = x.double().numpy() @ dense.T
    err = np.abs(to_np(got).astype(np.float64) - ref)
    # rounding of x * scale to bf16 (2^-9 per term, random signs) and of the result (2^-9)
    assert np.all(err <= 1e-2 + 2.0 ** -8 * np.abs(ref)), err.max()
    # the fp16 kernel on the same values (exactly representable: bf16 -> fp16 of |x| < 1 loses nothing
    # above 2^-14) agrees to the bf16 rounding of the result
    got16 = OP.quantized_matmul(x.to(torch.float16), qm, transpose_b=True)
    d = np.abs(to_np(got).astype(np.float64) - to_np(got16).astype(np.float64))
    assert np.all(d <= 1e-2 + 2.0 ** -7 * np.abs(ref)), d.max()


@pytest.mark.parametrize("M,N,K,xdt,zs", [(1, 28672, 7168, "float16", "float16"),
                                            (16, 7168, 28672, "float16", "float32"),
                                            (3, 29936, 9000, "float16", "float32"),
                                            (5, 28672, 7168, "bfloat16", "bfloat16"),
                                            (2, 32000, 5120, "float16", "float16")])
def test_qmatmul_streaming_kernel_large_matrices(OP, M, N, K, xdt, zs):
    """M <= 16 on matrices of 80 MB and more runs the decode kernel's ring-loop form (long row range per
    workgroup, register ring of loads); (3, 29936, 9000) has a ragged last k-step, a partial
    last strip and fractional zero points.  Reference: fp32 dense product by torch on the
    device (the host evaluation of these sizes takes minutes)."""
    import torch
    import jax_gptq_amd.gptq as G
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    pk = torch.randint(0, 256, (K // 2, N), dtype=torch.uint8, device="cuda", generator=g)
    tz = getattr(torch, zs)
    zero = (15.0 * torch.rand((N,), device="cuda", generator=g)).to(tz)
    scale = (0.001 + 0.009 * torch.rand((N,), device="cuda", generator=g)).to(tz)
    x = torch.randn((M, K), device="cuda", generator=g).to(getattr(torch, xdt))
    got = OP.quantized_matmul(x, G.QuantizedMatrix(pk, zero, scale))
    assert got.dtype == x.dtype and tuple(got.shape) == (M, N)
    codes = torch.stack([pk & 15, pk >> 4], dim=1).reshape(K, N).float()
    dense = (codes - zero.float()[None]) * scale.float()[None]
    del codes
    ref = x.double() @ dense.double() if M <= 4 else (x.float() @ dense).double()
    err = (got.double() - ref).abs()
    rtol = 2.0 ** -8 if xdt == "bfloat16" else 2 * RTOL       # rounding of the result itself
    assert bool((err <= ATOL + rtol * ref.abs()).all()), float(err.max())
    # not 16-byte aligned activations take the chunked kernel: same values up to summation order
    xu = torch.empty((M * K + 2,), device="cuda", dtype=x.dtype)[2:].view(M, K)
    xu.copy_(x)
    assert xu.data_ptr() % 16 != 0
    got_u = OP.quantized_matmul(xu, G.QuantizedMatrix(pk, zero, scale))
    assert bool(((got_u.double() - ref).abs() <= ATOL + rtol * ref.abs()).all())


def test_qmatmul_leading_dims_and_errors(OP):
    qm = _matrix(8, 256, 192)
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 3, 5, 256)).astype(np.float32)
    got = OP.quantized_matmul(x, qm)
    assert tuple(got.shape) == (2, 3, 5, 192)
    _check(to_np(got).reshape(-1, 192), x.reshape(-1, 256), qm, False)
    with pytest.raises(AssertionError):
        OP.quantized_matmul(x[..., :-2], qm)
    with pytest.raises(AssertionError):
        OP.quantized_matmul(x, qm, transpose_b=True)


def test_qmatmul_gradient_wrt_x(OP):
    """custom-VJP counterpart (reference op.py:71-81): grad wrt x is y_bar @ dequant(W)^T."""
    import torch
    qm = _matrix(9, 256, 128)
    dense = O.unpack_matrix(qm)
    x = torch.randn((6, 256), generator=torch.Generator().manual_seed(1)).cuda().requires_grad_(True)
    y = OP.quantized_matmul(x, qm)
    y[3].sum().backward()
    ref = np.zeros((6, 256), np.float32)
    ref[3] = dense.sum(axis=1)
    assert np.allclose(to_np(x.grad), ref, atol=1e-1)      # reference tests.py:186 uses atol 1e-1
    assert np.allclose(to_np(x.grad), ref, atol=ATOL, rtol=RTOL)


def test_qmatmul_after_gptq_matches_dense(OP):
    """End to end as in the reference's test_kernel.py: solve, pack, multiply."""
    import jax_gptq_amd.gptq as G
    rng = np.random.default_rng(4)
    M, N, K = 137, 909, 256
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    quant_w, params = G.gptq(W, [x])
    packed = G.pack_matrix(quant_w, params)
    for transpose in (False, True):
        inp = rng.standard_normal((M, N)).astype(np.float32) if transpose else x
        ret = to_np(OP.quantized_matmul(inp, packed, transpose_b=transpose))
        qw = to_np(quant_w)
        expected = inp @ (qw.T if transpose else qw)
        assert np.mean(np.abs(ret - expected)) < 3e-2        # reference test_kernel.py:41


@pytest.mark.parametrize("M,xdt", [(1, "float16"), (16, "bfloat16"), (200, "float16"), (3, "float32"),
                                   (2048, "float16")])      # (2048 rows: three launches, 128 x 512 tiles first)
def test_qmatmul_in_a_captured_graph(OP, M, xdt):
    """A decode loop would capture the matmul in a HIP graph: the call only enqueues kernels (no
    memset, no allocation of its own, split-K counters left at zero by every launch), so a graph
    that holds it can be replayed; every replay, with eager calls in between, must give the eager
    result for the input contents of that moment."""
    import torch
    import jax_gptq_amd.gptq as G
    K, N = 4096, 11008
    g = torch.Generator(device="cuda").manual_seed(M)
    pk = torch.randint(0, 256, (K // 2, N), dtype=torch.uint8, device="cuda", generator=g)
    zero = torch.randint(0, 16, (N,), device="cuda", generator=g).float()
    scale = 0.001 + 0.009 * torch.rand((N,), device="cuda", generator=g)
    qm = G.QuantizedMatrix(pk, zero, scale)
    x = torch.randn((M, K), device="cuda", generator=g).to(getattr(torch, xdt))
    eager = OP.quantized_matmul(x, qm).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        OP.quantized_matmul(x, qm)                       # warm-up on the capture stream (workspace)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        y = OP.quantized_matmul(x, qm)
    for rep in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), rep
        # eager work and new input contents between the replays
        x.copy_(torch.randn((M, K), device="cuda", generator=g).to(x.dtype))
        eager = OP.quantized_matmul(x, qm).clone()
        torch.cuda.synchronize()


@pytest.mark.parametrize("xdt", ["float16", "float32"])
@pytest.mark.parametrize("kind", ["positive", "tiny"])
@pytest.mark.parametrize("M,N,K", [(1, 11008, 4096), (16, 11008, 4096), (1, 4096, 11008), (16, 4096, 11008),
                                   (16, 28672, 7168)])
def test_qmatmul_decode_shapes_with_nonzero_mean_and_tiny_activations(OP, M, N, K, kind, xdt):
    """Activations that are all positive (|N(0,1)| + 1, as after a GELU / SiLU: any constant the
    kernel adds to the codes and removes afterwards is multiplied by a large sum of x) and
    activations of magnitude 1e-3 (anything the kernel scales down inside fp16 would go
    subnormal), at the decode shapes, against the fp64 dense product at the operator's bar."""
    qm = _matrix(M + N + K, K, N, np.float16)
    rng = np.random.default_rng(17)
    x = rng.standard_normal((M, K))
    x = (np.abs(x) + 1.0) if kind == "positive" else 1e-3 * x
    x = x.astype(xdt)
    got = OP.quantized_matmul(x, qm)
    _check(got, x.astype(np.float32), qm, False)
