"""Seeded random sweep of the packed matmul over everything the dispatcher distinguishes: code width, rows,
ragged and tiny shapes, direction, activation and parameter types, grouped parameters, unaligned weights.
Every case is checked against the fp64 dense product (atol 1e-2, rtol 2e-3 for fp16 activations and results,
3e-3 for fp32 ones, which enter rounded to fp16 precision, 2^-7 for bf16 ones; for bf16 activations the terms'
own rounding, eight standard deviations of it, is allowed on top)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(rng):
    bits = int(rng.choice([4, 8]))
    M = int(rng.choice([1, 2, 7, 16, 17, 31, 64, 65, 100, 255, 256, 257, 700]))
    K = int(rng.choice([8, 10, 24, 32, 34, 40, 64, 66, 96, 128, 130, 250, 256, 520, 1024, 2050, 4096]))
    if bits == 4 and K % 2:
        K += 1
    N = int(rng.choice([8, 9, 15, 16, 17, 64, 100, 127, 128, 129, 255, 256, 300, 909, 1024, 2047, 4096]))
    tr = bool(rng.integers(0, 2))
    xdt = str(rng.choice(["float16", "bfloat16", "float32"]))
    zs = str(rng.choice(["float32", "float16", "bfloat16"]))
    group = 0
    if rng.random() < 0.3:
        cands = [g for g in (2, 32, 64, 128, 256) if K % g == 0]
        if cands:
            group = int(rng.choice(cands))
    return bits, M, K, N, tr, xdt, zs, group, int(rng.integers(0, 2))


def _wide_case(rng):
    """More than 64 rows against 160 or more column tiles of 128 channels: the shapes that run on 128-row tiles
    (aligned, ragged and grouped instantiations; k-steps that end inside a 32-wide step)."""
    bits = int(rng.choice([4, 8]))
    M = int(rng.choice([65, 128, 129, 200, 257]))
    K = int(rng.choice([32, 40, 64, 72, 96, 160, 200]))
    N = int(rng.choice([20480, 20488, 20490, 24001, 50257]))
    xdt = str(rng.choice(["float16", "bfloat16", "float32"]))
    zs = str(rng.choice(["float32", "float16", "bfloat16"]))
    group = 0
    if rng.random() < 0.3:
        cands = [g for g in (32, 64, 96) if K % g == 0]
        if cands:
            group = int(rng.choice(cands))
    return bits, M, K, N, False, xdt, zs, group, int(rng.integers(0, 2))


@pytest.mark.parametrize("seed", range(3))
def test_qmatmul_random_cases_with_many_column_tiles(seed):
    _run_cases(np.random.default_rng(2000 + seed), _wide_case, 14)


def _ragged_decode_case(rng):
    """Up to 16 rows, 4-bit, K a multiple of 8, N no multiple of 16: the decode kernel's form for rows of any
    length (unaligned row starts; a last strip whose lanes reach past the row), from tiny to vocabulary-sized."""
    M = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 16]))
    K = int(rng.choice([8, 64, 128, 256, 520, 768, 1024, 4096]))
    N = int(rng.choice([17, 31, 100, 255, 257, 300, 909, 1000, 4097, 8193, 50257]))
    xdt = str(rng.choice(["float16", "bfloat16"]))
    zs = str(rng.choice(["float32", "float16", "bfloat16"]))
    return 4, M, K, N, False, xdt, zs, 0, int(rng.integers(0, 2))


@pytest.mark.parametrize("seed", range(3))
def test_qmatmul_random_cases_few_rows_ragged_columns(seed):
    _run_cases(np.random.default_rng(3000 + seed), _ragged_decode_case, 30)


@pytest.mark.parametrize("seed", range(6))
def test_qmatmul_random_cases(seed):
    _run_cases(np.random.default_rng(1000 + seed), _case, 25)


def _run_cases(rng, make_case, count):
    import torch
    import jax_gptq_amd.gptq as G
    from jax_gptq_amd.op import quantized_matmul
    failures = []
    for it in range(count):
        bits, M, K, N, tr, xdt, zs, group, off = make_case(rng)
        top = 16 if bits == 4 else 256
        codes = rng.integers(0, top, (K, N)).astype(np.uint8)
        tdt = getattr(torch, zs)
        shape = (K // group, N) if group else (N,)
        scale = torch.from_numpy((rng.uniform(0.001, 0.01, shape) / (1 if bits == 4 else 16)).astype(np.float32)).to(tdt)
        zero = torch.from_numpy(rng.integers(0, top, shape).astype(np.float32)).to(tdt)
        iw = (codes[0::2] | (codes[1::2] << 4)).astype(np.uint8) if bits == 4 else codes
        buf = torch.zeros(iw.size + 8, dtype=torch.uint8, device="cuda")      # off = 1: a view 3 bytes into it
        iwt = buf[3 * off: 3 * off + iw.size].view(iw.shape)
        iwt.copy_(torch.from_numpy(iw))
        qm = G.QuantizedMatrix(iwt, zero.cuda(), scale.cuda(), bits=bits, group_size=group)
        z64, s64 = zero.double().numpy(), scale.double().numpy()
        if group:
            z64, s64 = np.repeat(z64, group, 0), np.repeat(s64, group, 0)
        dense = (codes.astype(np.float64) - z64) * s64
        dense = dense.T if tr else dense
        x32 = (rng.standard_normal((M, dense.shape[0])) * (0.05 if tr else 1.0)).astype(np.float32)
        x = torch.from_numpy(x32).to(getattr(torch, xdt)).cuda()
        got = quantized_matmul(x, qm, transpose_b=tr).double().cpu().numpy()
        xd = x.double().cpu().numpy()
        want = xd @ dense
        rtol = {"float16": 2e-3, "float32": 3e-3, "bfloat16": 2.0 ** -7}[xdt]
        tol = 1e-2 + rtol * np.abs(want)
        if xdt == "bfloat16":
            tol = tol + 8 * 2.0 ** -9 / np.sqrt(3.0) * np.sqrt((xd ** 2) @ (dense ** 2))
        err = np.abs(got - want)
        if np.isnan(got).any() or not np.all(err <= tol):
            failures.append((bits, M, K, N, tr, xdt, zs, group, off, float((err - tol).max())))
    assert not failures, failures
