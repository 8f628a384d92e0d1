"""The packed matmul's dispatch, asked on the host (no GPU): every kernel family is reached by at least one of the
shapes that the GPU parity tests and the benchmark run, so a threshold edit cannot strand a family untested; and the
kernels that the benchmark's headline cases run are the ones the design names."""
import pytest


@pytest.fixture(scope="module")
def N():
    from jax_gptq_amd import _native
    _native.load()
    return _native


# (M, N, K, transposed, x dtype, bits, aligned): shapes of tests/test_gpu_qmatmul.py, test_gpu_bits8.py and bench.py
CASES = [
    # test_qmatmul_fp16 (the reference's test_kernel.py:13 shapes + the decode shapes)
    *[(M, Nc, K, t, "F16", 4, 1) for (M, Nc, K) in [(137, 909, 256), (32, 1024, 2048), (37, 32000, 5120),
                                                     (1, 11008, 4096), (16, 4096, 11008), (128, 11008, 4096),
                                                     (128, 4096, 11008), (70, 2304, 768), (3, 130, 66), (1, 64, 2)]
      for t in (0, 1)],
    # bench.py
    *[(M, 11008, 4096, 0, "F16", 4, 1) for M in (1, 16, 32, 64, 128, 2048)],
    *[(M, 4096, 11008, 0, "F16", 4, 1) for M in (1, 16, 32, 64, 128, 2048)],
    (2048, 11008, 4096, 1, "F16", 4, 1), (2048, 4096, 11008, 1, "F16", 4, 1), (2048, 11008, 4096, 1, "BF16", 4, 1),
    (1, 11008, 4096, 0, "F32", 4, 1), (128, 11008, 4096, 0, "F32", 4, 1),
    (1, 28672, 7168, 0, "F16", 4, 1), (16, 28672, 7168, 0, "F16", 4, 1), (2048, 28672, 7168, 0, "F16", 4, 1),
    (2048, 28672, 7168, 1, "F16", 4, 1), (2048, 28672, 7168, 1, "BF16", 4, 1), (2048, 11008, 4096, 0, "F16", 8, 1),
    (1, 11008, 4096, 0, "F16", 8, 1), (128, 11008, 4096, 0, "F16", 8, 1), (2048, 11008, 4096, 1, "F16", 8, 1),
    (1, 50257, 768, 0, "F16", 4, 1), (512, 50257, 768, 0, "F16", 4, 1), (512, 50257, 768, 1, "F16", 4, 1),
    # the tall, narrow tiles, the 128 x 512 / 128 x 256 tiles and their transposed forms
    (17, 11008, 4096, 0, "F16", 4, 1), (50, 80, 2304, 0, "F16", 4, 1), (256, 3072, 768, 0, "F16", 4, 1),
    (3500, 4480, 512, 0, "F16", 4, 1), (2000, 4224, 1088, 0, "F16", 4, 1), (3500, 512, 4480, 1, "F16", 4, 1),
    (2000, 1088, 4224, 1, "F16", 4, 1),
    # test_qmatmul_streaming_kernel_large_matrices: matrices of 80 MB and more, aligned and not
    (3, 29936, 9000, 0, "F16", 4, 1), (16, 28672, 7168, 0, "F16", 4, 0), (4, 4096, 4096, 0, "F16", 4, 0),
    # transposed products of few rows, and of many rows on the tiled kernel
    (16, 11008, 4096, 1, "F16", 4, 1), (512, 4096, 11008, 1, "F16", 4, 1), (600, 1024, 8192, 1, "F16", 4, 1),
    # small forward products whose register-operand tiles are too few, and matrices of fewer than 8 channels
    (100, 128, 192, 0, "F16", 4, 1), (3, 4, 64, 0, "F16", 4, 1), (3, 4, 64, 1, "F16", 4, 1),
]


def _plan(N, M, Nc, K, t, xdt, bits, aligned):
    R = K // 2 if bits == 4 else K
    return N.qmatmul_plan(M, R, Nc, transpose_b=t, x_dtype=getattr(N, xdt), bits=bits, aligned=aligned)


def test_every_kernel_family_is_reached(N):
    seen = {}
    for case in CASES:
        p = _plan(N, *case)
        assert p["kernel_id"] > 0, case
        seen.setdefault(p["kernel"], case)
        if p["rest"]:
            seen.setdefault(p["rest"], case)
    import ctypes
    lib = N.load()
    families = {lib.gptq_hip_qmatmul_kernel_name(i).decode() for i in range(1, 40)} - {"none"}
    missing = sorted(families - set(seen))
    assert not missing, f"kernel families that no listed shape reaches: {missing}"


def test_headline_cases_run_on_the_kernels_the_design_names(N):
    dec = _plan(N, 1, 11008, 4096, 0, "F16", 4, 1)
    assert dec["kernel"] == "qmm_fwd_dec_kernel" and dec["splits"] > 1
    assert _plan(N, 16, 11008, 4096, 0, "F16", 4, 1)["kernel"] == "qmm_fwd_dec_kernel"
    for M in (17, 32, 64):
        for (Nc, K) in ((11008, 4096), (4096, 11008)):
            assert _plan(N, M, Nc, K, 0, "F16", 4, 1)["kernel"] == "qmm_fwd_mid_kernel", (M, Nc, K)
    assert _plan(N, 64, 11008, 4096, 0, "BF16", 4, 1)["kernel"] == "qmm_fwd_mid_kernel"
    assert _plan(N, 128, 11008, 4096, 0, "F16", 4, 1)["kernel"].startswith("qmm_fwd_reg_kernel")
    big = _plan(N, 2048, 11008, 4096, 0, "F16", 4, 1)
    # the leading 8192 channels on 128 x 512 tiles, the 2816 behind them on 128 x 256 tiles
    assert big["kernel"] == "qmm_fwd_wide_kernel (128 x 512)" and big["rest"] == "qmm_fwd_wide_kernel (128 x 256)"
    # where those would be more than a round, the 128-row register-operand tiles take the rest
    big2 = _plan(N, 4096, 11008, 4096, 0, "F16", 4, 1)
    assert big2["kernel"].startswith("qmm_fwd_wide_kernel") and big2["rest"].startswith("qmm_fwd_reg_kernel")
    assert _plan(N, 2048, 11008, 4096, 1, "F16", 4, 1)["kernel"].startswith("qmm_bwd_wide_kernel")
    assert _plan(N, 2048, 11008, 4096, 1, "BF16", 4, 1)["kernel"].startswith("qmm_bwd_wide_kernel")
    # bf16 rows: the constants of more than 16384 channels do not fit beside the stages
    assert _plan(N, 2048, 28672, 7168, 1, "BF16", 4, 1)["kernel"].startswith("qmm_bwd_reg_kernel (128")
    # 8-bit codes with many fp16 rows, both directions (bf16 rows stay on the 128-row tiles)
    assert _plan(N, 2048, 11008, 4096, 0, "F16", 8, 1)["kernel"].startswith("qmm_fwd_wide_kernel")
    assert _plan(N, 2048, 11008, 4096, 1, "F16", 8, 1)["kernel"].startswith("qmm_bwd_wide_kernel")
    assert _plan(N, 2048, 11008, 4096, 0, "BF16", 8, 1)["kernel"].startswith("qmm_fwd_reg_kernel (128")
    # fp32 rows: converted inside the decode kernel up to 16 rows, staged as fp16 rows beyond
    assert _plan(N, 1, 11008, 4096, 0, "F32", 4, 1)["fp32_rows"] == 2
    assert _plan(N, 128, 11008, 4096, 0, "F32", 4, 1)["fp32_rows"] == 1
    # 8-bit codes and a vocabulary-sized C
    assert _plan(N, 1, 11008, 4096, 0, "F16", 8, 1)["kernel"] == "qmm_fwd_dec_kernel"
    assert "rows of any length" in _plan(N, 1, 50257, 768, 0, "F16", 4, 1)["kernel"]


def test_plan_query_rejects_bad_arguments(N):
    import ctypes
    lib = N.load()
    assert lib.gptq_hip_qmatmul_plan_query(4, 64, 64, 0, N.F16, N.F16, 4, 0, 1, None) == N.EINVAL
    plan = N.QmatmulPlan()
    assert lib.gptq_hip_qmatmul_plan_query(4, 64, 64, 0, N.F16, N.F16, 5, 0, 1, ctypes.byref(plan)) == N.EINVAL
    assert lib.gptq_hip_qmatmul_plan_query(4, 64, 64, 0, 7, N.F16, 4, 0, 1, ctypes.byref(plan)) == N.EDTYPE
