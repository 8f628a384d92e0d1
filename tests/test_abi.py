"""CPU checks of the C-ABI library: it loads, exports every symbol the header declares,
and the ctypes table mirrors the header.  No compute entry point is called."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gptq_hip.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(gptq_hip_\w+)\s*\(", src)))


def test_header_declares_entry_points():
    names = _declared()
    for must in ("gptq_hip_hessian_accumulate", "gptq_hip_damp_invert", "gptq_hip_solve",
                 "gptq_hip_pack_int4", "gptq_hip_qmatmul"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from jax_gptq_amd import _native
    lib = _native.load()
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in gptq_hip.h but not exported"
    assert lib.gptq_hip_abi_version() == 1
    assert lib.gptq_hip_error_string(0) == b"ok"


def test_ctypes_table_matches_header():
    from jax_gptq_amd import _native
    assert sorted(_native.SIGNATURES) == _declared()
    # argument counts
    src = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, (_, args) in _native.SIGNATURES.items():
        m = re.search(name + r"\s*\(([^;]*?)\)\s*;", src, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(args), f"{name}: header has {n} parameters, ctypes table {len(args)}"


def test_workspace_queries_are_pure_host_functions():
    from jax_gptq_amd import _native
    lib = _native.load()
    assert lib.gptq_hip_col_params_workspace_bytes(4096, 11008) > 0
    kp = 4096
    assert lib.gptq_hip_damp_invert_workspace_bytes(4096, _native.F32) >= 3 * kp * kp * 4
    assert lib.gptq_hip_damp_invert_workspace_bytes(4096, _native.F64) >= 3 * kp * kp * 8
    assert lib.gptq_hip_damp_invert_workspace_bytes(100, _native.F32) >= 3 * 128 * 128 * 4
    # K = 28672: so many tiles that no row slices are needed; what is left is the two partial-tile slots for each of
    # the 256 workgroups of a short call
    assert lib.gptq_hip_hessian_accumulate_workspace_bytes(28672, _native.F32) == 512 * 256 * 256 * 4
    assert lib.gptq_hip_hessian_accumulate_workspace_bytes(768, _native.F32) > 0
    assert lib.gptq_hip_hessian_accumulate_workspace_bytes(256, _native.F64) == 0
    assert lib.gptq_hip_solve_workspace_bytes(4096, 11008, 128) == 512 * 11008 * 4      # error rows of a 512-row group
    assert lib.gptq_hip_solve_workspace_bytes(4096, 11008, 129) == 0


def test_argument_validation_without_gpu():
    """Entry points reject bad arguments before touching the device."""
    from jax_gptq_amd import _native
    lib = _native.load()
    null = ctypes.c_void_p(0)
    assert lib.gptq_hip_pack_int4(null, null, 1, 1, 3, 1, null) == _native.EINVAL      # odd axis
    assert lib.gptq_hip_pack_int4(null, null, 1, 0, 4, 1, null) == _native.OK          # empty
    assert lib.gptq_hip_solve(null, null, 8, 8, null, null, null, 15, 4, null, 0, null, null, 0) \
        == _native.EINVAL
    assert lib.gptq_hip_qmatmul(null, null, 0, 0, null, 4, 4, null, null, 0, 0, null, null, 0) \
        == _native.OK                                                                   # M == 0
    assert lib.gptq_hip_qmatmul(null, null, 0, 3, null, 4, 4, null, null, 0, 0, null, null, 0) \
        == _native.EINVAL                                                               # null x
    with pytest.raises(ValueError):
        _native.check(_native.EINVAL, "x")
    with pytest.raises(TypeError):
        _native.check(_native.EDTYPE, "x")
    with pytest.raises(RuntimeError):
        _native.check(_native.EWORKSPACE, "x")
