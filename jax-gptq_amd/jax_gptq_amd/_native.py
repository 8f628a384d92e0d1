"""ctypes binding of libgptq_hip.so (the C ABI declared in include/gptq_hip.h).

There is no CPU fallback: importing the compute entry points without the built
library raises, so that a missing HIP extension is never silently papered over.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# GPTQ_HIP_LIBRARY selects another build of the same ABI (e.g. an instrumented one)
LIB_PATH = os.environ.get("GPTQ_HIP_LIBRARY") or os.path.join(HERE, "libgptq_hip.so")

F32, F16, BF16, F64 = 0, 1, 2, 3
OK, EINVAL, EDTYPE, EWORKSPACE, ELAUNCH, ETOOBIG = 0, 1, 2, 3, 4, 5
QMATMUL_STATIC_BYTES = 32 << 20

_vp, _i64, _i32, _f32, _f64, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float,
                                   ctypes.c_double, ctypes.c_size_t)

# name -> (restype, argtypes); mirrors include/gptq_hip.h one to one
SIGNATURES = {
    "gptq_hip_abi_version": (_i32, []),
    "gptq_hip_error_string": (ctypes.c_char_p, [_i32]),
    "gptq_hip_fill_zero": (_i32, [_vp, _vp, _sz]),
    "gptq_hip_copy": (_i32, [_vp, _vp, _vp, _sz]),
    "gptq_hip_to_f32": (_i32, [_vp, _vp, _i32, _i64, _vp]),
    "gptq_hip_read_probe": (_i32, [_vp, _vp, _sz, _i32, _vp]),
    "gptq_hip_col_params_workspace_bytes": (_sz, [_i64, _i64]),
    "gptq_hip_col_params": (_i32, [_vp, _vp, _i32, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _sz]),
    "gptq_hip_hessian_accumulate_workspace_bytes": (_sz, [_i64, _i32]),
    "gptq_hip_hessian_accumulate": (_i32, [_vp, _vp, _vp, _i32, _i32, _i64, _vp, _i32, _vp, _sz]),
    "gptq_hip_hessian_accumulate_split16_workspace_bytes": (_sz, [_i64, _i64]),
    "gptq_hip_hessian_accumulate_split16": (_i32, [_vp, _vp, _vp, _i32, _i64, _vp, _vp, _sz]),
    "gptq_hip_hessian_finalize": (_i32, [_vp, _vp, _i32, _i64, _f64]),
    "gptq_hip_damp_invert_workspace_bytes": (_sz, [_i64, _i32]),
    "gptq_hip_damp_invert": (_i32, [_vp, _vp, _i32, _vp, _i64, _i64, _i64, _f64, _i32, _vp, _vp, _vp,
                                    _vp, _sz]),
    "gptq_hip_zero_dead_rows": (_i32, [_vp, _vp, _i32, _i64, _vp, _i64, _i64]),
    "gptq_hip_solve_workspace_bytes": (_sz, [_i64, _i64, _i32]),
    "gptq_hip_solve": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _i32, _i32, _vp, _i32, _vp, _vp, _sz]),
    "gptq_hip_process_block": (_i32, [_vp, _vp, _i64, _vp, _i64, _i32, _vp, _vp, _i32, _vp, _i32, _vp, _vp]),
    "gptq_hip_lazy_update": (_i32, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _i64]),
    "gptq_hip_gather_rows": (_i32, [_vp, _vp, _vp, _i32, _i64, _i64, _vp]),
    "gptq_hip_gather_sym": (_i32, [_vp, _vp, _vp, _i32, _i64, _vp]),
    "gptq_hip_pack_int4": (_i32, [_vp, _vp, _i32, _i64, _i64, _i64, _vp]),
    "gptq_hip_unpack_int4": (_i32, [_vp, _vp, _i64, _i64, _i64, _vp]),
    "gptq_hip_quantize_pack": (_i32, [_vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp]),
    "gptq_hip_dequant": (_i32, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _i32, _vp]),
    "gptq_hip_qmatmul_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32]),
    "gptq_hip_qmatmul_workspace_bytes_x": (_sz, [_i64, _i64, _i64, _i32, _i32]),
    "gptq_hip_qmatmul": (_i32, [_vp, _vp, _i32, _i64, _vp, _i64, _i64, _vp, _vp, _i32, _i32, _vp, _vp, _sz]),
    "gptq_hip_quantize_pack_bits": (_i32, [_vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _i32, _vp]),
    "gptq_hip_dequant_bits": (_i32, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _i32, _i32, _vp]),
    "gptq_hip_qmatmul_bits_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32, _i32, _i32]),
    "gptq_hip_qmatmul_bits": (_i32, [_vp, _vp, _i32, _i64, _vp, _i64, _i64, _vp, _vp, _i32, _i32, _i32, _vp, _vp,
                                     _sz]),
    "gptq_hip_solve_grouped_workspace_bytes": (_sz, [_i64, _i64, _i32, _i32]),
    "gptq_hip_solve_grouped": (_i32, [_vp, _vp, _i64, _i64, _vp, _i32, _i32, _i32, _vp, _i32, _vp, _vp, _vp, _vp, _sz]),
    "gptq_hip_quantize_pack_grouped": (_i32, [_vp, _vp, _i32, _i64, _i64, _vp, _vp, _i64, _i32, _vp]),
    "gptq_hip_dequant_grouped": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp, _i32, _i64, _i32, _vp]),
    "gptq_hip_qmatmul_grouped": (_i32, [_vp, _vp, _i32, _i64, _vp, _i64, _i64, _vp, _vp, _i32, _i64, _i32, _i32, _vp,
                                        _vp, _sz]),
    "gptq_hip_qmatmul_static": (_i32, [_vp, _vp, _i32, _i64, _vp, _i64, _i64, _vp, _vp, _i32, _i32, _vp]),
    "gptq_hip_qmatmul_plan_query": (_i32, [_i64, _i64, _i64, _i32, _i32, _i32, _i32, _i64, _i32, _vp]),
    "gptq_hip_qmatmul_kernel_name": (ctypes.c_char_p, [_i32]),
}


class QmatmulPlan(ctypes.Structure):
    """gptq_hip_qmatmul_plan of include/gptq_hip.h."""
    _fields_ = [("kernel", ctypes.c_int), ("kernel_rest", ctypes.c_int), ("splits", ctypes.c_int),
                ("fp32_rows", ctypes.c_int), ("workgroups", ctypes.c_int64)]


def qmatmul_plan(M, R, C, transpose_b=0, x_dtype=F16, zs_dtype=F16, bits=4, group_size=0, aligned=1):
    """Which kernel(s) the packed matmul runs for these arguments (host only): a dict with the kernels' names,
    the splits of the contraction, the first kernel's workgroups and how fp32 rows travel."""
    lib = load()
    plan = QmatmulPlan()
    check(lib.gptq_hip_qmatmul_plan_query(M, R, C, transpose_b, x_dtype, zs_dtype, bits, group_size, aligned,
                                          ctypes.byref(plan)), "qmatmul_plan_query")
    return {"kernel_id": plan.kernel, "kernel": lib.gptq_hip_qmatmul_kernel_name(plan.kernel).decode(),
            "rest": lib.gptq_hip_qmatmul_kernel_name(plan.kernel_rest).decode() if plan.kernel_rest else None,
            "rest_id": plan.kernel_rest, "splits": plan.splits, "workgroups": plan.workgroups,
            "fp32_rows": plan.fp32_rows}

_lib = None


def load():
    """Load the shared library (once) and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python jax-gptq_amd/build.py` "
            "(hipcc, gfx950). There is no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.gptq_hip_abi_version() != 1:
        raise ImportError("libgptq_hip.so has an unexpected ABI version")
    _lib = lib
    return lib


def check(code, what):
    """Map a status code to the exception type the reference raises in that situation."""
    if code == OK:
        return
    msg = f"{what}: {load().gptq_hip_error_string(code).decode()}"
    if code == EINVAL:
        raise ValueError(msg)
    if code == EDTYPE:
        raise TypeError(msg)
    raise RuntimeError(msg)
