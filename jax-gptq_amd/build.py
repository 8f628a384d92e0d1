"""Builds libgptq_hip.so (gfx950 only) next to the Python package.

    python jax-gptq_amd/build.py [--force]

hipcc cross-compiles without a GPU; the .so is kept in-tree (git-ignored).
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "jax_gptq_amd")
LIB = os.path.join(OUT_DIR, "libgptq_hip.so")
SOURCES = ["api.hip", "codec.hip", "gemm_f32.hip", "gemm_f64.hip", "hessian.hip", "cholinv.hip", "solve.hip",
           "qmatmul.hip", "qmatmul_mid.hip", "qmatmul_reg.hip", "qmatmul_reg_bwd.hip", "qmatmul_wide.hip"]
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-result"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def needs_build():
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)]
    deps.append(os.path.join(HERE, "..", "include", "gptq_hip.h"))
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True):
    if not force and not needs_build():
        return LIB
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = _hipcc()
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    failed = False
    for src, p in procs:
        out = p.communicate()[0].decode()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"[build] {src} FAILED\n{out}\n")
        elif verbose and out.strip():
            sys.stderr.write(f"[build] {src}:\n{out}\n")
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "-shared", "--offload-arch=gfx950", "-fPIC", *objs, "-o", LIB]
    subprocess.check_call(cmd)
    if verbose:
        print(f"[build] wrote {LIB}")
    return LIB


JAX_SHIM = os.path.join(OUT_DIR, "libgptq_hip_jax.so")
JAX_SHIM_ERROR = None       # compiler log of a failed shim build


def jax_ffi_include_dir():
    """Directory of the XLA FFI headers (xla/ffi/api/ffi.h) that ships inside jaxlib, or None where JAX
    or its FFI module is absent."""
    try:
        import jax.ffi
        inc = jax.ffi.include_dir()
    except Exception:
        return None
    return inc if os.path.exists(os.path.join(inc, "xla", "ffi", "api", "ffi.h")) else None


def build_jax_ffi(verbose=True):
    """Compile csrc/jax_ffi.cc (XLA FFI handlers over the C ABI) into libgptq_hip_jax.so, linked against
    libgptq_hip.so.  Returns the path, or None where the XLA FFI headers are not installed: the shim is
    optional, the ctypes binding is the one that is always built."""
    inc = jax_ffi_include_dir()
    if inc is None:
        if verbose:
            print("[build] jax.ffi.include_dir() does not resolve: the XLA FFI shim is not built")
        return None
    build()
    cmd = [_hipcc(), "-O2", "-fPIC", "-std=c++17", "-shared", "-x", "hip", "--offload-arch=gfx950",
           "-I", inc, os.path.join(CSRC, "jax_ffi.cc"), "-o", JAX_SHIM,
           "-L", OUT_DIR, "-l:libgptq_hip.so", "-Wl,-rpath,$ORIGIN"]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if p.returncode != 0:
        # the shim is optional and has never been compiled against a real jaxlib: a failure here must
        # not take the mandatory library down with it
        global JAX_SHIM_ERROR
        JAX_SHIM_ERROR = p.stdout.decode(errors="replace")
        sys.stderr.write("[build] the XLA FFI shim did not compile (the ctypes library is unaffected):\n"
                         + JAX_SHIM_ERROR + "\n")
        if os.path.exists(JAX_SHIM):
            os.remove(JAX_SHIM)
        return None
    if verbose:
        print(f"[build] wrote {JAX_SHIM}")
    return JAX_SHIM


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    if "--jax" in sys.argv:
        build_jax_ffi()
