#!/usr/bin/env python3
"""Benchmark of the GPTQ hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one complete per-layer solve of the Llama-7B up-projection shape:
W [4096, 11008] fp16 ~ N(0, 0.02), calibration 128 batches x [2048, 4096] fp32 ~ N(0, 1)
(262144 tokens), 4-bit per-output-channel asymmetric min-max, damping 1 %, block 128.
Inputs are resident in HBM when the timed region starts.  The step covers column
parameters, Hessian accumulation, damping + Cholesky factor of the inverse, the blocked
column loop and nibble packing.

Prints ONE JSON line.  Besides the contract keys it carries
  roofline       the dominant kernel (X^T X, fp32 MFMA) against the fp32 matrix peak,
  cpu_baseline   the NumPy/SciPy oracle timed on this host's cores on the very layer the GPU timed,
  parity         the GPU result against that oracle run: scale / zero, codes, reconstruction error,
  hessian_streamed  X^T X as the reference calls it: one call per batch of 2048 rows (gptq.py:97-98),
  phases_ms      per-phase GPU time of one step,
  fp16_calibration  the same layer with the calibration rows stored in fp16,
  fp32_rows_split_fp16  the fp32 rows multiplied as pairs of fp16 numbers (opt-in path),
  qmatmul        packed-int4 matmul at M = 1, 16, 128, 2048 against the HBM and 16-bit MFMA rooflines
                 (weights rotated over > 512 MB of copies so that they come from HBM), 8-bit codes and
                 a vocabulary-sized N included,
  hbm_read_ceiling  a kernel that only reads, at the packed sizes of the matmul cases.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "jax-gptq_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

K_IN, N_OUT = 4096, 11008
N_BATCH, ROWS = 128, 2048
FP32_MFMA_PEAK_TFLOPS = 157.3
MFMA16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0


def _events(n):
    import torch
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def make_inputs(k_in, n_out, n_batch, rows, x_dtype):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    W = (0.02 * torch.randn((k_in, n_out), generator=g, device="cuda")).to(torch.float16)
    xs = [torch.randn((rows, k_in), generator=g, device="cuda", dtype=torch.float32).to(x_dtype)
          for _ in range(n_batch)]
    return W, xs


def one_layer(G, W, xs, timers=None, split_fp16=False):
    """The hot path, phase by phase (same calls as jax_gptq_amd.gptq.gptq + pack_matrix)."""
    import torch
    ev = _events(6) if timers is not None else None

    def mark(i):
        if ev is not None:
            ev[i].record()

    mark(0)
    W32 = G._to_f32_copy(W)
    params = G.get_col_quantize_params(W32)
    mark(1)
    H = G.accumulate_H(xs, split_fp16=split_fp16)
    mark(2)
    W32, L, any_nan = G._damp_and_invert(W32, H, 0.01)     # reads one status word (host sync)
    mark(3)
    if any_nan:
        raise ValueError("NaN when computing Hinv")
    Q, _ = G._solve(W32, L, params, 128, W.dtype)
    mark(4)
    packed = G.pack_matrix(Q, params)
    mark(5)
    if timers is not None:
        torch.cuda.synchronize()
        names = ["col_params", "hessian", "damp_invert", "column_loop", "pack"]
        for i, nm in enumerate(names):
            timers.setdefault(nm, []).append(ev[i].elapsed_time(ev[i + 1]))
    return packed, params


def _profile_number(fname, pattern):
    """A figure quoted from a committed rocprofv3 summary under profiles/ (None if the file or the
    line is missing): the byte counters cannot be read from inside the timed process."""
    import re
    try:
        with open(os.path.join(ROOT, "profiles", fname)) as f:
            m = re.search(pattern, f.read())
        return float(m.group(1)) if m else None
    except OSError:
        return None


def hessian_traffic_bytes(wide):
    """FETCH_SIZE + WRITE_SIZE per launch of the Hessian kernel, from its counter summary."""
    fname = ("syrk32d_kernel_K4096_n262144_fp32_counters.md" if wide
             else "syrk16d_kernel_K4096_n262144_fp16_counters.md")
    f = _profile_number(fname, r"FETCH_SIZE[^\n]*?=\s*([0-9.]+)\s*GiB per launch")
    w = _profile_number(fname, r"WRITE_SIZE[^\n]*?=\s*([0-9.]+)\s*GiB per launch")
    return None if f is None or w is None else round((f + w) * 2 ** 30)


def qmatmul_traffic_bytes(case="M=1, K=4096, N=11008, float16"):
    """FETCH + WRITE MB per launch of one matmul case, from the matmul kernels' summary table."""
    import re
    pat = r"\|\s*" + re.escape(case) + r"\s*\|[^\n]*\|\s*([0-9.]+)\s*\|\s*([0-9.]+)\s*\|\s*\n"
    try:
        with open(os.path.join(ROOT, "profiles", "qmm_kernels_llama7b_opt30b_shapes.md")) as f:
            m = re.search(pat, f.read())
        return None if not m else round((float(m.group(1)) + float(m.group(2))) * 1e6)
    except OSError:
        return None


def bench_hessian_streamed(G, xs, reps=2):
    """The reference's calling pattern (gptq.py:97-98): one entry-point call per calibration batch,
    H updated in place, one finalisation at the end.  Also timed through `_accumulate_H_step`, whose
    state is completed to a full symmetric matrix when the caller looks at it (once per chain here)."""
    import torch
    from jax_gptq_amd import _native
    lib = _native.load()
    K = xs[0].shape[1]
    n = sum(x.shape[0] for x in xs)

    def streamed():
        H = G._zeros((K, K), torch.float32)
        for x in xs:
            G._hessian_accumulate(H, [x])
        _native.check(lib.gptq_hip_hessian_finalize(G._stream(), G._ptr(H), _native.F32, K, float(n)), "finalize")
        return H

    def stepped():
        H = G._zeros((K, K), torch.float32)
        m = G._zeros((K,), torch.float32)
        cnt = 0
        for x in xs:
            H, m, cnt = G._accumulate_H_step(H, m, cnt, x)
        return H / cnt + torch.outer(m, m)

    out = {}
    ref = G.accumulate_H(xs)
    for name, fn in (("one_call_per_batch", streamed), ("accumulate_H_step_chain", stepped)):
        H = fn()
        torch.cuda.synchronize()
        e0, e1 = _events(2)
        e0.record()
        for _ in range(reps):
            H = fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        tiles = (K + 255) // 256
        alg = 2.0 * n * K * K / (ms * 1e-3) * 1e-12
        out[name] = {"ms_total": round(ms, 3), "us_per_call": round(ms * 1e3 / len(xs), 1),
                     "algorithmic_tflops": round(alg, 2),
                     "executed_frac_of_fp32_mfma_peak": round(alg * (tiles + 1) / (2 * tiles) / FP32_MFMA_PEAK_TFLOPS, 4),
                     "max_abs_diff_vs_one_launch": float((H - ref).abs().max())}
    return out


def bench_qmatmul(reps=240):
    """Packed-int4 matmul against the HBM roofline, called through the C ABI with
    preallocated buffers (the Python operator adds ~10 us of host time per call, which
    would hide a ~10 us kernel).  The packed weight (22.5 MB) would fit the 256 MB Infinity
    Cache, so the timed loop rotates over 24 independent copies (540 MB)."""
    import ctypes
    import torch
    from jax_gptq_amd import _native
    lib = _native.load()
    out = []
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # the two Llama-7B MLP shapes of the benchmark layer, then the OPT-30B fc1 shape (103 MB packed:
    # decode matmuls of that size run the decode kernel's ring-loop form)
    # (K, N, bits): the last two are what the register-operand kernels serve: 8-bit codes (one per byte)
    # and a vocabulary-sized N that is not a multiple of 16 channels
    for (K, N, bits) in ((4096, 11008, 4), (11008, 4096, 4), (7168, 28672, 4), (4096, 11008, 8), (768, 50257, 4)):
        R = K // 2 if bits == 4 else K
        copies = max(6, min(24, (560 << 20) // (R * N)))
        iws = [torch.randint(0, 256, (R, N), generator=g, device="cuda", dtype=torch.uint8)
               for _ in range(copies)]
        scale = (0.001 + 0.009 * torch.rand(N, generator=g, device="cuda")).to(torch.float16)
        zero = torch.randint(0, 16, (N,), generator=g, device="cuda").to(torch.float16)
        # forward at the decode / small-batch sizes, and the transposed (VJP) product at 2048 rows
        cases = [(1, 0, "float16"), (16, 0, "float16"), (128, 0, "float16"), (2048, 0, "float16"),
                 (2048, 1, "float16")]
        if bits == 4 and K * N == K_IN * N_OUT:
            cases[2:2] = [(32, 0, "float16"), (64, 0, "float16")]
        if K == K_IN and bits == 4:
            cases += [(1, 0, "bfloat16"), (16, 0, "bfloat16"), (2048, 1, "bfloat16")]
            # fp32 rows in and out (what a JAX caller of the reference passes by default): rounded to fp16
            # precision on the way in, as the reference's dot rounds them to TF32
            cases += [(1, 0, "float32"), (128, 0, "float32")]
        if K == N_OUT and bits == 4:
            cases += [(2048, 1, "bfloat16")]
        if K * N >= (1 << 27):
            cases = [(1, 0, "float16"), (16, 0, "float16"), (2048, 0, "float16"), (2048, 1, "float16")]
        if N % 16:
            cases = [(1, 0, "float16"), (16, 0, "float16"), (512, 0, "float16"), (512, 1, "float16")]
        for (M, tr, xdt) in cases:
            tdt = getattr(torch, xdt)
            xcode = {"float16": _native.F16, "bfloat16": _native.BF16, "float32": _native.F32}[xdt]
            esz = 4 if xdt == "float32" else 2
            x = torch.randn((M, N if tr else K), generator=g, device="cuda").to(tdt)
            y = torch.empty((M, K if tr else N), dtype=tdt, device="cuda")
            ws = torch.zeros(max(lib.gptq_hip_qmatmul_bits_workspace_bytes(M, R, N, tr, xcode, bits), 256),
                             dtype=torch.uint8, device="cuda")

            def call(i):
                rc = lib.gptq_hip_qmatmul_bits(st, x.data_ptr(), xcode, M, iws[i % copies].data_ptr(),
                                               R, N, zero.data_ptr(), scale.data_ptr(), _native.F16, bits, tr,
                                               y.data_ptr(), ws.data_ptr(), ws.numel())
                assert rc == 0, rc

            for i in range(copies):
                call(i)
            torch.cuda.synchronize()
            e0, e1 = _events(2)
            e0.record()
            for i in range(reps):
                call(i)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / reps
            # the same call on ONE weight copy: served by the 256 MB Infinity Cache, not by HBM
            e0.record()
            for i in range(reps):
                call(0)
            e1.record()
            torch.cuda.synchronize()
            us_cached = e0.elapsed_time(e1) * 1e3 / reps
            nbytes = R * N + 2 * N * 2 + M * K * esz + M * N * esz
            plan = _native.qmatmul_plan(M, R, N, transpose_b=tr, x_dtype=xcode, zs_dtype=_native.F16, bits=bits)
            out.append({"M": M, "K": K, "N": N, "bits": bits, "transpose_b": tr, "x_dtype": xdt, "us": round(us, 2),
                        "kernel": plan["kernel"] + (" + " + plan["rest"] if plan["rest"] else ""),
                        "splits": plan["splits"],
                        "us_cache_resident": round(us_cached, 2),
                        "algorithmic_bytes": nbytes,
                        "GBps": round(nbytes / us * 1e-3, 1),
                        "hbm_frac": round(nbytes / us * 1e-3 / HBM_PEAK_GBS, 4),
                        "TFLOPs": round(2.0 * M * K * N / us * 1e-6, 2),
                        "mfma16_frac": round(2.0 * M * K * N / us * 1e-6 / MFMA16_PEAK_TFLOPS, 4)})
        del iws
    return out


def bench_read_ceiling(reps=100):
    """What a kernel that only reads gets from the memory system at the packed sizes of the matmul cases
    (gptq_hip_read_probe: linear 16-byte loads, eight in flight per thread; buffers rotated like the weights):
    the practical ceiling of any HBM-bound kernel launched on its own at that size."""
    import ctypes
    import torch
    from jax_gptq_amd import _native
    lib = _native.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    out = []
    for nbytes in (4096 * 11008 // 2, 4096 * 11008, 7168 * 28672 // 2, 1 << 30):
        copies = max(2, min(24, (1200 << 20) // nbytes))
        bufs = [torch.full((nbytes,), i + 1, dtype=torch.uint8, device="cuda") for i in range(copies)]
        best = None
        for wgs in (256, 512, 2048):
            for i in range(copies):
                assert lib.gptq_hip_read_probe(st, bufs[i].data_ptr(), nbytes, wgs, sink.data_ptr()) == 0
            torch.cuda.synchronize()
            e0, e1 = _events(2)
            e0.record()
            for i in range(reps):
                lib.gptq_hip_read_probe(st, bufs[i % copies].data_ptr(), nbytes, wgs, sink.data_ptr())
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / reps
            if best is None or us < best[0]:
                best = (us, wgs)
        out.append({"bytes": nbytes, "us": round(best[0], 2), "workgroups": best[1],
                    "GBps": round(nbytes / best[0] * 1e-3, 1), "hbm_frac": round(nbytes / best[0] * 1e-3 / HBM_PEAK_GBS, 4)})
        del bufs
    return out


def cpu_baseline_and_parity(W, xs, packed_gpu, params_gpu):
    """The oracle (NumPy/SciPy restatement of the reference) on this host's cores, on the very
    W and calibration rows the GPU timed (copied to the host outside every timed region): its time
    is the CPU baseline, its result is what the GPU result is compared with.  Bars of the task:
    scale / zero within 1e-5 relative, >= 99.9 % of the codes equal and the rest off by one, layer
    reconstruction error within 1 % of the oracle's."""
    import numpy as np
    import torch
    from oracle import gptq_oracle as O
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    W_np = W.cpu().numpy()
    xs_np = [x.float().cpu().numpy() for x in xs]
    t0 = time.perf_counter()
    H = O.accumulate_H(xs_np)
    t_h = time.perf_counter() - t0
    t0 = time.perf_counter()
    Q, params = O.gptq(W_np, None, _H=H)
    packed = O.pack_matrix(Q, params)
    t_rest = time.perf_counter() - t0
    base = {"value": round(t_h + t_rest, 2), "unit": "s/layer", "cores": int(threads), "kind": "port",
            "sample": f"oracle (NumPy/SciPy) on the complete layer the GPU timed: Hessian over all {len(xs)} "
                      f"batches ({t_h:.1f} s) + Cholesky-of-inverse, column loop and packing ({t_rest:.1f} s)",
            "hessian_s": round(t_h, 2), "rest_s": round(t_rest, 2)}
    # ---- parity of the GPU result on the same inputs
    gb = packed_gpu.int_weight.cpu().numpy()
    rb = packed.int_weight
    d_lo = (gb & 15).astype(np.int16) - (rb & 15).astype(np.int16)
    d_hi = (gb >> 4).astype(np.int16) - (rb >> 4).astype(np.int16)
    unequal = int((d_lo != 0).sum() + (d_hi != 0).sum())
    sc_g, z_g = params_gpu["scale"].cpu().numpy(), params_gpu["zero"].cpu().numpy()
    # reconstruction error over the first two batches, in double on the device (checker only)
    X = torch.cat([xs[0], xs[1]]).double()
    Wd = W.double()
    sc = torch.from_numpy(np.asarray(params["scale"])).cuda().double()
    zz = torch.from_numpy(np.asarray(params["zero"])).cuda().double()

    def dense(b):
        b = torch.from_numpy(b).cuda()
        c = torch.empty((2 * b.shape[0], b.shape[1]), dtype=torch.float64, device="cuda")
        c[0::2] = (b & 15).double()
        c[1::2] = (b >> 4).double()
        return (c - zz) * sc

    ref = (X @ Wd).norm()
    e_gpu = float((X @ (Wd - dense(gb))).norm() / ref)
    e_cpu = float((X @ (Wd - dense(rb))).norm() / ref)
    parity = {"oracle": "oracle/gptq_oracle.py on the same W and calibration rows",
              "codes_equal_frac": round(1.0 - unequal / (2.0 * rb.size), 7),
              "codes_max_abs_diff": int(max(np.abs(d_lo).max(), np.abs(d_hi).max())),
              "scale_max_rel_diff": float(np.max(np.abs(sc_g - params["scale"]) / np.abs(params["scale"]))),
              "zero_max_abs_diff": float(np.max(np.abs(z_g - params["zero"]))),
              "recon_error_gpu": round(e_gpu, 6), "recon_error_oracle": round(e_cpu, 6),
              "recon_error_rel_diff": round(abs(e_gpu - e_cpu) / e_cpu, 6)}
    parity["within_bars"] = bool(parity["codes_equal_frac"] >= 0.999 and parity["codes_max_abs_diff"] <= 1
                                 and parity["scale_max_rel_diff"] <= 1e-5 and parity["zero_max_abs_diff"] == 0.0
                                 and parity["recon_error_rel_diff"] <= 0.01)
    return base, parity


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--x-dtype", default="float32", choices=["float32", "float16", "bfloat16"])
    ap.add_argument("--split-fp16", action="store_true",
                    help="--section hessian only: fp32 rows as pairs of fp16 numbers (accumulate_H(split_fp16=True))")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-qmatmul", action="store_true", help="skip the int4 matmul section")
    ap.add_argument("--no-streamed", action="store_true",
                    help="skip the one-call-per-batch Hessian section (a kernel trace of the run then holds "
                         "syrk32d_kernel's one-launch-per-layer calls only)")
    ap.add_argument("--section", default="all", choices=["all", "hessian", "streamed", "factor", "solve", "qmatmul", "copy"],
                    help="profiling aid: run only one part (hessian: X^T X over the 128 batches; factor: damping + "
                         "Cholesky factor of the inverse of a K = 4096 Hessian; solve: the blocked column loop of the "
                         "4096 x 11008 layer; qmatmul: the packed matmul loop; copy: a plain 1 GiB device copy used "
                         "to calibrate the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (use --gpus 1)")

    import torch
    import jax_gptq_amd.gptq as G
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    if args.section == "copy":
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")      # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(max(1, args.steps)):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"section": "copy", "bytes_read": src.numel() * 4,
                          "bytes_written": src.numel() * 4, "launches": max(1, args.steps)}))
        return
    if args.section == "qmatmul":
        print(json.dumps({"section": "qmatmul", "qmatmul": bench_qmatmul(), "hbm_read_ceiling": bench_read_ceiling()}))
        return
    if args.section in ("factor", "solve"):
        # a well-conditioned Hessian from 8 batches is enough: the phases below do not depend on its content
        W, xs = make_inputs(K_IN, N_OUT, 8, ROWS, torch.float16)
        H0 = G.accumulate_H(xs)
        params = G.get_col_quantize_params(G._to_f32_copy(W))
        n = max(1, args.steps)
        if args.section == "factor":
            G._damp_invert(None, G._clone(H0), 0.01, fix_dead=False)
            e0, e1 = _events(2)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(n):
                G._damp_invert(None, G._clone(H0), 0.01, fix_dead=False)
            e1.record()
        else:
            L, _, _ = G._damp_invert(None, G._clone(H0), 0.01, fix_dead=False)
            G._solve(G._to_f32_copy(W), L, params, 128, W.dtype)
            e0, e1 = _events(2)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(n):
                G._solve(G._to_f32_copy(W), L, params, 128, W.dtype)
            e1.record()
        torch.cuda.synchronize()
        print(json.dumps({"section": args.section, "ms": round(e0.elapsed_time(e1) / n, 3)}))
        return

    W, xs = make_inputs(K_IN, N_OUT, N_BATCH, ROWS, getattr(torch, args.x_dtype))
    torch.cuda.synchronize()
    if args.section == "streamed":
        # the Hessian as the reference calls it, one call per batch (for a kernel trace of those launches alone)
        print(json.dumps({"section": "streamed", "hessian_streamed": bench_hessian_streamed(G, xs)}))
        return
    if args.section == "hessian":
        G.accumulate_H(xs, split_fp16=args.split_fp16)
        e0, e1 = _events(2)
        e0.record()
        for _ in range(max(1, args.steps)):
            G.accumulate_H(xs, split_fp16=args.split_fp16)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / max(1, args.steps)
        print(json.dumps({"section": "hessian", "ms": round(ms, 3),
                          "algorithmic_tflops": round(2.0 * N_BATCH * ROWS * K_IN * K_IN / ms * 1e-9, 2)}))
        return

    for _ in range(args.warmup):
        one_layer(G, W, xs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_layer(G, W, xs)
    torch.cuda.synchronize()
    sec_per_step = (time.perf_counter() - t0) / args.steps

    # phase breakdown and the live duration of the dominant kernel (events on the stream the
    # kernels are launched on, which is torch's current stream)
    timers = {}
    for _ in range(max(1, args.steps)):
        one_layer(G, W, xs, timers)
    phases = {k: round(sum(v) / len(v), 3) for k, v in timers.items()}
    hess_ms = phases["hessian"]
    # One launch covers all 128 batches; the phase time also contains the (tiny) slice
    # reduction, the zero fill of H and the finalisation, which makes the figure conservative.
    n_tokens = N_BATCH * ROWS
    flop_per_launch = 2.0 * n_tokens * K_IN * K_IN          # the full GEMM the reference executes
    wide = args.x_dtype == "float32"
    # the kernels compute the upper tiles only: 256 x 256 from K = 1024 on, 128 x 128 below
    tile_edge = 128 if K_IN < 1024 else 256
    tiles = (K_IN + tile_edge - 1) // tile_edge
    executed_flop = flop_per_launch * (tiles + 1) / (2 * tiles)
    achieved = flop_per_launch / (hess_ms * 1e-3) * 1e-12
    executed = executed_flop / (hess_ms * 1e-3) * 1e-12
    peak = FP32_MFMA_PEAK_TFLOPS if wide else MFMA16_PEAK_TFLOPS
    roofline = {"kernel": "syrk32d_kernel (fp32 X^T X, fp32 MFMA, upper 256 x 256 tiles)" if wide else
                          f"syrk16d_kernel ({args.x_dtype} X^T X, 16-bit MFMA with fp32 accumulation, upper tiles)",
                "bound": "mfma",
                "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4),
                # bytes per launch beyond L2: rocprofv3 FETCH_SIZE + WRITE_SIZE (scaled by what the
                # counters read for a 1 GiB copy: x2.000 / x1.000), quoted from the summary under profiles/
                "traffic": hessian_traffic_bytes(wide),
                "flop_per_launch": flop_per_launch, "avg_launch_ms": round(hess_ms, 4),
                "launches_per_step": 1,
                "executed_tflops": round(executed, 2),
                "executed_frac": round(executed / peak, 4),
                "note": "achieved counts the algorithmic 2*n*K^2 flop; the kernel computes only the "
                        "upper tiles of the symmetric result (executed_*), which is what MFMA "
                        "utilisation counters see"}

    result = {
        "metric": "GPTQ s/layer @4096x11008", "value": round(sec_per_step, 5), "unit": "s/layer",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec_per_step * 1e3, 3), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32" if wide else "f16/bf16 products, f32 sums", "data": "synthetic",
        "config": {"workload": "llama7b_up_proj W[4096,11008] fp16, 128x[2048,4096] "
                               f"{args.x_dtype} calibration (262144 tokens), 4-bit, damp 0.01, block 128"},
        "roofline": roofline,
        "xtx_tflops": round(achieved, 2),
        "phases_ms": phases,
    }
    if wide and args.section == "all":
        # the same layer with the calibration rows stored in fp16 (as the activations of an fp16
        # model are): products of fp16 numbers are exact in fp32, the Hessian runs on 16-bit MFMA
        xs16 = [x.to(torch.float16) for x in xs]
        one_layer(G, W, xs16)
        t16 = {}
        for _ in range(max(1, args.steps)):
            one_layer(G, W, xs16, t16)
        ph16 = {k: round(sum(v) / len(v), 3) for k, v in t16.items()}
        result["fp16_calibration"] = {"ms_per_layer": round(sum(ph16.values()), 3), "phases_ms": ph16,
                                      "xtx_tflops": round(flop_per_launch / (ph16["hessian"] * 1e-3) * 1e-12, 2)}
        del xs16
        # the fp32 rows again, multiplied as pairs of fp16 numbers on the 16-bit matrix cores (opt-in:
        # accumulate_H(..., split_fp16=True)); codes_equal compares the packed result with the one above
        ref_packed, _ = one_layer(G, W, xs)
        got_packed, _ = one_layer(G, W, xs, split_fp16=True)
        ts = {}
        for _ in range(max(1, args.steps)):
            one_layer(G, W, xs, ts, split_fp16=True)
        phs = {k: round(sum(v) / len(v), 3) for k, v in ts.items()}
        rb, gb = ref_packed.int_weight, got_packed.int_weight
        same = ((rb & 15) == (gb & 15)).sum() + ((rb >> 4) == (gb >> 4)).sum()
        result["fp32_rows_split_fp16"] = {"ms_per_layer": round(sum(phs.values()), 3), "phases_ms": phs,
                                          "xtx_tflops": round(flop_per_launch / (phs["hessian"] * 1e-3) * 1e-12, 2),
                                          "codes_equal": round(float(same) / (2 * rb.numel()), 6)}
    if not args.no_qmatmul:
        qm = bench_qmatmul()
        result["qmatmul"] = qm
        m1 = [r for r in qm if r["M"] == 1 and r["K"] == 4096 and r["x_dtype"] == "float16"][0]
        result["int4_matmul_hbm_gbps"] = m1["GBps"]
        result["roofline_qmatmul"] = {"kernel": "qmatmul M=1 4096x11008", "bound": "hbm",
                                      "achieved": m1["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                      "frac": m1["hbm_frac"], "traffic": qmatmul_traffic_bytes()}
        # the practical ceiling: a kernel that only reads, at the same sizes
        result["hbm_read_ceiling"] = bench_read_ceiling()
    if args.section == "all" and not args.no_streamed:
        result["hessian_streamed"] = bench_hessian_streamed(G, xs)
    if not args.no_cpu:
        packed_gpu, params_gpu = one_layer(G, W, xs)
        torch.cuda.synchronize()
        result["cpu_baseline"], result["parity"] = cpu_baseline_and_parity(W, xs, packed_gpu, params_gpu)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
