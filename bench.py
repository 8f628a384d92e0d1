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
  cpu_baseline   the NumPy/SciPy oracle timed on this host on a bounded sample,
  phases_ms      per-phase GPU time of one step,
  fp16_calibration  the same layer with the calibration rows stored in fp16,
  fp32_rows_split_fp16  the fp32 rows multiplied as pairs of fp16 numbers (opt-in path),
  qmatmul        packed-int4 matmul at M = 1, 16, 128 against the HBM roofline
                 (weights rotated over > 512 MB of copies so that they come from HBM).
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
    W32 = W.to(torch.float32)
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
    return packed


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
    # decode matmuls of that size run the streaming kernel)
    for (K, N) in ((4096, 11008), (11008, 4096), (7168, 28672)):
        copies = 24 if K * N < (1 << 27) else 6
        iws = [torch.randint(0, 256, (K // 2, N), generator=g, device="cuda", dtype=torch.uint8)
               for _ in range(copies)]
        scale = (0.001 + 0.009 * torch.rand(N, generator=g, device="cuda")).to(torch.float16)
        zero = torch.randint(0, 16, (N,), generator=g, device="cuda").to(torch.float16)
        # forward at the decode / small-batch sizes, and the transposed (VJP) product at 2048 rows
        cases = [(1, 0, "float16"), (16, 0, "float16"), (128, 0, "float16"), (2048, 0, "float16"),
                 (2048, 1, "float16")]
        if K == K_IN:
            cases += [(1, 0, "bfloat16"), (16, 0, "bfloat16"), (2048, 1, "bfloat16")]
        if K * N >= (1 << 27):
            cases = [(1, 0, "float16"), (16, 0, "float16")]
        for (M, tr, xdt) in cases:
            tdt = getattr(torch, xdt)
            xcode = _native.F16 if xdt == "float16" else _native.BF16
            x = torch.randn((M, N if tr else K), generator=g, device="cuda").to(tdt)
            y = torch.empty((M, K if tr else N), dtype=tdt, device="cuda")
            ws = torch.zeros(max(lib.gptq_hip_qmatmul_workspace_bytes(M, K // 2, N, tr), 256),
                             dtype=torch.uint8, device="cuda")

            def call(i):
                rc = lib.gptq_hip_qmatmul(st, x.data_ptr(), xcode, M, iws[i % copies].data_ptr(),
                                          K // 2, N, zero.data_ptr(), scale.data_ptr(), _native.F16, tr,
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
            nbytes = K * N // 2 + 2 * N * 2 + M * K * 2 + M * N * 2
            out.append({"M": M, "K": K, "N": N, "transpose_b": tr, "x_dtype": xdt, "us": round(us, 2),
                        "us_cache_resident": round(us_cached, 2),
                        "algorithmic_bytes": nbytes,
                        "GBps": round(nbytes / us * 1e-3, 1),
                        "hbm_frac": round(nbytes / us * 1e-3 / HBM_PEAK_GBS, 4),
                        "TFLOPs": round(2.0 * M * K * N / us * 1e-6, 2)})
    return out


def cpu_baseline(sample_batches=16):
    """The oracle (NumPy/SciPy restatement of the reference) timed on this host's cores on a
    bounded sample of the same workload: the Hessian over `sample_batches` of the 128
    batches (scaled linearly), then the complete factorisation, column loop and packing."""
    import numpy as np
    from oracle import gptq_oracle as O
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    rng = np.random.default_rng(0)
    W = (0.02 * rng.standard_normal((K_IN, N_OUT))).astype(np.float16)
    xs = [rng.standard_normal((ROWS, K_IN), dtype=np.float32) for _ in range(sample_batches)]
    t0 = time.perf_counter()
    H = O.accumulate_H(xs)
    t_h = (time.perf_counter() - t0) * (N_BATCH / sample_batches)
    t0 = time.perf_counter()
    Q, params = O.gptq(W, None, _H=H)
    packed = O.pack_matrix(Q, params)
    t_rest = time.perf_counter() - t0
    assert packed.int_weight.shape == (K_IN // 2, N_OUT)
    return {"value": round(t_h + t_rest, 2), "unit": "s/layer", "cores": int(threads), "kind": "port",
            "sample": f"oracle (NumPy/SciPy): Hessian over {sample_batches} of {N_BATCH} batches scaled "
                      f"x{N_BATCH // sample_batches} ({t_h:.1f} s extrapolated) + full Cholesky-of-inverse, "
                      f"column loop and packing of the 4096x11008 layer ({t_rest:.1f} s measured)",
            "hessian_s_extrapolated": round(t_h, 2), "rest_s": round(t_rest, 2)}


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
    ap.add_argument("--section", default="all", choices=["all", "hessian", "qmatmul", "copy"],
                    help="profiling aid: run only one part (hessian: X^T X over the 128 batches; "
                         "qmatmul: the int4 matmul loop; copy: a plain 1 GiB device copy used to "
                         "calibrate the FETCH_SIZE / WRITE_SIZE counters)")
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
        print(json.dumps({"section": "qmatmul", "qmatmul": bench_qmatmul()}))
        return

    W, xs = make_inputs(K_IN, N_OUT, N_BATCH, ROWS, getattr(torch, args.x_dtype))
    torch.cuda.synchronize()
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
                # bytes per launch beyond L2 from rocprofv3 FETCH_SIZE + WRITE_SIZE (scaled by what the
                # counters read for a 1 GiB copy: x2.000 / x1.000), summary kept under profiles/
                "traffic": 1.74e10 if wide else 1.06e10,
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
        ref_packed = one_layer(G, W, xs)
        got_packed = one_layer(G, W, xs, split_fp16=True)
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
                                      "frac": m1["hbm_frac"], "traffic": 2.32e7}
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
