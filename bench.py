"""Benchmark of the GEMM hot path on one MI355X.

A "step" is one launch of ttamd_batched_matmul over the workload that the headline metric is quoted on:
fp32 C[4096,4096] = A[4096,4096] . B[4096,4096], operands uniform(-1,1) from the reference's seeded generator,
resident in HBM before the timed region.  Prints ONE JSON line (see README / DESIGN for the fields).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f32": 157.3, "f64": 78.6}  # MI355X dense matrix peaks

# Bytes moved between the L2s and the memory fabric per launch of the default workload, from the rocprofv3
# FETCH_SIZE / WRITE_SIZE passes summarised in profiles/gemm_4096_f32_f64_mfma.txt (scaled by the same counters'
# reading for a copy kernel of known size: x2.000 for reads, x1.000 for writes).  Only valid for that exact
# kernel and size; reported as null otherwise.  Algorithmic bytes are 3 * 4096^2 * 4 = 201.3e6.
MEASURED_TRAFFIC = {("mfma_f32_128x128_akc4_bmc4", 4096): (365531.4 * 2.0 + 65536.0) * 1024.0}


def gpu_gemm_timing(tt, np, dtype, n, steps, warmup):
    """Returns (wall ms/step, event-timed average kernel ms, variant name, C as numpy)."""
    from oracle import tt_oracle as oracle  # input generation only (the reference's RNG restated on the host)

    lib = tt._capi.lib
    A = oracle.Generator(0).uniform_real(-1, 1, (n, n), dtype)
    B = oracle.Generator(1).uniform_real(-1, 1, (n, n), dtype)
    tA, tB = tt.Tensor.from_numpy(A), tt.Tensor.from_numpy(B)
    out = tt.Tensor.empty((1, n, n), tA.dtype)
    be = tt.get_backend(tt.kAMD)
    lv, rv = tA.unsqueeze(0).view3(), tB.unsqueeze(0).view3()
    variant = be.batched_matmul_variant(tA.unsqueeze(0), tB.unsqueeze(0))

    def step():
        st = lib.ttamd_batched_matmul(0, tA.dtype, 1, n, n, n, C.byref(lv), C.byref(rv), C.c_void_p(out.storage.ptr),
                                      None, None)
        if st != 0:
            raise RuntimeError(tt._capi.last_error())

    for _ in range(warmup):
        step()
    be.synchronize(0)
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.ttamd_event_create(0, C.byref(e0))
    lib.ttamd_event_create(0, C.byref(e1))
    t0 = time.perf_counter()
    lib.ttamd_event_record(e0, None)  # same (default) stream as the kernels
    for _ in range(steps):
        step()
    lib.ttamd_event_record(e1, None)
    be.synchronize(0)
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = C.c_float()
    lib.ttamd_event_elapsed_ms(e0, e1, C.byref(ms))
    lib.ttamd_event_destroy(e0)
    lib.ttamd_event_destroy(e1)
    return wall_ms, ms.value / steps, variant, (A, B, out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--n", type=int, default=4096, help="square size (the metric is quoted at 4096)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first run one dense 256 MiB copy kernel (known HBM traffic) to scale profiler byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np

    import tinytensor_amd as tt

    if args.copy_calibration:
        # 64 Mi f32 elements: reads 256 MiB and writes 256 MiB, both exactly known.
        src = tt.Tensor.empty((64 * 1024 * 1024,), tt._capi.F32)
        tt.get_backend(tt.kAMD).identity(tt.Tensor(src.storage, src.dtype, (8192, 8192), (8192, 1), 0))
        tt.get_backend(tt.kAMD).synchronize(0)

    n = args.n
    flop = 2.0 * n * n * n
    wall_ms, kern_ms, variant, (A, B, out) = gpu_gemm_timing(tt, np, np.float32, n, args.steps, args.warmup)
    gflops = flop / (wall_ms * 1e-3) / 1e9
    achieved_tflops = flop / (kern_ms * 1e-3) / 1e12

    # spot parity inside the bench run: one band of rows against the oracle
    from oracle import tt_oracle as oracle

    Cg = out.to_numpy()[0]
    rows = slice(0, 64)
    want = oracle.matmul(A[rows], B, "fast")
    scale = np.abs(A[rows]).astype(np.float64) @ np.abs(B).astype(np.float64)
    parity = float(np.max(np.abs(Cg[rows].astype(np.float64) - want.astype(np.float64)) / scale))

    wall64, kern64, variant64, _ = gpu_gemm_timing(tt, np, np.float64, n, max(args.steps // 2, 1), args.warmup)
    f64_tflops = flop / (kern64 * 1e-3) / 1e12

    cpu = None
    if not args.no_cpu:
        # Bounded sample of the same workload on one host core: the full product at n <= 4096 (~10 s),
        # timed once; the tiled restatement of the reference CPU kernel, fma flavour.
        t0 = time.perf_counter()
        oracle.matmul_kernel(A, B, "fast")
        dt = time.perf_counter() - t0
        cpu = {"value": round(flop / dt / 1e9, 3), "unit": "GFLOP/s", "cores": 1, "kind": "port",
               "sample": f"one full f32 {n}x{n}x{n} product, {dt:.1f} s, gcc -O3 x86-64 128-bit fma, host has "
                         f"{os.cpu_count()} logical cores"}

    line = {
        "metric": "fp32 GEMM GFLOP/s at 4096^3 on 1 MI355X",
        "value": round(gflops, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic: uniform(-1,1) from the reference's seeded generator (seeds 0 and 1)",
        "config": {"workload": f"configs[2]: fp32 {n}x{n} @ {n}x{n}, dense row-major", "kernel": variant,
                   "parity_k_scaled_err_rows0_63": parity},
        "roofline": {"bound": "mfma", "achieved": round(achieved_tflops, 2), "peak": PEAK_TFLOPS["f32"],
                     "unit": "TFLOP/s", "frac": round(achieved_tflops / PEAK_TFLOPS["f32"], 4),
                     "traffic": MEASURED_TRAFFIC.get((variant, n)), "algorithmic_bytes": 3.0 * n * n * 4,
                     "kernel_ms": round(kern_ms, 4)},
        "cpu_baseline": cpu,
        "fp64": {"kernel": variant64, "kernel_ms": round(kern64, 4), "achieved": round(f64_tflops, 2),
                 "peak": PEAK_TFLOPS["f64"], "unit": "TFLOP/s", "frac": round(f64_tflops / PEAK_TFLOPS["f64"], 4)},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
