"""Benchmark of the GEMM hot path on one MI355X.

A "step" is one launch of ttamd_batched_matmul over the workload that the headline metric is quoted on:
fp32 C[4096,4096] = A[4096,4096] . B[4096,4096], operands uniform(-1,1) from the reference's seeded generator,
resident in HBM before the timed region.  Prints ONE JSON line: metric / value / unit (GFLOP/s of the whole job),
ms_per_step, dtype, config.workload and the kernel variant, `roofline` (achieved TFLOP/s of the kernel from HIP events
on its stream against the fp32 MFMA peak, HBM traffic per launch) and `cpu_baseline` (the CPU oracle on one core over
a bounded sample of the same workload).
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
WARMUP_SECONDS = 0.25  # minimum untimed GPU work in front of the timed launches

# Bytes moved between the L2s and the memory fabric per launch of the default workload, from the rocprofv3
# FETCH_SIZE / WRITE_SIZE passes summarised in profiles/gemm_4096_f32_f64_mfma.txt (scaled by the same counters'
# reading for a copy kernel of known size: x2.000 for reads, x1.000 for writes).  Only valid for that exact
# kernel and size; reported as null otherwise.  Algorithmic bytes are 3 * 4096^2 * 4 = 201.3e6.
MEASURED_TRAFFIC = {("mfma_f32_256x256_akc4_bmc4", 4096): (196783.0 * 2.0 + 65536.0) * 1024.0}


def gpu_gemm_timing(tt, np, dtype, n, steps, warmup):
    """Returns (wall ms/step, event-timed average kernel ms, variant name, (A, B, C), warm-up launches made)."""
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

    # Untimed warm-up: the requested number of launches and at least WARMUP_SECONDS of GPU work, because the clocks
    # take on the order of 100 ms of load to settle and a short `--warmup` count would charge the ramp to the timed
    # launches.  The number of launches actually made is reported as `warmup_effective`.
    warm, t_end = 0, time.perf_counter() + WARMUP_SECONDS
    while warm < warmup or time.perf_counter() < t_end:
        step()
        warm += 1
        if warm % 8 == 0:
            be.synchronize(0)
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
    return wall_ms, ms.value / steps, variant, (A, B, out), warm


def time_launches(tt, fn, iters, warmup):
    """Average milliseconds per call of fn() (which enqueues GPU work on the default stream), by HIP events."""
    lib = tt._capi.lib
    # Warm up for at least `warmup` calls AND ~50 ms of GPU work: the clocks take tens of milliseconds to ramp,
    # which would otherwise be charged to short kernels.
    t_end = time.perf_counter() + 0.05
    n = 0
    while n < warmup or time.perf_counter() < t_end:
        fn()
        n += 1
        if n % 64 == 0:
            tt.get_backend(tt.kAMD).synchronize(0)
    tt.get_backend(tt.kAMD).synchronize(0)
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.ttamd_event_create(0, C.byref(e0))
    lib.ttamd_event_create(0, C.byref(e1))
    lib.ttamd_event_record(e0, None)
    for _ in range(iters):
        fn()
    lib.ttamd_event_record(e1, None)
    ms = C.c_float()
    lib.ttamd_event_elapsed_ms(e0, e1, C.byref(ms))
    lib.ttamd_event_destroy(e0)
    lib.ttamd_event_destroy(e1)
    return ms.value / iters


def detail_report(tt, np, path, cpu=True):
    """Times every benchmark configuration (GPU only, inputs resident) and writes a JSON report to `path`.
    Not part of the one-line contract; used to track the small-shape, strided and conv paths."""
    from oracle import tt_oracle as oracle  # seeded input generation only

    be = tt.get_backend(tt.kAMD)
    rows = []

    def gemm_case(name, tA, tB, iters=200):
        Bn, N, K = tA.shape
        M = tB.shape[2]
        out = tt.Tensor.empty((Bn, N, M), tA.dtype)
        ms = time_launches(tt, lambda: be.batched_matmul(tA, tB, out=out), iters, 20)
        flop = 2.0 * Bn * N * K * M
        nbytes = (Bn * N * K + Bn * K * M + Bn * N * M) * tA.itemsize
        rows.append({"case": name, "kernel": be.batched_matmul_variant(tA, tB), "ms": round(ms, 5),
                     "GFLOP/s": round(flop / ms / 1e6, 1), "GB/s": round(nbytes / ms / 1e6, 1)})

    f32 = np.float32
    g = oracle.Generator(0)
    A = tt.Tensor.from_numpy(g.uniform_real(-1, 1, (1, 256, 512)))
    B = tt.Tensor.from_numpy(g.uniform_real(-1, 1, (1, 512, 256)))
    gemm_case("cfg1 f32 256x512x256", A, B)
    A = tt.Tensor.from_numpy(g.uniform_real(-1, 1, (32, 128, 64)))
    Bs = tt.Tensor.from_numpy(g.uniform_real(-1, 1, (32, 128, 64)))
    gemm_case("cfg2 f32 32x(128x64x128) B=transposed view", A, Bs.permute(0, 2, 1))
    for dt, nm in ((f32, "f32"), (np.float64, "f64")):
        S = tt.Tensor.from_numpy(oracle.Generator(3).uniform_real(-1, 1, (1, 4096, 4096), dt))
        gemm_case(f"cfg3 {nm} 4096^3 A.B", S, S, 30)
        gemm_case(f"cfg3 {nm} 4096^3 A.B^T (view)", S, S.permute(0, 2, 1), 30)
        gemm_case(f"cfg3 {nm} 4096^3 A^T.B (view)", S.permute(0, 2, 1), S, 30)
    # config 5: the nine GEMMs of one MLP training step (batch 1024, 784-1024-1024-10)
    rnd = lambda *shape: tt.Tensor.from_numpy(g.uniform_real(-1, 1, shape))
    X, W1, H, W3, Y = rnd(1, 1024, 784), rnd(1, 784, 1024), rnd(1, 1024, 1024), rnd(1, 1024, 10), rnd(1, 1024, 10)
    t = lambda x: x.permute(0, 2, 1)
    for name, a, b in (("fwd1 X.W1", X, W1), ("fwd2 H.W2", H, H), ("fwd3 H.W3 (N=10)", H, W3),
                       ("bwd3 dH=dY.W3^T (K=10)", Y, t(W3)), ("bwd3 dW3=H^T.dY (N=10)", t(H), Y),
                       ("bwd2 dH=dZ.W2^T", H, t(H)), ("bwd2 dW2=H^T.dZ", t(H), H),
                       ("bwd1 dX=dZ.W1^T", H, t(W1)), ("bwd1 dW1=X^T.dZ", t(X), H)):
        gemm_case("cfg5 " + name, a, b)
    # config 5 as a whole: one training step through the tensor interface (fused Linear GEMMs, relu, mse_loss, the
    # backward pass op for op; every result is a fresh allocation served by the library's block cache)
    gp = oracle.Generator(0)
    Xh, Th = oracle.Generator(0).uniform_real(0.0, 1.0, (1024, 784)), oracle.Generator(1).uniform_real(0.0, 1.0, (1024, 10))
    params_h = [oracle.linear_init(gp, a, b) for a, b in ((784, 1024), (1024, 1024), (1024, 10))]
    xs, ts = tt.Tensor.from_numpy(Xh), tt.Tensor.from_numpy(Th)
    (P1, c1), (P2, c2), (P3, c3) = [(tt.Tensor.from_numpy(W), tt.Tensor.from_numpy(b)) for W, b in params_h]

    def train_step():
        z1 = tt.linear(xs, P1, c1); a1 = z1.relu(); z2 = tt.linear(a1, P2, c2); a2 = z2.relu(); y = tt.linear(a2, P3, c3)
        diff = y - ts
        loss = diff.pow(2.0).mean()
        gy = tt.full(y.shape, 2.0 / y.numel(), y.dtype) * diff
        grads = [gy.sum(0)]
        da2, dW3 = tt.matmul_backward(a2.unsqueeze(0), P3.unsqueeze(0), gy.unsqueeze(0))
        dz2 = da2.squeeze(0) * tt.where(z2 < 0.0, 0.0, 1.0)
        da1, dW2 = tt.matmul_backward(a1.unsqueeze(0), P2.unsqueeze(0), dz2.unsqueeze(0))
        dz1 = da1.squeeze(0) * tt.where(z1 < 0.0, 0.0, 1.0)
        dX, dW1 = tt.matmul_backward(xs.unsqueeze(0), P1.unsqueeze(0), dz1.unsqueeze(0))
        grads += [dz2.sum(0), dz1.sum(0), dW3, dW2, dW1, dX]
        return loss, grads

    for _ in range(5):
        train_step()
    be.synchronize(0)
    t0 = time.perf_counter()
    for _ in range(30):
        train_step()
    be.synchronize(0)
    step_ms = (time.perf_counter() - t0) / 30 * 1e3
    step_flop = 2.0 * 1024 * (784 * 1024 + 1024 * 1024 + 1024 * 10) * 3
    rows.append({"case": "cfg5 whole MLP training step (tensor interface, wall clock incl. host overhead)",
                 "kernel": "9 products (the two gradients of layers 1 and 2 as one launch each) + the streaming launches around them", "ms": round(step_ms, 4), "GFLOP/s": round(step_flop / step_ms / 1e6, 1)})
    # the same step recorded once into a HIP graph and replayed: one launch per step, no per-op host work
    gstream = tt.graph.Stream()
    graph = tt.graph.Graph(gstream, train_step)
    for _ in range(5):
        graph.launch()
    gstream.synchronize()
    t0 = time.perf_counter()
    for _ in range(30):
        graph.launch()
    gstream.synchronize()
    graph_ms = (time.perf_counter() - t0) / 30 * 1e3
    rows.append({"case": "cfg5 whole MLP training step replayed from a HIP graph", "kernel": f"{graph.num_nodes()} graph nodes",
                 "ms": round(graph_ms, 4), "GFLOP/s": round(step_flop / graph_ms / 1e6, 1)})
    graph.close()
    gstream.close()
    # the same step from the fused forms (Linear + ReLU, the last layer with the loss, each layer's two gradients as one call)

    def fused_step():
        z1, a1 = tt.linear_relu(xs, P1, c1); z2, a2 = tt.linear_relu(a1, P2, c2)
        y, loss, dz2, dW3, db3 = tt.linear_mse_head(a2, P3, c3, ts, relu_input=z2)
        dz1, dW2, db2 = tt.linear_backward(dz2, a1, P2, relu_input=z1, bias_grad="own")
        dX, dW1, db1 = tt.linear_backward(dz1, xs, P1, bias_grad="own")
        return [loss, dW1, db1, dW2, db2, dW3, db3, dX]

    gstream = tt.graph.Stream()
    graph = tt.graph.Graph(gstream, fused_step)
    for _ in range(20):
        graph.launch()
    gstream.synchronize()
    t0 = time.perf_counter()
    for _ in range(100):
        graph.launch()
    gstream.synchronize()
    fused_ms = (time.perf_counter() - t0) / 100 * 1e3
    rows.append({"case": "cfg5 whole MLP training step from the fused forms, replayed from a HIP graph", "kernel": f"{graph.num_nodes()} graph nodes",
                 "ms": round(fused_ms, 4), "GFLOP/s": round(step_flop / fused_ms / 1e6, 1)})
    graph.close()
    gstream.close()
    # one training step of the network of the reference's examples/mnist_cnn_example.cpp:31-63 at its batch size of 256
    # (conv 1->32, ReLU, conv 32->64, ReLU, max-pool, Linear 9216->128, ReLU, Linear 128->10; no dropout; squared error)
    crng = np.random.default_rng(3)
    cdev = lambda *shape, scale=0.1: tt.Tensor.from_numpy(crng.normal(0, scale, shape).astype(f32))
    cx, ct = cdev(256, 1, 28, 28, scale=1.0), cdev(256, 10, scale=1.0)
    cw1, cb1, cw2, cb2 = cdev(32, 1, 3, 3, scale=0.3), cdev(32), cdev(64, 32, 3, 3, scale=0.06), cdev(64)
    cW3, cb3, cW4, cb4 = cdev(9216, 128, scale=0.01), cdev(128), cdev(128, 10), cdev(10)
    mask = lambda z: tt.where(z < 0.0, 0.0, 1.0)

    def cnn_step():
        z1 = tt.conv2d(cx, cw1, cb1, 1, 0); a1 = z1.relu(); z2 = tt.conv2d(a1, cw2, cb2, 1, 0); a2 = z2.relu()
        pooled = tt.max_pool2d(a2, 2, 2, 0); flat = pooled.flatten(1)
        z3 = tt.linear(flat, cW3, cb3); a3 = z3.relu(); y = tt.linear(a3, cW4, cb4)
        gy = (y - ct) * 2.0
        da3, dW4 = tt.matmul_backward(a3.unsqueeze(0), cW4.unsqueeze(0), gy.unsqueeze(0))
        dz3 = da3.squeeze(0) * mask(z3)
        dflat, dW3 = tt.matmul_backward(flat.unsqueeze(0), cW3.unsqueeze(0), dz3.unsqueeze(0))
        da2 = tt.pool2d_backward(dflat.squeeze(0).reshape(list(pooled.shape)), a2, pooled, "max", 2, 2, 0)
        da1, dw2, db2 = tt.conv2d_backward(da2 * mask(z2), a1, cw2, cb2, 1, 0)
        dx, dw1, db1 = tt.conv2d_backward(da1 * mask(z1), cx, cw1, cb1, 1, 0)
        return [y, gy.sum(0), dW4, dz3.sum(0), dW3, dw2, db2, dw1, db1, dx]

    for _ in range(3):
        cnn_step()
    be.synchronize(0)
    t0 = time.perf_counter()
    for _ in range(20):
        cnn_step()
    be.synchronize(0)
    cnn_ms = (time.perf_counter() - t0) / 20 * 1e3
    cnn_flop = 3 * 2.0 * 256 * (32 * 26 * 26 * 9 + 64 * 24 * 24 * 288 + 9216 * 128 + 128 * 10)
    rows.append({"case": "mnist_cnn_example network, one training step at batch 256 (tensor interface, wall clock)",
                 "kernel": "2 conv + 2 Linear layers, pooling, elementwise", "ms": round(cnn_ms, 4), "GFLOP/s": round(cnn_flop / cnn_ms / 1e6, 1)})
    gstream = tt.graph.Stream()
    graph = tt.graph.Graph(gstream, cnn_step)
    for _ in range(3):
        graph.launch()
    gstream.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        graph.launch()
    gstream.synchronize()
    cnn_graph_ms = (time.perf_counter() - t0) / 20 * 1e3
    rows.append({"case": "mnist_cnn_example network, one training step at batch 256 replayed from a HIP graph",
                 "kernel": f"{graph.num_nodes()} graph nodes", "ms": round(cnn_graph_ms, 4), "GFLOP/s": round(cnn_flop / cnn_graph_ms / 1e6, 1)})
    graph.close()
    gstream.close()
    if cpu:
        sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests"))
        from helpers import mlp_train_step  # the same step written over an abstract GEMM
        t0 = time.perf_counter()
        mlp_train_step(Xh, Th, params_h, lambda a, b: oracle.matmul(a, b, "fast"),
                       lambda a, b, gr: tuple(v[0] for v in oracle.matmul_backward(a[None], b[None], gr[None], "fast")))
        rows[-1]["cpu_oracle_ms_1core"] = round((time.perf_counter() - t0) * 1e3, 1)
        rows[-1]["speedup_vs_cpu"] = round(rows[-1]["cpu_oracle_ms_1core"] / step_ms, 1)
    # config 4: conv2d forward / backward, input [64,32,28,28], weight [64,32,3,3], s1 p1
    x = tt.Tensor.from_numpy(oracle.Generator(0).normal(0, 0.1, (64, 32, 28, 28)))
    w = tt.Tensor.from_numpy(oracle.Generator(1).normal(0, 0.1, (64, 32, 3, 3)))
    go = tt.Tensor.from_numpy(np.ones((64, 64, 28, 28), f32))
    out = be.conv2d(x, w, None, 1, 1)
    ms = time_launches(tt, lambda: be.conv2d(x, w, None, 1, 1, out=out), 100, 10)
    lib_last = tt._capi.lib.ttamd_conv2d_last_kernel

    def conv_kernel(which, implicit):  # which family the last launch took (include/ttamd.h: ttamd_conv2d_last_kernel)
        code = tt._capi.lib.ttamd_conv2d_last_kernel(which)
        if code & 0xF00 == 0x200:
            return f"conv_patch_kernel (weights resident in LDS, {(code >> 4) & 0xF} waves, {code & 0xF} patch buffer(s))"
        return implicit

    rows.append({"case": "cfg4 conv2d forward", "kernel": conv_kernel(0, "conv_fwd_kernel (implicit GEMM)"), "ms": round(ms, 5),
                 "GFLOP/s": round(1.850e9 / ms / 1e6, 1)})
    bufs = be.conv2d_backward(go, x, w, None, 1, 1, return_buffers=True)
    ms = time_launches(tt, lambda: be.conv2d_backward(go, x, w, None, 1, 1, buffers=bufs), 50, 5)
    rows.append({"case": "cfg4 conv2d backward (grad_input + grad_weight)",
                 "kernel": conv_kernel(1, "conv_dgrad_kernel (implicit GEMM)") + " + "
                           + ("conv_wgrad_patch kernel (operands staged in LDS)" if lib_last(2) == 0x200 else "conv_wgrad_kernel (implicit GEMM)")
                           + {0: "", 1: " + a launch that adds up its partial tiles", 2: "; its partial tiles added up by workgroups appended to grad_input's launch"}[lib_last(3)],
                 "ms": round(ms, 5), "GFLOP/s": round(3.700e9 / ms / 1e6, 1)})
    # Streaming kernels around the GEMMs (HBM-bound; GB/s counts each operand and the result once), called through
    # the C ABI with preallocated results so that no allocation is timed.
    lib, cap = tt._capi.lib, tt._capi
    i64 = lambda v: (C.c_int64 * len(v))(*v)
    ptr = lambda t: C.c_void_p(t.storage.ptr)

    def stream_case(name, kernel, nbytes, fn, iters=50):
        ms = time_launches(tt, fn, iters, 5)
        rows.append({"case": name, "kernel": kernel, "ms": round(ms, 5), "GB/s": round(nbytes / ms / 1e6, 1),
                     "of_hbm_peak": round(nbytes / ms / 1e6 / 8000.0, 3)})

    n = 8192
    Ea = tt.Tensor.from_numpy(np.random.default_rng(0).random((n, n), dtype=f32))
    Eb = tt.Tensor.from_numpy(np.random.default_rng(2).random((n, n), dtype=f32))
    Eo = tt.Tensor.empty((n, n), cap.F32)
    Eo64 = tt.Tensor.empty((n, n), cap.F64)
    sh, st, stT = i64((n, n)), i64((n, 1)), i64((1, n))
    stream_case("add 8192x8192 f32", "binary_kernel", 3 * n * n * 4,
                lambda: lib.ttamd_binary(0, cap.F32, cap.BIN["add"], 2, sh, ptr(Ea), 0, st, ptr(Eb), 0, st, ptr(Eo), None))
    stream_case("relu 8192x8192 f32", "unary_kernel", 2 * n * n * 4,
                lambda: lib.ttamd_unary(0, cap.F32, cap.UN["relu"], 2, sh, ptr(Ea), 0, st, ptr(Eo), None))
    stream_case("contiguous of a transposed 8192x8192 f32 view", "contiguous_kernel", 2 * n * n * 4,
                lambda: lib.ttamd_contiguous(0, cap.F32, 2, sh, stT, ptr(Ea), 0, ptr(Eo), None))
    stream_case("cast 8192x8192 f32 -> f64", "cast_kernel", n * n * 12,
                lambda: lib.ttamd_cast(0, cap.F32, cap.F64, 2, sh, ptr(Ea), 0, st, ptr(Eo64), None))
    stream_case("sum 8192x8192 f32 (all)", "sum_all_kernel", n * n * 4,
                lambda: lib.ttamd_sum(0, cap.F32, 2, sh, ptr(Ea), 0, st, -1, ptr(Eo), None))
    m = 1024
    shm, stm = i64((m, m)), i64((m, 1))
    stream_case("cfg5 add 1024x1024 f32", "binary_kernel", 3 * m * m * 4,
                lambda: lib.ttamd_binary(0, cap.F32, cap.BIN["add"], 2, shm, ptr(Ea), 0, stm, ptr(Eb), 0, stm, ptr(Eo), None), 200)
    # pooling on [64,64,112,112] f32 (205 MB): k2 s2 p0 and k3 s2 p1
    Pb, Pc, Ph, Pw = 64, 64, 112, 112
    Px = tt.Tensor.from_numpy(np.random.default_rng(1).random((Pb, Pc, Ph, Pw), dtype=f32))
    for k, S_, P_ in ((2, 2, 0), (3, 2, 1)):
        Ho, Wo = (Ph + 2 * P_ - k) // S_ + 1, (Pw + 2 * P_ - k) // S_ + 1
        Pout = tt.Tensor.empty((Pb, Pc, Ho, Wo), cap.F32)
        Pg = tt.Tensor.from_numpy(np.ones((Pb, Pc, Ho, Wo), f32))
        Pgx = tt.Tensor.empty((Pb, Pc, Ph, Pw), cap.F32)
        iv = Px.view4()
        in_b, out_b = Pb * Pc * Ph * Pw * 4, Pb * Pc * Ho * Wo * 4
        for op in ("max", "avg"):
            code = cap.POOL[op]
            nonoverlap = S_ == k and P_ == 0
            fwd_kernel = "pool_forward_k2_kernel" if (nonoverlap and k == 2) else "pool_forward_k3s2_kernel"
            stream_case(f"{op}_pool2d forward k{k} s{S_} p{P_} [64,64,112,112] f32", fwd_kernel, in_b + out_b,
                        lambda: lib.ttamd_pool2d_forward(0, cap.F32, code, C.byref(iv), ptr(Pout), Pb, Pc, Ph, Pw, k, S_, P_, None), 30)
            if nonoverlap:
                bwd_kernel = "pool_backward_window_kernel"
            else:
                bwd_kernel = "pool_backward_quad_kernel" if op == "avg" else "pool_backward_k3s2_tile_kernel"
            # algorithmic bytes of backward: grad_out and grad_input, plus the input and the result for max / min
            bwd_b = (in_b + out_b) if op == "avg" else (2 * in_b + 2 * out_b)
            stream_case(f"{op}_pool2d backward k{k} s{S_} p{P_} [64,64,112,112] f32", bwd_kernel, bwd_b,
                        lambda: lib.ttamd_pool2d_backward(0, cap.F32, code, ptr(Pg), C.byref(iv), ptr(Pout), ptr(Pgx), Pb, Pc, Ph, Pw,
                                                          k, S_, P_, None), 30)
    if cpu:
        ph = np.random.default_rng(1).random((8, 64, 112, 112), dtype=f32)  # an eighth of the batch
        for k, S_, P_ in ((2, 2, 0), (3, 2, 1)):
            for op in ("max", "avg"):
                t0 = time.perf_counter()
                res = oracle.pool2d_forward(ph, op, k, S_, P_)
                t1 = time.perf_counter()
                oracle.pool2d_backward(np.ones_like(res), ph, res, op, k, S_, P_)
                t2 = time.perf_counter()
                for r in rows:
                    if r["case"] == f"{op}_pool2d forward k{k} s{S_} p{P_} [64,64,112,112] f32":
                        r["cpu_oracle_ms_1core"] = round((t1 - t0) * 8e3, 1)
                    if r["case"] == f"{op}_pool2d backward k{k} s{S_} p{P_} [64,64,112,112] f32":
                        r["cpu_oracle_ms_1core"] = round((t2 - t1) * 8e3, 1)
        for r in rows:
            if "pool2d" in r["case"] and "cpu_oracle_ms_1core" in r:
                r["speedup_vs_cpu"] = round(r["cpu_oracle_ms_1core"] / r["ms"], 1)
    if cpu:
        # The same configurations on the CPU oracle (one core), timed once each.
        xh, wh = oracle.Generator(0).normal(0, 0.1, (64, 32, 28, 28)), oracle.Generator(1).normal(0, 0.1, (64, 32, 3, 3))
        for name, fn in (
            ("cfg1 f32 256x512x256", lambda: oracle.matmul(np.ones((256, 512), f32), np.ones((512, 256), f32), "fast")),
            ("cfg2 f32 32x(128x64x128) B=transposed view",
             lambda: oracle.matmul(np.ones((32, 128, 64), f32), np.ones((32, 128, 64), f32).transpose(0, 2, 1), "fast")),
            ("cfg4 conv2d forward", lambda: oracle.conv2d_forward(xh, wh, None, 1, 1, "fast")),
            ("cfg4 conv2d backward (grad_input + grad_weight)",
             lambda: oracle.conv2d_backward(np.ones((64, 64, 28, 28), f32), xh, wh, False, 1, 1, "fast")),
            ("cfg5 fwd2 H.W2", lambda: oracle.matmul(np.ones((1024, 1024), f32), np.ones((1024, 1024), f32), "fast")),
            ("cfg5 fwd3 H.W3 (N=10)", lambda: oracle.matmul(np.ones((1024, 1024), f32), np.ones((1024, 10), f32), "fast")),
        ):
            fn()
            t0 = time.perf_counter()
            fn()
            dt = (time.perf_counter() - t0) * 1e3
            for r in rows:
                if r["case"] == name:
                    r["cpu_oracle_ms_1core"] = round(dt, 3)
                    r["speedup_vs_cpu"] = round(dt / r["ms"], 1)
    with open(path, "w") as f:
        json.dump(rows, f, indent=1)
    for r in rows:
        print(json.dumps(r), file=sys.stderr)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--n", type=int, default=4096, help="square size (the metric is quoted at 4096)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first run one dense 256 MiB copy kernel (known HBM traffic) to scale profiler byte counters")
    ap.add_argument("--detail", metavar="FILE", help="also time every benchmark configuration and write a JSON report")
    ap.add_argument("--conv-loop", type=int, metavar="N", default=0,
                    help="only run N conv2d forward + backward passes of benchmark configuration 4 (input [64,32,28,28], weight [64,32,3,3], s1 p1) (a short target for profilers) and exit")
    ap.add_argument("--mlp-loop", type=int, metavar="N", default=0,
                    help="only run N training steps of benchmark configuration 5 (batch 1024, 784-1024-1024-10, mse_loss) from the fused "
                         "forms (a short target for profilers), print the wall-clock time per step and exit")
    ap.add_argument("--mlp-ops", action="store_true", help="with --mlp-loop: the step op by op (unfused) instead")
    ap.add_argument("--mlp-separate-head", action="store_true",
                    help="with --mlp-loop: the last layer, the loss and their backward as four launches instead of the two of linear_mse_head")
    ap.add_argument("--conv-shape", metavar="B,C,O,H,W[,k,S,P]", default="64,32,64,28,28",
                    help="geometry for --conv-loop (kernel 3, stride 1, padding 1 unless given); the default is benchmark "
                         "configuration 4")
    ap.add_argument("--conv-time", action="store_true",
                    help="with --conv-loop: also time forward and backward by HIP events (min of three bursts of N passes)")
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

    if args.conv_loop:
        be = tt.get_backend(tt.kAMD)
        rng = np.random.default_rng(0)
        dims = [int(v) for v in args.conv_shape.split(",")]
        cb, cc, co, ch, cw = dims[:5]
        ck, cs, cp = (dims[5:] + [3, 1, 1][len(dims) - 5:]) if len(dims) > 5 else (3, 1, 1)
        x = tt.Tensor.from_numpy(rng.normal(0, 0.1, (cb, cc, ch, cw)).astype(np.float32))
        w = tt.Tensor.from_numpy(rng.normal(0, 0.1, (co, cc, ck, ck)).astype(np.float32))
        out = be.conv2d(x, w, None, cs, cp)
        go = tt.Tensor.from_numpy(np.ones(out.shape, np.float32))
        bufs = be.conv2d_backward(go, x, w, None, cs, cp, return_buffers=True)
        for _ in range(args.conv_loop):
            be.conv2d(x, w, None, cs, cp, out=out)
            be.conv2d_backward(go, x, w, None, cs, cp, buffers=bufs)
        be.synchronize(0)
        line = {"conv_loop": args.conv_loop, "config": f"input [{cb},{cc},{ch},{cw}], weight [{co},{cc},{ck},{ck}], s{cs} p{cp}, f32"}
        if args.conv_time:
            fwd_ms = min(time_launches(tt, lambda: be.conv2d(x, w, None, cs, cp, out=out), args.conv_loop, 3) for _ in range(3))
            bwd_ms = min(time_launches(tt, lambda: be.conv2d_backward(go, x, w, None, cs, cp, buffers=bufs), args.conv_loop, 3) for _ in range(3))
            flop = 2.0 * cb * co * out.shape[2] * out.shape[3] * cc * ck * ck
            line.update({"forward_us": round(fwd_ms * 1e3, 2), "forward_tflops": round(flop / fwd_ms / 1e9, 1),
                         "backward_us": round(bwd_ms * 1e3, 2), "backward_tflops": round(2 * flop / bwd_ms / 1e9, 1)})
        print(json.dumps(line))
        return

    if args.mlp_loop:
        from oracle import tt_oracle as oracle  # seeded inputs and default init (host restatement of the reference's RNG)

        be = tt.get_backend(tt.kAMD)
        gp = oracle.Generator(0)
        xs = tt.Tensor.from_numpy(oracle.Generator(0).uniform_real(0.0, 1.0, (1024, 784)))
        ts = tt.Tensor.from_numpy(oracle.Generator(1).uniform_real(0.0, 1.0, (1024, 10)))
        (P1, c1), (P2, c2), (P3, c3) = [tuple(tt.Tensor.from_numpy(v) for v in oracle.linear_init(gp, a, b))
                                        for a, b in ((784, 1024), (1024, 1024), (1024, 10))]

        def fused_step():
            z1, a1 = tt.linear_relu(xs, P1, c1); z2, a2 = tt.linear_relu(a1, P2, c2)
            if args.mlp_separate_head:
                y = tt.linear(a2, P3, c3)
                loss, gy, db3 = tt.mse_loss(y, ts, grad=True, bias_grad=True)
                dz2, dW3, _ = tt.linear_backward(gy, a2, P3, relu_input=z2, bias_grad=False)
            else:  # the 10-class layer, the loss and their backward: two launches
                y, loss, dz2, dW3, db3 = tt.linear_mse_head(a2, P3, c3, ts, relu_input=z2)
            # (bias gradients of layers 1 and 2 from the vectors of dz that the weight-gradient products stage)
            dz1, dW2, db2 = tt.linear_backward(dz2, a1, P2, relu_input=z1, bias_grad="own")
            dX, dW1, db1 = tt.linear_backward(dz1, xs, P1, bias_grad="own")
            return [loss, dW1, db1, dW2, db2, dW3, db3, dX]

        def ops_step():
            z1 = tt.linear(xs, P1, c1); a1 = z1.relu(); z2 = tt.linear(a1, P2, c2); a2 = z2.relu(); y = tt.linear(a2, P3, c3)
            diff = y - ts
            loss = diff.pow(2.0).mean()
            gy = tt.full(y.shape, 2.0 / y.numel(), y.dtype) * diff
            da2, dW3 = tt.matmul_backward(a2.unsqueeze(0), P3.unsqueeze(0), gy.unsqueeze(0))
            dz2 = da2.squeeze(0) * tt.where(z2 < 0.0, 0.0, 1.0)
            da1, dW2 = tt.matmul_backward(a1.unsqueeze(0), P2.unsqueeze(0), dz2.unsqueeze(0))
            dz1 = da1.squeeze(0) * tt.where(z1 < 0.0, 0.0, 1.0)
            dX, dW1 = tt.matmul_backward(xs.unsqueeze(0), P1.unsqueeze(0), dz1.unsqueeze(0))
            return [loss, gy.sum(0), dz2.sum(0), dz1.sum(0), dW3, dW2, dW1, dX]

        step = ops_step if args.mlp_ops else fused_step
        stream = tt.graph.Stream()
        graph = tt.graph.Graph(stream, step)  # replayed from a HIP graph: the kernels' own time, no per-op host work
        for _ in range(20):
            graph.launch()
        stream.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.mlp_loop):
            graph.launch()
        stream.synchronize()
        ms = (time.perf_counter() - t0) / args.mlp_loop * 1e3
        print(json.dumps({"mlp_loop": args.mlp_loop, "form": "op by op" if args.mlp_ops else "fused", "graph_nodes": graph.num_nodes(),
                          "ms_per_step": round(ms, 4), "config": "batch 1024, 784-1024-1024-10, f32, forward + backward"}))
        graph.close()
        stream.close()
        return

    if args.detail:
        detail_report(tt, np, args.detail, cpu=not args.no_cpu)

    n = args.n
    flop = 2.0 * n * n * n
    wall_ms, kern_ms, variant, (A, B, out), warm_eff = gpu_gemm_timing(tt, np, np.float32, n, args.steps, args.warmup)
    gflops = flop / (wall_ms * 1e-3) / 1e9
    achieved_tflops = flop / (kern_ms * 1e-3) / 1e12

    # spot parity inside the bench run: one band of rows against the oracle
    from oracle import tt_oracle as oracle

    Cg = out.to_numpy()[0]
    rows = slice(0, 64)
    want = oracle.matmul(A[rows], B, "fast")
    scale = np.abs(A[rows]).astype(np.float64) @ np.abs(B).astype(np.float64)
    parity = float(np.max(np.abs(Cg[rows].astype(np.float64) - want.astype(np.float64)) / scale))

    wall64, kern64, variant64, _, _ = gpu_gemm_timing(tt, np, np.float64, n, max(args.steps // 2, 1), args.warmup)
    f64_tflops = flop / (kern64 * 1e-3) / 1e12

    cpu = None
    if not args.no_cpu:
        # Bounded sample of the same workload on one host core: the full product at n <= 4096 (~10 s),
        # timed once; the tiled restatement of the reference CPU kernel, fma flavour.
        t0 = time.perf_counter()
        oracle.matmul_kernel(A, B, "fast")
        dt = time.perf_counter() - t0
        cpu = {"value": round(flop / dt / 1e9, 3), "unit": "GFLOP/s", "cores": 1, "kind": "port",
               "sample": f"one full f32 {n}x{n}x{n} product, {dt:.1f} s, oracle built with gcc -O3 -ffp-contract=fast "
                         + ("-march=x86-64-v4 -mprefer-vector-width=128" if oracle._cpu_has("avx512vl") else "-march=x86-64-v3")
                         + f" (same arithmetic either way), host has {os.cpu_count()} logical cores"}

    line = {
        "metric": f"fp32 GEMM GFLOP/s at {n}^3 on 1 MI355X",
        "value": round(gflops, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "warmup_effective": warm_eff,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic: uniform(-1,1) from the reference's seeded generator (seeds 0 and 1)",
        "config": {"workload": (f"configs[2]: fp32 {n}x{n} @ {n}x{n}, dense row-major" if n == 4096 else
                                f"fp32 {n}x{n} @ {n}x{n}, dense row-major (not a benchmark configuration)"), "kernel": variant,
                   "parity_k_scaled_err_rows0_63": parity},
        "roofline": {"bound": "mfma", "achieved": round(achieved_tflops, 2), "peak": PEAK_TFLOPS["f32"],
                     "unit": "TFLOP/s", "frac": round(achieved_tflops / PEAK_TFLOPS["f32"], 4),
                     "traffic": MEASURED_TRAFFIC.get((variant, n)),
                     "traffic_source": ("profiles/gemm_4096_f32_f64_mfma.txt (rocprofv3 FETCH_SIZE / WRITE_SIZE passes of this "
                                        "kernel and size; a recorded figure, not measured in this run)"
                                        if (variant, n) in MEASURED_TRAFFIC else None),
                     "algorithmic_bytes": 3.0 * n * n * 4,
                     "kernel_ms": round(kern_ms, 4)},
        "cpu_baseline": cpu,
        "fp64": {"kernel": variant64, "kernel_ms": round(kern64, 4), "achieved": round(f64_tflops, 2),
                 "peak": PEAK_TFLOPS["f64"], "unit": "TFLOP/s", "frac": round(f64_tflops / PEAK_TFLOPS["f64"], 4)},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
