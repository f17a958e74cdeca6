#!/usr/bin/env python3
"""Benchmark of the dense-layer training step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload wide_mlp|sine_mlp]

Default workload (the one the headline metric is quoted on): 8 Linear layers 4096 -> 4096 with bias,
tanh between, MSE against N(0,1) targets, batch 4096, Adam(lr 1e-3, betas 0.9/0.999, eps 1e-8),
x ~ N(0,1), W ~ N(0, 1/4096), b ~ N(0, 1/4096); synthetic data, random-init weights. One step is
forward + loss + backward + Adam + zero_grad, the loop of the reference's MLP benchmark
(benchmarks/mlp_benchmarks/mlp_imp.mojo:47-75), with inputs resident in HBM before the timed region.

Prints ONE JSON line. `value` is train steps/s. `roofline` describes the dominant kernel (the fp32 MFMA
GEMM): algorithmic 2*M*N*K flops per launch over the average launch duration, measured with HIP event
pairs around every GEMM launch inside the timed region, against the 157.3 TFLOP/s dense fp32 matrix
peak. `cpu_baseline` times the single-threaded CPU restatement of the reference's algorithms
(oracle/) on a bounded sample of the same workload and extrapolates to one step.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0
# HBM-side bytes per 4096^3 GEMM launch, averaged over the launch mix of one training step (1 NN with the bias epilogue,
# 7 NN with bias+tanh, 7 NT with the tanh' epilogue, 8 TN, all on the 256 x 256 tile; MiB per launch as in the per-kernel table). It cannot be read while the benchmark runs: it comes
# from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE in KiB per dispatch), each scaled by what the same counter
# reads for a 64 MiB copy kernel (x1.999 and x1.000); the per-kernel table is in profiles/.
GEMM_TRAFFIC_BYTES = int((1 * 456.7 + 7 * 449.1 + 7 * 512.3 + 8 * 456.4) / 23 * 1024 * 1024)


def build_wide_mlp(nd, width=4096, layers=8, batch=4096, seed=2, fused_backward=False):
    rng = np.random.default_rng(seed)
    std = 1.0 / np.sqrt(width)
    mlp = nd.nn.MLP([width] * (layers + 1), compute_backward=True, activation="tanh", fused=True)
    for i in range(layers):
        mlp.weights[i] = nd.array((rng.standard_normal((width, width)) * std).astype(np.float32), requires_grad=True)
        mlp.biases[i] = nd.array((rng.standard_normal(width) * std).astype(np.float32), requires_grad=True)
    x = nd.array(rng.standard_normal((batch, width)).astype(np.float32))
    y = nd.array(rng.standard_normal((batch, width)).astype(np.float32))
    opt = nd.optim.Adam(mlp.params(), lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, fused_backward=fused_backward)
    return mlp, opt, x, y


def build_sine_mlp(nd, seed=0, optimizer="sgd", per_layer=False):
    rng = np.random.default_rng(seed)
    widths = [1, 32, 64, 128, 128, 128, 64, 32, 1]
    # fused="model": the whole stack is one op (one launch forward, two backward); per_layer keeps one op per layer
    mlp = nd.nn.MLP(widths, compute_backward=True, activation="relu", fused=True if per_layer else "model")
    for i in range(8):
        s = np.sqrt(2.0 / widths[i])
        mlp.weights[i] = nd.array((rng.standard_normal((widths[i], widths[i + 1])) * s).astype(np.float32), requires_grad=True)
        mlp.biases[i] = nd.array((rng.standard_normal(widths[i + 1]) * s).astype(np.float32), requires_grad=True)
    xb = rng.uniform(0, 1, (128, 1)).astype(np.float32)
    x, y = nd.array(xb), nd.array(np.sin(2 * np.pi * xb).astype(np.float32))
    # "adam" is what the reference's own script uses (benchmarks/mlp_benchmarks/mlp_imp.mojo:38-40); its step counter
    # lives in device memory here so that the step can be replayed as a graph
    opt = nd.optim.SGD(mlp.params(), lr=1e-3) if optimizer == "sgd" else nd.optim.Adam(mlp.params(), lr=1e-3, capturable=True)
    return mlp, opt, x, y


def train_step(nd, mlp, opt, x, y, fused_loss=False):
    if fused_loss:  # forward and loss behind one method, which a whole-model MLP evaluates in its forward launch
        loss = mlp.mse_loss(x, y)
    else:  # the reference script's call shape: forward, then mse (mlp_imp.mojo:56-60)
        loss = nd.mse(mlp.forward(x), y)
    loss.backward()
    opt.step()
    loss.zero_grad()
    return loss


def cpu_baseline_wide(width=4096, layers=8, batch=4096, rows=None, target_seconds=15.0):
    # (the probe below under-estimates the cost per row about 2.5x: the divisor 1.3 is calibrated on the box)
    """Single-threaded ref-order restatement, timed on row slices of the real shapes and composed by op
    count: one step = 8 NN + 7 NT + 8 TN GEMMs, 7 tanh forward + 7 tanh VJPs, 8 bias adds, 8 column sums,
    1 MSE, Adam over 8 weight matrices (biases are 0.02 % of the work and are ignored)."""
    from oracle import endia_ref as R
    rng = np.random.default_rng(0)
    t_all0 = time.perf_counter()
    X = rng.standard_normal((batch, width)).astype(np.float32)
    W = (rng.standard_normal((width, width)) / 64).astype(np.float32)
    if rows is None:
        # size the sample to about target_seconds of CPU work: a 64-row probe of the NN GEMM sets the rate
        t0 = time.perf_counter()
        R.matmul(X[:64], W)
        per_row = (time.perf_counter() - t0) / 64
        rows = int(target_seconds / (1.3 * per_row)) // 64 * 64
        rows = max(64, min(rows, batch))
    scale = batch / rows

    def timed(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    t_nn = timed(lambda: R.matmul(X[:rows], W)) * scale              # Z = A W          (rows of the batch)
    t_nt = timed(lambda: R.matmul(X[:rows], W.T)) * scale            # dA = dZ W^T
    t_tn = timed(lambda: R.matmul(X[:, :rows].T, X)) * (width / rows)  # dW = A^T dZ    (rows of dW)
    Z = X[:rows]
    t_tanh = timed(lambda: R.unary("tanh", Z)) * scale
    t_tanh_vjp = timed(lambda: R.unary_vjp("tanh", Z, Z)) * scale
    t_bias = timed(lambda: R.binary("add", Z, W[0])) * scale
    t_col = timed(lambda: R.reduce_add(Z, [0])) * scale
    t_mse = timed(lambda: R.mse(Z, Z)) * scale
    Wp = W[:rows].copy()
    t_adam = timed(lambda: R.adam(Wp, Wp, Wp, Wp)) * (width / rows)
    step = (layers * t_nn + (layers - 1) * t_nt + layers * t_tn + (layers - 1) * (t_tanh + t_tanh_vjp) +
            layers * (t_bias + t_col) + t_mse + layers * t_adam)
    return {
        "value": 1.0 / step, "unit": "steps/s", "cores": 1, "kind": "port",
        "host_cores_available": os.cpu_count(),
        "sample": "ref-order CPU restatement (oracle/endia_ref.c, 1 thread): %d-row slices of each of the three "
                  "4096^3 GEMM modes and of each streaming op, extrapolated to full size and composed by op count "
                  "(8 NN + 7 NT + 8 TN GEMMs, 14 tanh passes, 8 bias adds, 8 column sums, MSE, Adam); "
                  "%.1f s of CPU work" % (rows, time.perf_counter() - t_all0),
        "seconds_per_step": step,
        "gemm_seconds_per_step": layers * t_nn + (layers - 1) * t_nt + layers * t_tn,
    }


def cpu_baseline_sine(steps=200, optimizer="sgd"):
    from oracle import endia_ref as R
    rng = np.random.default_rng(0)
    widths = [1, 32, 64, 128, 128, 128, 64, 32, 1]
    Ws = [(rng.standard_normal((widths[i], widths[i + 1])) * np.sqrt(2.0 / widths[i])).astype(np.float32) for i in range(8)]
    bs = [(rng.standard_normal(widths[i + 1]) * np.sqrt(2.0 / widths[i])).astype(np.float32) for i in range(8)]
    xb = rng.uniform(0, 1, (128, 1)).astype(np.float32)
    yb = np.sin(2 * np.pi * xb).astype(np.float32)
    state = None
    if optimizer == "adam":
        state = {k: [np.zeros_like(a) for a in (Ws if k.endswith("W") else bs)] for k in ("mW", "vW", "mb", "vb")}
    R.mlp_step(widths, "relu", xb, yb, Ws, bs, opt=optimizer, lr=1e-3, t=1.0, state=state)
    t0 = time.perf_counter()
    for i in range(steps):
        R.mlp_step(widths, "relu", xb, yb, Ws, bs, opt=optimizer, lr=1e-3, t=float(i + 2), state=state)
    dt = time.perf_counter() - t0
    return {"value": steps / dt, "unit": "steps/s", "cores": 1, "kind": "port", "host_cores_available": os.cpu_count(),
            "sample": "%d full fwd+bwd+%s steps of the ref-order CPU restatement, 1 thread" % (steps, optimizer.upper() if optimizer == "sgd" else "Adam")}


def _timed(fn):
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


def _extrapolate(fn, r1, r2, full):
    """Time fn(r) on two slice heights and extend the straight line through them to `full` rows: the per-call
    copies of the reference's matmul (contiguous LHS, transposed RHS) are then counted once, not once per slice."""
    t1, t2 = _timed(lambda: fn(r1)), _timed(lambda: fn(r2))
    per_row = max((t2 - t1) / (r2 - r1), 0.0)
    return max(t1 - r1 * per_row, 0.0) + full * per_row


def cpu_baseline_hvp():
    """The reference's single-threaded path for one Hessian-vector product, composed by op count: one full
    product of each mode timed at its real shape (the tape issues 11 NN, 9 NT and 11 TN products of
    1024 x 2048 x 2048) plus the elementwise and reduction passes over [1024, 2048] arrays that the double
    backward adds (counted on the device trace)."""
    from oracle import endia_ref as R
    rng = np.random.default_rng(3)
    t_all0 = time.perf_counter()
    B, Wd = 1024, 2048
    X = rng.standard_normal((B, Wd)).astype(np.float32)
    W = (rng.standard_normal((Wd, Wd)) / np.sqrt(Wd)).astype(np.float32)
    t_nn = _timed(lambda: R.matmul(X, W))
    t_nt = _timed(lambda: R.matmul(X, W.T))
    t_tn = _timed(lambda: R.matmul(X.T, X))
    t_bin = _timed(lambda: R.binary("mul", X, X))
    t_un = _timed(lambda: R.unary("sin", X))
    t_red = _timed(lambda: R.reduce_add(X, [0]))
    n_bin, n_un, n_red = 58, 12, 17
    step = 11 * t_nn + 9 * t_nt + 11 * t_tn + n_bin * t_bin + n_un * t_un + n_red * t_red
    return {"value": 1.0 / step, "unit": "HVP/s", "cores": 1, "kind": "port", "host_cores_available": os.cpu_count(),
            "seconds_per_step": step,
            "sample": "ref-order CPU restatement (oracle/endia_ref.c, 1 thread): one full 1024 x 2048 x 2048 product of each mode "
                      "(NN, NT, TN) composed as 11 + 9 + 11 products, plus %d binary, %d unary and %d reduction passes over "
                      "[1024, 2048], each timed once at full size; %.1f s of CPU work" % (n_bin, n_un, n_red, time.perf_counter() - t_all0)}


def cpu_baseline_complex(rows=512):
    """The reference's complex matmul (four real multiply-adds per element, matmul_op.mojo:201-238) on row slices
    of the 2048^3 products, composed as the step issues them: 4 forward (NN), 3 data gradients (NT), 4 weight
    gradients (TN)."""
    from oracle import endia_ref as R
    rng = np.random.default_rng(4)
    t_all0 = time.perf_counter()
    n = 2048
    Z = (rng.standard_normal((n, n)) + 1j * rng.standard_normal((n, n))).astype(np.complex64)
    t_nn = _extrapolate(lambda r: R.matmul(Z[:r], Z), rows, 2 * rows, n)
    t_nt = _extrapolate(lambda r: R.matmul(Z[:r], Z.T), rows, 2 * rows, n)
    t_tn = _extrapolate(lambda r: R.matmul(Z[:, :r].T, Z), rows, 2 * rows, n)
    step = 4 * t_nn + 3 * t_nt + 4 * t_tn
    return {"value": 1.0 / step, "unit": "steps/s", "cores": 1, "kind": "port", "host_cores_available": os.cpu_count(),
            "seconds_per_step": step,
            "sample": "ref-order CPU restatement (1 thread): %d- and 2x%d-row slices of the complex NN, NT and TN products of 2048^3, "
                      "extrapolated linearly and composed as 4 + 3 + 4 products (the elementwise loss passes are under 1 %% and "
                      "left out); %.1f s of CPU work" % (rows, rows, time.perf_counter() - t_all0)}


def cpu_baseline_conv(n_img=16):
    """The reference's 7-deep convolution loop (conv2d_op.mojo:127-196) and the brute-force adjoints of it, on n_img
    images of the batch of 64, extrapolated; plus the ReLU / mean passes over those images' output."""
    from oracle import endia_ref as R
    rng = np.random.default_rng(5)
    t_all0 = time.perf_counter()
    C, H, K = 64, 56, 128
    x = rng.standard_normal((n_img, C, H, H)).astype(np.float32)
    w = (rng.standard_normal((K, C, 3, 3)) * np.sqrt(2.0 / (C * 9))).astype(np.float32)
    bias = rng.standard_normal(K).astype(np.float32)
    dy = rng.standard_normal((n_img, K, H, H)).astype(np.float32)
    scale = 64 / n_img
    t_fwd = _timed(lambda: R.conv2d(x, w, bias, (1, 1), (1, 1), (1, 1))) * scale
    t_bwd = _timed(lambda: R.conv2d_bwd(x, w, dy, (1, 1), (1, 1), (1, 1))) * scale   # dx, dw and db together
    t_ew = (_timed(lambda: R.unary("relu", dy)) + _timed(lambda: R.unary_vjp("relu", dy, dy)) +
            _timed(lambda: R.reduce_add(dy.reshape(1, -1), [1]))) * scale
    step = t_fwd + t_bwd + t_ew
    return {"value": 1.0 / step, "unit": "steps/s", "cores": 1, "kind": "port", "host_cores_available": os.cpu_count(),
            "seconds_per_step": step, "forward_seconds": t_fwd, "gradients_seconds": t_bwd,
            "sample": "ref-order CPU restatement (1 thread): forward loop and its adjoints (dx, dw, db) on %d of the 64 "
                      "images, extrapolated by %g, plus relu / relu-gradient / mean passes; %.1f s of CPU work"
                      % (n_img, scale, time.perf_counter() - t_all0)}


def kernel_table(reps=10):
    """Times each hot kernel alone at the wide-MLP shape with HIP events on the library's stream and
    prices it against its roofline (fp32 MFMA peak for the GEMMs, HBM peak for the rest). Algorithmic
    bytes: every operand read once, every result written once. The `copy` row (out = 1.0 * a, 64 MiB in,
    64 MiB out) is the known-size kernel that scales the FETCH_SIZE / WRITE_SIZE counters."""
    from endia_amd import _lib as L
    L.ensure_init(0)
    n = 4096
    nn = n * n

    def dmalloc(nbytes):
        p = ctypes.c_void_p()
        L.call("endia_hip_malloc", nbytes, ctypes.byref(p))
        return p.value

    rng = np.random.default_rng(0)
    host = (rng.standard_normal(nn) / 64).astype(np.float32)
    bufs = [dmalloc(4 * nn) for _ in range(5)]
    for b in bufs:
        L.call("endia_hip_memcpy_h2d", b, host.ctypes.data, host.nbytes)
    A, B, C, D, E = bufs
    bias = dmalloc(4 * n)
    L.call("endia_hip_memcpy_h2d", bias, host.ctypes.data, 4 * n)
    loss = dmalloc(4)
    I = L.OP_IDENTITY

    def gemm(ta, tb, epi=L.EPI_NONE, act=I, aux=None):
        return lambda: L.call("endia_hip_sgemm", ta, tb, n, n, n, A, n, B, n, C, n, 1, 0, 0, 0, epi, act, bias, aux, None)

    gflop = 2.0 * n * n * n
    cases = [
        ("sgemm_nn  Z = A W", gemm(0, 0), gflop, "mfma"),
        ("sgemm_nn  tanh(A W + b) epilogue", gemm(0, 0, L.EPI_BIAS_ACT, L.OP_TANH), gflop, "mfma"),
        ("sgemm_nt  dA = dZ W^T", gemm(0, 1), gflop, "mfma"),
        ("sgemm_nt  (dZ W^T) * tanh' epilogue", gemm(0, 1, L.EPI_ACT_GRAD, L.OP_TANH | L.ACT_FROM_OUTPUT, D), gflop, "mfma"),
        ("sgemm_tn  dW = A^T dZ", gemm(1, 0), gflop, "mfma"),
        ("copy      out = a (64 MiB)", lambda: L.call("endia_hip_axpby", nn, 1.0, A, 0.0, None, C), 8.0 * nn, "hbm"),
        ("col_reduce  db = 1^T dZ", lambda: L.call("endia_hip_reduce_add", 2, L.i64_array([n, n]), 1, A, bias, 1.0, 0),
         4.0 * nn + 4.0 * n, "hbm"),
        ("mse_fwd_bwd", lambda: L.call("endia_hip_mse_fwd_bwd", nn, A, B, loss, C), 12.0 * nn, "hbm"),
        ("adam_step (one 4096^2 weight)", lambda: L.call("endia_hip_adam_step", nn, C, A, D, E, 1e-3, 0.9, 0.999, 1e-8, 1.0),
         28.0 * nn, "hbm"),
        ("sgd_step", lambda: L.call("endia_hip_sgd_step", nn, C, A, 1e-3), 12.0 * nn, "hbm"),
        ("tanh_fwd", lambda: L.call("endia_hip_unary_fwd", L.OP_TANH, nn, A, C, 0), 8.0 * nn, "hbm"),
        ("tanh_vjp", lambda: L.call("endia_hip_unary_vjp", L.OP_TANH, nn, A, B, C, 0), 12.0 * nn, "hbm"),
    ]
    # fused elementwise programs: tanh(a * b + bias) in one pass (two full inputs, one output) and a
    # two-output gradient program (four full inputs, two outputs)
    I_, S_, M_ = L.EW_SRC_INPUT, L.EW_SRC_SLOT, L.EW_SRC_IMM
    fwd_steps = [(L.EW_LOAD, 0, I_, 0, 0.0), (L.EW_BINARY, L.BIN_MUL, I_, 1, 0.0), (L.EW_BINARY, L.BIN_ADD, I_, 2, 0.0),
                 (L.EW_UNARY, L.OP_TANH, 0, 0, 0.0), (L.EW_STORE, 0, 0, 0, 0.0)]
    bwd_steps = [(L.EW_LOAD, 0, I_, 2, 0.0), (L.EW_UNARY, L.OP_SQUARE, 0, 0, 0.0), (L.EW_RBINARY, L.BIN_SUB, M_, 0, 1.0),
                 (L.EW_BINARY, L.BIN_MUL, I_, 3, 0.0), (L.EW_SAVE, 0, 0, 0, 0.0), (L.EW_BINARY, L.BIN_MUL, I_, 1, 0.0),
                 (L.EW_STORE, 0, 0, 0, 0.0), (L.EW_LOAD, 0, S_, 0, 0.0), (L.EW_BINARY, L.BIN_MUL, I_, 0, 0.0),
                 (L.EW_STORE, 0, 0, 1, 0.0)]

    def program(steps, ins, modes, outs):
        arr = (L.EwStep * len(steps))(*[L.EwStep(*st) for st in steps])
        pin = (ctypes.c_void_p * len(ins))(*ins)
        pm = (ctypes.c_int32 * len(ins))(*modes)
        po = (ctypes.c_void_p * len(outs))(*outs)
        return lambda: L.call("endia_hip_ew_program", n, n, len(ins), pin, pm, len(outs), po, len(steps), arr)

    F_, R_ = L.EW_FULL, L.EW_ROW_VECTOR
    cases += [
        ("ew_program  tanh(a*b + bias), 5 steps", program(fwd_steps, [A, B, bias], [F_, F_, R_], [C]), 12.0 * nn, "hbm"),
        ("ew_program  gradients of it, 10 steps, 2 outputs", program(bwd_steps, [A, B, D, E], [F_, F_, F_, F_], [C, bufs[4]]),
         24.0 * nn, "hbm"),
    ]
    rows = []
    ms = ctypes.c_float()
    for _ in range(30):  # bring the clocks up before the first timed kernel
        cases[0][1]()
    for name, fn, work, bound in cases:
        for _ in range(5):
            fn()
        L.call("endia_hip_timer_start", 0)
        for _ in range(reps):
            fn()
        L.call("endia_hip_timer_stop", 0)
        L.call("endia_hip_timer_elapsed_ms", 0, ctypes.byref(ms))
        t = ms.value / reps
        if bound == "mfma":
            ach, peak, unit = work / (t * 1e-3) / 1e12, FP32_MFMA_PEAK_TFLOPS, "TFLOP/s"
        else:
            ach, peak, unit = work / (t * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s"
        rows.append({"kernel": name, "ms": t, "bound": bound, "achieved": ach, "peak": peak, "unit": unit,
                     "frac": ach / peak, "algorithmic_work": work})
    return rows


def gemm_mid_table(reps=100, warm=600):
    """Products with fewer than 256 tiles of 256 x 256 (the shapes of the Hessian-vector and complex configurations), each
    form, timed per launch with a HIP-event pair around every launch (endia_hip_gemm_timing_*) after `warm` launches of
    the same product: the core clock needs a few hundred short launches to reach its sustained value, and a probe that
    starts from an idle chip under-reports short kernels by a fifth."""
    from endia_amd import _lib as L
    L.ensure_init(0)
    rng = np.random.default_rng(0)

    def put(a):
        p = ctypes.c_void_p()
        L.call("endia_hip_malloc", a.nbytes, ctypes.byref(p))
        L.call("endia_hip_memcpy_h2d", p.value, a.ctypes.data, a.nbytes)
        return p.value

    rows = []
    # 4096 x 4096 x 4095 cannot be read 16 bytes at a time and takes the same tiles with 4-byte loads; 4096 x 10 x 4096 is a
    # classifier head, one pass over A (timed over six copies of A in turn, 384 MiB, so that none is served from the last-level cache)
    for (M, N, K) in ((2048, 4096, 4096), (1024, 2048, 2048), (2048, 2048, 1024), (2048, 2048, 2048), (4096, 4096, 4095), (4096, 10, 4096)):
        for form, (ta, tb) in (("NN", (0, 0)), ("NT", (0, 1)), ("TN", (1, 0)), ("TT", (1, 1))):
            if (ta and tb and K != 4095) or (N == 10 and ta):
                continue
            host_a = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
            copies = [put(host_a) for _ in range(6 if N == 10 else 1)]
            B = put(rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32))
            C = put(np.zeros((M, N), np.float32))
            lda, ldb = (M if ta else K), (K if tb else N)
            turn = [0]

            def go():
                A = copies[turn[0] % len(copies)]
                turn[0] += 1
                L.call("endia_hip_sgemm", ta, tb, M, N, K, A, lda, B, ldb, C, N, 1, 0, 0, 0, L.EPI_NONE, L.OP_IDENTITY, None, None, None)

            for _ in range(warm if M * N * K < (1 << 34) else warm // 10):
                go()
            # (a product whose reduction is summed by a second launch is timed as a whole, with one event pair around the loop)
            L.call("endia_hip_timer_start", 1)
            for _ in range(reps):
                go()
            L.call("endia_hip_timer_stop", 1)
            ms = ctypes.c_float()
            L.call("endia_hip_timer_elapsed_ms", 1, ctypes.byref(ms))
            L.call("endia_hip_gemm_timing_begin")
            for _ in range(reps):
                go()
            L.call("endia_hip_sync")
            launches, g_ms, g_flops = ctypes.c_int64(), ctypes.c_double(), ctypes.c_double()
            L.call("endia_hip_gemm_timing_end", ctypes.byref(launches), ctypes.byref(g_ms), ctypes.byref(g_flops))
            us = 1e3 * g_ms.value / launches.value if launches.value else 1e3 * ms.value / reps
            tf = 2.0 * M * N * K / (us * 1e-6) / 1e12
            row = {"kernel": "sgemm %s %d x %d x %d" % (form, M, N, K), "us": us, "us_back_to_back": 1e3 * ms.value / reps,
                   "bound": "mfma", "achieved": tf, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tf / FP32_MFMA_PEAK_TFLOPS}
            if N == 10:  # bound by reading A once
                row.update({"bound": "hbm", "achieved": 4.0 * (M * K + K * N + M * N) / (row["us_back_to_back"] * 1e-6) / 1e9, "peak": HBM_PEAK_GBS,
                            "unit": "GB/s"})
                row["frac"] = row["achieved"] / row["peak"]
            rows.append(row)
            for p in copies + [B, C]:
                L.call("endia_hip_free", p)
    return rows


def gemm_grouped_table(reps=100, warm=400):
    """endia_hip_sgemm_grouped against the same products issued one by one, at the shapes of the second-order
    configuration: x2 / x4 of each shape and form, and the mix a step of the double-backward chain offers."""
    from endia_amd import _lib as L
    L.ensure_init(0)
    rng = np.random.default_rng(0)

    def put(a):
        p = ctypes.c_void_p()
        L.call("endia_hip_malloc", a.nbytes, ctypes.byref(p))
        L.call("endia_hip_memcpy_h2d", p.value, a.ctypes.data, a.nbytes)
        return p.value

    def member(M, N, K, ta, tb):
        return (ta, tb, M, N, K, put(rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)), (M if ta else K),
                put(rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)), (K if tb else N), put(np.zeros((M, N), np.float32)))

    dx, dw = (1024, 2048, 2048), (2048, 2048, 1024)
    cases = [("4 x NN 1024 x 2048 x 2048", [member(*dx, 0, 0) for _ in range(4)]),
             ("4 x NT 1024 x 2048 x 2048", [member(*dx, 0, 1) for _ in range(4)]),
             ("2 x TN 2048 x 2048 x 1024", [member(*dw, 1, 0) for _ in range(2)]),
             ("2 x NN 1024 x 2048 x 2048", [member(*dx, 0, 0) for _ in range(2)]),
             ("NT + NN 1024 x 2048 x 2048 and 2 x TN 2048 x 2048 x 1024", [member(*dx, 0, 1), member(*dx, 0, 0), member(*dw, 1, 0), member(*dw, 1, 0)]),
             ("NN 1024 x 2048 x 2048 and TN 2048 x 2048 x 1024", [member(*dx, 0, 0), member(*dw, 1, 0)]),
             ("NT 1024 x 2048 x 2048 and 3 x TN 2048 x 2048 x 1024", [member(*dx, 0, 1)] + [member(*dw, 1, 0) for _ in range(3)]),
             ("3 x NN 1024 x 2048 x 2048 and TN 2048 x 2048 x 1024", [member(*dx, 0, 0) for _ in range(3)] + [member(*dw, 1, 0)]),
             ("4 x TN 2048 x 2048 x 1024", [member(*dw, 1, 0) for _ in range(4)]),
             ("8 x NN 1024 x 2048 x 2048", [member(*dx, 0, 0) for _ in range(8)])]
    rows = []
    ms = ctypes.c_float()
    for name, members in cases:
        descs = (L.SgemmDesc * len(members))()
        for d, (ta, tb, M, N, K, A, lda, B, ldb, C) in zip(descs, members):
            d.transA, d.transB, d.M, d.N, d.K, d.A, d.lda, d.B, d.ldb, d.C, d.ldc, d.epilogue, d.bias = ta, tb, M, N, K, A, lda, B, ldb, C, N, L.EPI_NONE, None

        def grouped():
            L.call("endia_hip_sgemm_grouped", len(members), descs, -1, None)

        def one_by_one():
            for (ta, tb, M, N, K, A, lda, B, ldb, C) in members:
                L.call("endia_hip_sgemm", ta, tb, M, N, K, A, lda, B, ldb, C, N, 1, 0, 0, 0, L.EPI_NONE, L.OP_IDENTITY, None, None, None)

        flops = sum(2.0 * m[2] * m[3] * m[4] for m in members)
        row = {"products": name}
        for label, fn in (("one_by_one", one_by_one), ("grouped", grouped)):
            for _ in range(warm // len(members)):
                fn()
            L.call("endia_hip_timer_start", 1)
            for _ in range(reps):
                fn()
            L.call("endia_hip_timer_stop", 1)
            L.call("endia_hip_timer_elapsed_ms", 1, ctypes.byref(ms))
            us = 1e3 * ms.value / reps
            row[label + "_us"] = us
            row[label + "_tflops"] = flops / (us * 1e-6) / 1e12
        row["frac"] = row["grouped_tflops"] / FP32_MFMA_PEAK_TFLOPS
        rows.append(row)
        for m in members:
            for ptr in (m[5], m[7], m[9]):
                L.call("endia_hip_free", ptr)
    return rows


def conv_table(reps=10, only=None):
    """conv2d at the benchmark configuration: x [64,64,56,56], w [128,64,3,3], stride 1, pad 1 (fp32, NCHW).
    Algorithmic flops per pass: 2*N*K*C*R*S*P*Q = 29.6 GFLOP for each of forward, data and weight gradient."""
    from endia_amd import _lib as L
    L.ensure_init(0)
    N, C, H, W, K, R, S = 64, 64, 56, 56, 128, 3, 3
    d = L.Conv2dDesc(N, C, H, W, K, R, S, 1, 1, 1, 1, 1, 1, 1)
    P = Q = 56
    rng = np.random.default_rng(5)

    def put(a):
        p = ctypes.c_void_p()
        L.call("endia_hip_malloc", a.nbytes, ctypes.byref(p))
        L.call("endia_hip_memcpy_h2d", p.value, a.ctypes.data, a.nbytes)
        return p.value

    x = put(rng.standard_normal((N, C, H, W)).astype(np.float32))
    w = put((rng.standard_normal((K, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32))
    b = put(rng.standard_normal(K).astype(np.float32))
    dy = put(rng.standard_normal((N, K, P, Q)).astype(np.float32))
    y = put(np.zeros((N, K, P, Q), np.float32))
    dx = put(np.zeros((N, C, H, W), np.float32))
    dw = put(np.zeros((K, C, R, S), np.float32))
    db = put(np.zeros(K, np.float32))
    flop = 2.0 * N * K * C * R * S * P * Q
    ref = ctypes.byref(d)
    cases = [
        ("conv2d_fwd (+bias, relu)", lambda: L.call("endia_hip_conv2d_fwd", ref, x, w, b, y, L.OP_RELU), flop, "mfma"),
        ("conv2d_bwd_data", lambda: L.call("endia_hip_conv2d_bwd_data", ref, dy, w, dx), flop, "mfma"),
        ("conv2d_bwd_weight", lambda: L.call("endia_hip_conv2d_bwd_weight", ref, x, dy, dw), flop, "mfma"),
        ("conv2d_bwd_bias", lambda: L.call("endia_hip_conv2d_bwd_bias", ref, dy, db), 4.0 * N * K * P * Q, "hbm"),
        # all three gradients of relu(conv + bias) from the stored output, dy * [y > 0] formed in the operand loads
        ("conv2d_bwd_relu (dx, dw, db)", lambda: L.call("endia_hip_conv2d_bwd_relu", ref, x, w, y, dy, 0, dx, dw, db), 2 * flop, "mfma"),
        ("conv2d_bwd_relu (dw, db; scalar dy)", lambda: L.call("endia_hip_conv2d_bwd_relu", ref, x, w, y, dy, 1, None, dw, db), flop, "mfma"),
    ]
    # conv3d: x [8,32,16,56,56], w [64,32,3,3,3], stride 1, pad 1: 2*N*K*C*T*R*S*O*P*Q = 44.4 GFLOP per pass
    d3 = L.Conv3dDesc()
    d3.N, d3.C, d3.D, d3.H, d3.W, d3.K, d3.T, d3.R, d3.S = 8, 32, 16, 56, 56, 64, 3, 3, 3
    d3.stride[:], d3.padding[:], d3.dilation[:], d3.groups = [1, 1, 1], [1, 1, 1], [1, 1, 1], 1
    x3 = put(rng.standard_normal((8, 32, 16, 56, 56)).astype(np.float32))
    w3 = put((rng.standard_normal((64, 32, 3, 3, 3)) * np.sqrt(2.0 / (32 * 27))).astype(np.float32))
    y3 = put(np.zeros((8, 64, 16, 56, 56), np.float32))
    dx3 = put(np.zeros((8, 32, 16, 56, 56), np.float32))
    dw3 = put(np.zeros((64, 32, 3, 3, 3), np.float32))
    flop3 = 2.0 * 8 * 64 * 32 * 27 * 16 * 56 * 56
    r3 = ctypes.byref(d3)
    cases += [
        ("conv3d_fwd", lambda: L.call("endia_hip_conv3d_fwd", r3, x3, w3, None, y3, L.OP_IDENTITY), flop3, "mfma"),
        ("conv3d_bwd_data", lambda: L.call("endia_hip_conv3d_bwd_data", r3, y3, w3, dx3), flop3, "mfma"),
        ("conv3d_bwd_weight", lambda: L.call("endia_hip_conv3d_bwd_weight", r3, x3, y3, dw3), flop3, "mfma"),
    ]
    # pooling of the conv output y [64,128,56,56]: 2x2 stride 2 (max, with argmax; average), forward and backward.
    # Algorithmic bytes: input once + output once (+ the int32 argmax for max pooling).
    pd = L.PoolDesc()
    pd.N, pd.C, pd.D, pd.H, pd.W = N, K, 1, P, Q
    pd.kernel[:], pd.stride[:], pd.padding[:], pd.dilation[:] = [1, 2, 2], [1, 2, 2], [0, 0, 0], [1, 1, 1]
    n_in, n_out = N * K * P * Q, N * K * (P // 2) * (Q // 2)
    py, parg = put(np.zeros(n_out, np.float32)), put(np.zeros(n_out, np.int32))
    pref = ctypes.byref(pd)
    cases += [
        ("max_pool2d 2x2/2 fwd", lambda: L.call("endia_hip_pool_fwd", pref, L.POOL_MAX, dy, py, parg), 4.0 * n_in + 8.0 * n_out, "hbm"),
        ("max_pool2d 2x2/2 bwd", lambda: L.call("endia_hip_pool_bwd", pref, L.POOL_MAX, py, parg, y), 4.0 * n_in + 8.0 * n_out, "hbm"),
        ("avg_pool2d 2x2/2 fwd", lambda: L.call("endia_hip_pool_fwd", pref, L.POOL_AVG, dy, py, None), 4.0 * n_in + 4.0 * n_out, "hbm"),
        ("avg_pool2d 2x2/2 bwd", lambda: L.call("endia_hip_pool_bwd", pref, L.POOL_AVG, py, None, y), 4.0 * n_in + 4.0 * n_out, "hbm"),
    ]
    if only:
        cases = [c for c in cases if c[0] in only]
    rows = []
    ms = ctypes.c_float()
    for _ in range(300):  # bring the clocks up before the first timed kernel (a few dozen launches are still on the ramp)
        cases[0][1]()
    for name, fn, work, bound in cases:
        for _ in range(20):
            fn()
        L.call("endia_hip_timer_start", 0)
        for _ in range(reps):
            fn()
        L.call("endia_hip_timer_stop", 0)
        L.call("endia_hip_timer_elapsed_ms", 0, ctypes.byref(ms))
        t = ms.value / reps
        if bound == "mfma":
            ach, peak, unit = work / (t * 1e-3) / 1e12, FP32_MFMA_PEAK_TFLOPS, "TFLOP/s"
        else:
            ach, peak, unit = work / (t * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s"
        rows.append({"kernel": name, "ms": t, "bound": bound, "achieved": ach, "peak": peak, "unit": unit,
                     "frac": ach / peak, "algorithmic_work": work})
    return rows


def conv_step(nd, steps, warmup, x_grad):
    """One training step of the convolution configuration through the public API: loss = mean(relu(conv2d(x, w,
    b))), backward to w and b (and to x when x_grad). Algorithmic work 2*N*K*C*R*S*P*Q = 29.6 GFLOP per
    convolution-shaped pass: forward + weight gradient (+ data gradient)."""
    rng = np.random.default_rng(5)
    N, C, H, W, K, R, S = 64, 64, 56, 56, 128, 3, 3
    x = nd.array(rng.standard_normal((N, C, H, W)).astype(np.float32), requires_grad=x_grad)
    w = nd.array((rng.standard_normal((K, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32), requires_grad=True)
    b = nd.array(rng.standard_normal(K).astype(np.float32), requires_grad=True)

    def step():
        loss = nd.mean(nd.conv2d(x, w, b, stride=1, padding=1, act="relu"))
        loss.backward()
        loss.zero_grad()
        return loss

    for _ in range(max(warmup, 3)):
        step()
    nd.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    nd.synchronize()
    dt = (time.perf_counter() - t0) / steps
    flops = (3 if x_grad else 2) * 2.0 * N * K * C * R * S * H * W
    return {"passes": "forward + weight gradient + bias gradient" + (" + data gradient" if x_grad else ""),
            "ms_per_step": dt * 1e3, "steps_per_s": 1.0 / dt, "algorithmic_tflops": flops / dt / 1e12,
            "frac_of_fp32_mfma_peak": flops / dt / 1e12 / FP32_MFMA_PEAK_TFLOPS}


def gemm_roofline(L, elapsed_s, algorithmic_flops_total, kernel):
    """Close a gemm_timing window and price the MFMA GEMM launches inside it: achieved = algorithmic flops /
    summed HIP-event kernel time of those launches (events recorded on the library's stream)."""
    launches, g_ms, g_flops = ctypes.c_int64(), ctypes.c_double(), ctypes.c_double()
    L.call("endia_hip_gemm_timing_end", ctypes.byref(launches), ctypes.byref(g_ms), ctypes.byref(g_flops))
    if not launches.value:
        return None
    achieved = algorithmic_flops_total / (g_ms.value * 1e-3) / 1e12
    return {"bound": "mfma", "kernel": kernel, "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / FP32_MFMA_PEAK_TFLOPS, "traffic": None, "launches": launches.value,
            "avg_launch_ms": g_ms.value / launches.value, "executed_tflops": g_flops.value / (g_ms.value * 1e-3) / 1e12,
            "gemm_share_of_step": g_ms.value / (1e3 * elapsed_s)}


def run_hvp(nd, steps, warmup):
    """Hessian-vector product by create_graph=True double backward: 4 Linear layers 2048 wide, sin
    between, batch 1024, loss = sum(out^2), v ~ N(0,1) per parameter. Algorithmic GEMM work of the
    reference's decomposition: 31 products of 2*1024*2048^2 flops (4 forward, 7 first backward, 20 second)."""
    rng = np.random.default_rng(3)
    B, Wd, Ly = 1024, 2048, 4
    mlp = nd.nn.MLP([Wd] * (Ly + 1), compute_backward=True, activation="sin", fused=True)
    vs = []
    for i in range(Ly):
        mlp.weights[i] = nd.array((rng.standard_normal((Wd, Wd)) / np.sqrt(Wd)).astype(np.float32), requires_grad=True)
        mlp.biases[i] = nd.array((rng.standard_normal(Wd) / np.sqrt(Wd)).astype(np.float32), requires_grad=True)
        vs += [nd.array(rng.standard_normal((Wd, Wd)).astype(np.float32)), nd.array(rng.standard_normal((1, Wd)).astype(np.float32))]
    x = nd.array(rng.standard_normal((B, Wd)).astype(np.float32))

    def step():
        out = mlp.forward(x)
        loss = nd.sum(out * out)
        loss.backward(create_graph=True)
        firsts = [p.grad() for p in mlp.params()]
        # the second reverse pass starts from the first-order gradients with v as their cotangents: the gradient of
        # <gradients, v> without forming the eight dot products
        hv = nd.grad(outs=firsts, inputs=mlp.params(), grad_outs=[nd.reshape(v, f.shape()) for v, f in zip(vs, firsts)])
        loss.zero_grad()
        return hv

    from endia_amd import _lib as L
    for _ in range(warmup):
        step()
    nd.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        hv = step()
    nd.synchronize()
    dt = (time.perf_counter() - t0) / steps
    # a second pass with an event pair around every GEMM launch prices the kernel; the pairs cost a few
    # microseconds each, which is why they stay out of the pass that `value` is taken from
    L.call("endia_hip_gemm_timing_begin")
    t0 = time.perf_counter()
    for _ in range(steps):
        hv = step()
    nd.synchronize()
    elapsed = time.perf_counter() - t0
    flops = 31 * 2.0 * B * Wd * Wd
    roof = gemm_roofline(L, elapsed, flops * steps, "the 1024 x 2048 x 2048 and 2048 x 2048 x 1024 products: sgemm_lone_grouped_kernel<4, 2> (256x128x32 tiles, "
                         "independent products of the backward passes sharing a launch, one tile per CU) and sgemm_mfma_kernel<F = 1> (64x64x32 "
                         "tiles, K split inside the launch) for those that find no company")
    return {"metric": "Hessian-vector products/s, 4 x 2048 sin MLP, batch 1024 (double backward)", "value": 1.0 / dt,
            "unit": "HVP/s", "n_gpus": 1, "ms_per_step": dt * 1e3, "higher_is_better": True, "vs_baseline": None,
            "algorithmic_gemm_tflops": flops / dt / 1e12,
            "frac_of_fp32_mfma_peak": flops / dt / 1e12 / FP32_MFMA_PEAK_TFLOPS, "steps": steps, "warmup": warmup,
            "dtype": "f32", "data": "synthetic",
            "config": {"workload": "hvp: 4 x Linear(2048->2048)+bias, sin, loss sum(out^2), batch 1024, H v by double backward"},
            "roofline": roof}


def run_complex(nd, steps, warmup, algo):
    """complex64 MLP: 4 complex Linear layers 2048 -> 2048 (identity activation), batch 2048, loss =
    sum |out|^2, backward with the reference's rule (no conjugation). 11 complex GEMMs of 8*2048^3 flops."""
    rng = np.random.default_rng(4)
    n, Ly = 2048, 4
    nd.set_complex_matmul_algorithm(algo)
    Ws = [nd.array(((rng.standard_normal((n, n)) + 1j * rng.standard_normal((n, n))) / np.sqrt(2 * n)).astype(np.complex64),
                   requires_grad=True) for _ in range(Ly)]
    z = nd.array((rng.standard_normal((n, n)) + 1j * rng.standard_normal((n, n))).astype(np.complex64))

    def step(wirtinger=False):
        h = z
        for W in Ws:
            h = nd.matmul(h, W, vjp_rule="wirtinger" if wirtinger else "reference")
        loss = nd.sum(nd.square(nd.abs(h)))
        loss.backward()
        loss.zero_grad()
        return loss

    from endia_amd import _lib as L
    # `value` is taken under the library's default, the reference's coded rule (no conjugation, matmul_op.mojo:278-283);
    # the Wirtinger rule (g B^H, A^H g: the gradient of the real loss, which the float64 checks of this configuration
    # compare with torch's complex128 autograd) costs the same launches with other conjugation flags and is timed beside it
    dt, _ = _time_steps(nd, lambda: step(False), steps, warmup)
    dt_wirtinger, _ = _time_steps(nd, lambda: step(True), steps, warmup)
    L.call("endia_hip_gemm_timing_begin")  # second pass, with an event pair around every GEMM launch
    t0 = time.perf_counter()
    for _ in range(steps):
        step(False)
    nd.synchronize()
    elapsed = time.perf_counter() - t0
    flops = 11 * 8.0 * n * n * n  # algorithmic: 8 real flops per complex multiply-add, whichever algorithm runs
    roof = gemm_roofline(L, elapsed, flops * steps, (
        "sgemm_mfma_kernel<F = 2> (128x128x32 tiles): three real 2048^3 products per complex product in one batched launch" if algo == "3m"
        else "sgemm_lone_kernel<FM = 4, FN = 2> (256x128x32 tiles, one work-group per CU): one real 2048 x 4096 x 4096 product "
             "per complex product (B embedded as a 2K x 2N real matrix)"))
    return {"metric": "fwd+bwd steps/s, complex64 MLP 4 x 2048, batch 2048, algorithm " + algo, "value": 1.0 / dt,
            "unit": "steps/s", "n_gpus": 1, "ms_per_step": dt * 1e3, "higher_is_better": True, "vs_baseline": None,
            "algorithmic_gemm_tflops": flops / dt / 1e12,
            "frac_of_fp32_mfma_peak": flops / dt / 1e12 / FP32_MFMA_PEAK_TFLOPS, "steps": steps, "warmup": warmup,
            "gradient_rule": "reference (dA = g B^T, dB = A^T g, no conjugation: matmul_op.mojo:278-283)",
            "wirtinger_rule": {"rule": "dA = g B^H, dB = A^H g (vjp_rule='wirtinger')", "ms_per_step": dt_wirtinger * 1e3,
                               "steps_per_s": 1.0 / dt_wirtinger, "algorithmic_gemm_tflops": flops / dt_wirtinger / 1e12},
            "dtype": "c64 (f32 pairs)", "data": "synthetic",
            "config": {"workload": "complex_mlp: 4 x complex Linear(2048->2048), identity, loss sum|out|^2, batch 2048, " + algo},
            "roofline": roof}


def _time_steps(nd, step, steps, warmup):
    for _ in range(warmup):
        step()
    nd.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    nd.synchronize()
    return (time.perf_counter() - t0) / steps, out


def run_sine(nd, steps, warmup, optimizer="sgd", eager=False, per_layer=False):
    """Benchmark configuration 1, the reference's own benchmark model (benchmarks/mlp_benchmarks/mlp_imp.mojo:35-75), as
    a HIP-graph replay of the eager step. `value` is taken with the reference script's call shape, mse(mlp.forward(x),
    y); the same step with forward and loss behind one method (MLP.mse_loss, no counterpart in the reference) is
    timed beside it. Launch-latency bound: no roofline claim."""
    w = [1, 32, 64, 128, 128, 128, 64, 32, 1]
    kn = sum(w[i] * w[i + 1] for i in range(8))
    flops = 2.0 * 128 * (3 * kn - w[0] * w[1])
    res = {}
    for fused_loss in (False, True):
        mlp, opt, x, y = build_sine_mlp(nd, optimizer=optimizer, per_layer=per_layer)
        step = lambda: train_step(nd, mlp, opt, x, y, fused_loss)
        for _ in range(max(warmup, 3)):
            step()
        nd.synchronize()
        captured = None if eager else nd.capture(step)
        dt, loss = _time_steps(nd, captured.replay if captured else step, steps, 20)
        res[fused_loss] = (dt, float(loss.item()))
        if captured:
            captured.close()
    dt, final_loss = res[False]
    return {"metric": "fwd+bwd+%s train steps/s, sine-fit MLP" % ("SGD" if optimizer == "sgd" else "Adam"),
            "value": 1.0 / dt, "unit": "steps/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": dt * 1e3,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "sine_mlp: widths 1-32-64-128-128-128-64-32-1, relu, MSE, %s 1e-3, batch 128, fp32"
                                   % ("SGD" if optimizer == "sgd" else "Adam"), "batch": 128, "optimizer": optimizer,
                       "execution": ("host-issued launches" if eager else "HIP graph replay of the eager step") +
                                    ("; one fused op per layer" if per_layer else "; nn.MLP(fused='model')") +
                                    "; loss = mse(mlp.forward(x), y) as in the reference's script"},
            "final_loss": final_loss, "gemm_tflops_whole_step": flops / dt / 1e12,
            "roofline": {"bound": "launch latency", "kernel": None, "achieved": None, "peak": None, "frac": None,
                         "note": "a step is a handful of dependent launches of 4-20 us; no roofline claim"},
            "fused_loss_call": {"call": "MLP.mse_loss(x, y): forward, loss and the cotangents of all layers in one launch",
                                "value": 1.0 / res[True][0], "ms_per_step": res[True][0] * 1e3, "final_loss": res[True][1]}}


def run_wide(nd, steps, warmup, fused_backward=False):
    from endia_amd import _lib as L
    mlp, opt, x, y = build_wide_mlp(nd, fused_backward=fused_backward)
    width, layers, batch = 4096, 8, 4096
    gemm_flops_step = (layers + layers + layers - 1) * 2.0 * batch * width * width
    for _ in range(warmup):
        train_step(nd, mlp, opt, x, y)
    nd.synchronize()
    L.call("endia_hip_gemm_timing_begin")
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = train_step(nd, mlp, opt, x, y)
    nd.synchronize()
    elapsed = time.perf_counter() - t0
    launches, g_ms, g_flops = ctypes.c_int64(), ctypes.c_double(), ctypes.c_double()
    L.call("endia_hip_gemm_timing_end", ctypes.byref(launches), ctypes.byref(g_ms), ctypes.byref(g_flops))
    ms_per_step = 1e3 * elapsed / steps
    out = {
        "metric": "fwd+bwd train steps/s + MFMA util %, 8-layer 4096-wide fp32 MLP, batch 4096",
        "value": steps / elapsed, "unit": "steps/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "wide_mlp: 8 x Linear(4096->4096)+bias, tanh, MSE, Adam, batch 4096, fp32",
                   "batch": batch, "width": width, "layers": layers, "optimizer": "adam"},
        "final_loss": float(loss.item()),
        "gemm_tflops_whole_step": gemm_flops_step / (ms_per_step * 1e-3) / 1e12,
    }
    if launches.value:
        avg_ms = g_ms.value / launches.value
        flops_per_launch = g_flops.value / launches.value
        achieved = flops_per_launch / (avg_ms * 1e-3) / 1e12
        out["roofline"] = {
            "bound": "mfma", "kernel": "sgemm_lone_kernel<FM = 4, FN = 4> (fp32 v_mfma_f32_32x32x2, 256x256x32 tiles, one work-group per CU)",
            "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / FP32_MFMA_PEAK_TFLOPS,
            "traffic": GEMM_TRAFFIC_BYTES,
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, see profiles/kernels_wide_mlp_counters.md",
            "algorithmic_bytes": 3 * 4096 * 4096 * 4,
            "launches": launches.value, "avg_launch_ms": avg_ms,
            "flops_per_launch": flops_per_launch, "gemm_share_of_step": g_ms.value / (1e3 * elapsed),
        }
        out["mfma_util_pct"] = 100.0 * achieved / FP32_MFMA_PEAK_TFLOPS
    return out


def run_conv(nd, steps, warmup):
    """Benchmark configuration 5 as a training step through the public API (forward with fused ReLU, mean loss, weight
    and bias gradients; the same with the data gradient beside it). `roofline` prices the forward entry point, the
    longest of the step's launches, timed alone with HIP events on the library's stream."""
    rows = conv_table(max(min(steps, 200), 3), only=("conv2d_fwd (+bias, relu)", "conv2d_bwd_data", "conv2d_bwd_weight"))
    step, with_dx = conv_step(nd, steps, warmup, False), conv_step(nd, steps, warmup, True)
    fwd = rows[0]
    return {"metric": "conv2d fwd + VJPs train steps/s, batch 64, 64->128 channels, 3x3, stride 1, pad 1, 56x56, fp32",
            "value": step["steps_per_s"], "unit": "steps/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": step["ms_per_step"], "higher_is_better": True, "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "conv2d: x [64,64,56,56], w [128,64,3,3], stride 1, pad 1, relu, mean loss; forward + dw + db"},
            "algorithmic_tflops": step["algorithmic_tflops"], "frac_of_fp32_mfma_peak": step["frac_of_fp32_mfma_peak"],
            "with_data_gradient": with_dx, "entry_points": rows,
            "roofline": {"bound": "mfma", "kernel": "conv_direct3x3_kernel (forward; weight packing included)", "achieved": fwd["achieved"],
                         "peak": fwd["peak"], "unit": fwd["unit"], "frac": fwd["frac"], "traffic": None, "avg_launch_ms": fwd["ms"]}}


def _brief(out):
    """What the headline line keeps of another configuration's result."""
    keep = ("value", "unit", "ms_per_step", "steps", "warmup", "dtype", "algorithmic_gemm_tflops", "algorithmic_tflops",
            "frac_of_fp32_mfma_peak", "fused_loss_call", "wirtinger_rule", "with_data_gradient", "gradient_rule", "final_loss")
    b = {"workload": out["config"]["workload"]}
    b.update({k: out[k] for k in keep if k in out})
    r = out.get("roofline") or {}
    b["roofline"] = {k: r.get(k) for k in ("bound", "kernel", "achieved", "peak", "unit", "frac", "launches", "avg_launch_ms") if k in r}
    c = out.get("cpu_baseline")
    if c:
        b["cpu_baseline"] = {k: c[k] for k in ("value", "unit", "cores", "kind", "sample") if k in c}
    return b


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="wide_mlp", choices=["wide_mlp", "sine_mlp", "kernels", "gemm_mid", "conv2d", "conv2d_kernels", "hvp", "complex_mlp", "complex_mlp_3m"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true", help="wide_mlp: leave the other four configurations out of the line")
    ap.add_argument("--adam-in-backward", action="store_true", help="wide_mlp: optim.Adam(fused_backward=True), the update of a layer "
                    "issued by backward() right behind that layer's gradients")
    ap.add_argument("--eager", action="store_true", help="sine_mlp: issue every kernel from the host instead of replaying a graph")
    ap.add_argument("--per-layer", action="store_true", help="sine_mlp: one fused op per layer instead of the whole-model op")
    ap.add_argument("--optimizer", default="sgd", choices=["sgd", "adam"], help="sine_mlp: SGD (the benchmark configuration) or Adam (the reference script's)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives, no sharding); --gpus %d is not supported. "
                 "`value` is one GPU's throughput." % args.gpus)

    import endia_amd as nd
    from endia_amd import _lib as L
    L.ensure_init(0)
    dev_name, cus, mhz = L.device_info()
    cpu = not args.no_cpu_baseline

    if args.workload == "hvp":
        # (short runs measure the clock ramp: 40 products after 3 read 2.24 ms where 200 after 20 read 2.20)
        out = run_hvp(nd, 200 if args.steps == 20 else args.steps, max(args.warmup, 20) if args.steps == 20 else args.warmup)
        if cpu:
            out["cpu_baseline"] = cpu_baseline_hvp()
    elif args.workload.startswith("complex_mlp"):
        out = run_complex(nd, args.steps, args.warmup, "3m" if args.workload.endswith("3m") else "4m")
        if cpu:
            out["cpu_baseline"] = cpu_baseline_complex()
    elif args.workload == "conv2d":
        # (short runs measure the clock ramp: 100 steps of half a millisecond read 0.511 ms where 1000 read 0.503)
        out = run_conv(nd, 1000 if args.steps == 20 else max(args.steps, 1), max(args.warmup, 50 if args.steps == 20 else 10))
        if cpu:
            out["cpu_baseline"] = cpu_baseline_conv()
    elif args.workload == "conv2d_kernels":
        out = {"metric": "conv2d / conv3d / pooling entry points, fp32", "device": dev_name, "reps": max(args.steps, 1),
               "kernels": conv_table(max(args.steps, 1))}
    elif args.workload == "gemm_mid":
        out = {"metric": "fp32 GEMM launches of the mid-size products, sustained clock", "device": dev_name,
               "reps": max(args.steps, 1), "kernels": gemm_mid_table(max(args.steps, 1)),
               "grouped": gemm_grouped_table(max(args.steps, 1))}
    elif args.workload == "kernels":
        out = {"metric": "per-kernel roofline at the wide-MLP shape (4096 x 4096 operands)", "device": dev_name,
               "reps": max(args.steps, 1), "kernels": kernel_table(max(args.steps, 1))}
    elif args.workload == "sine_mlp":
        out = run_sine(nd, max(args.steps, 200), args.warmup, args.optimizer, args.eager, args.per_layer)
        if cpu:
            out["cpu_baseline"] = cpu_baseline_sine(optimizer=args.optimizer)
    else:
        out = run_wide(nd, args.steps, args.warmup, args.adam_in_backward)
        if args.adam_in_backward:
            out["config"]["optimizer"] = "adam, applied by backward() layer by layer (optim.Adam(fused_backward=True))"
        out["device"] = dev_name
        if cpu:
            out["cpu_baseline"] = cpu_baseline_wide()
        if not args.headline_only:
            # the other four benchmark configurations, each bounded to a second or two of GPU time and a few seconds of
            # CPU baseline: the same functions that `--workload sine_mlp | hvp | complex_mlp | conv2d` run alone
            others = []
            for name, fn, base in (
                    ("sine_mlp", lambda: run_sine(nd, 2000, 3), lambda: cpu_baseline_sine(steps=200)),
                    ("hvp", lambda: run_hvp(nd, 200, 20), cpu_baseline_hvp),
                    ("complex_mlp", lambda: run_complex(nd, 20, 3, "4m"), lambda: cpu_baseline_complex(rows=256)),
                    ("conv2d", lambda: run_conv(nd, 1000, 50), lambda: cpu_baseline_conv(n_img=8))):
                r = fn()
                if cpu:
                    r["cpu_baseline"] = base()
                others.append(_brief(r))
                nd.synchronize()
            out["configs"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
