"""Benchmark of the matrix-multiply forward+backward path on one MI355X.

One step = MatrixMultiplyOperation forward (C = A.B) plus backward (dA = dC.B^T, dB = A^T.dC) on
device-resident square double matrices, N = 4096 by default: three launches of the MFMA product
kernel, 6 N^3 floating-point operations.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--n N] [--dtype f64|f32] [--no-cpu]
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f64": 78.6, "f32": 157.3}  # MI355X dense matrix-core peaks
METRIC = "fp64/fp32 matmul fwd+bwd TFLOP/s (% MFMA peak); MLP train steps/sec"


def gpu_leg(n, dtype_name, steps, warmup):
    from parallelreverseautodiff_amd import _lib, seeded
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer

    lib = _lib.load()
    CudaBlas.Instance.DeviceId = int(os.environ.get("LOCAL_RANK", "0"))
    CudaBlas.Instance.Initialize()
    dtype = np.float64 if dtype_name == "f64" else np.float32
    A = seeded.uniform(seeded.DEFAULT_SEED, 1, (n, n), -1, 1, dtype)
    B = seeded.uniform(seeded.DEFAULT_SEED, 2, (n, n), -1, 1, dtype)
    dC = seeded.normal(seeded.DEFAULT_SEED, 3, (n, n), 1.0, dtype)
    bufs = {k: DeviceBuffer.alloc(dtype, n, n) for k in ("A", "B", "C", "dC", "dA", "dB")}
    bufs["A"].upload(A); bufs["B"].upload(B); bufs["dC"].upload(dC)
    h = {k: v.handle for k, v in bufs.items()}

    def step():
        check(lib.prad_matmul_fwd(h["A"], h["B"], h["C"]))
        check(lib.prad_matmul_bwd(h["dC"], h["A"], h["B"], h["dA"], h["dB"], 0, 0))

    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.prad_event_create(ctypes.byref(e0)))
    check(lib.prad_event_create(ctypes.byref(e1)))
    for _ in range(warmup):
        step()
    check(lib.prad_stream_sync())
    t0 = time.perf_counter()
    check(lib.prad_event_record(e0))  # events are recorded on the stream the kernels run on
    for _ in range(steps):
        step()
    check(lib.prad_event_record(e1))
    check(lib.prad_stream_sync())
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms = ctypes.c_float()
    check(lib.prad_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
    # spot check of the timed buffers: a few entries against exactly rounded dot products
    import math
    C = bufs["C"].download()
    rng = np.random.default_rng(0)
    worst = 0.0
    for _ in range(8):
        i, j = int(rng.integers(n)), int(rng.integers(n))
        exact = math.fsum(A[i, :].astype(np.float64) * B[:, j].astype(np.float64))
        worst = max(worst, abs(float(C[i, j]) - exact) / math.sqrt(n / 3.0))
    tol = 1e-12 if dtype_name == "f64" else 1e-5
    if not worst <= tol:
        raise SystemExit("benchmark output failed its spot check: %.3e" % worst)
    return float(ms.value), wall_ms, worst


def bandwidth_leg(n_elems, dtype_name, steps, warmup, only=None):
    """Times each bandwidth kernel on n_elems elements (default 64 Mi: beyond the 256 MB last-level cache).
    Algorithmic bytes per element, s = element size: activation backward 3s (read src, dy; write dx),
    Hadamard backward 5s, accumulate 3s, copy 2s, clip 3s (read for statistics; read + write), Adam 7s,
    add 3s, add three 4s, transpose 2s, layer normalization 2s forward / 3s backward (rows of 4096)."""
    from parallelreverseautodiff_amd import _lib, seeded
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer

    lib = _lib.load()
    CudaBlas.Instance.DeviceId = 0
    CudaBlas.Instance.Initialize()
    dtype = np.float64 if dtype_name == "f64" else np.float32
    es = np.dtype(dtype).itemsize
    rows, cols = n_elems // 4096, 4096
    n = rows * cols
    host = [seeded.normal(7, t, (rows, cols), 1.0, dtype) for t in range(3)]
    host[2] = np.abs(host[2])
    b = [DeviceBuffer.alloc(dtype, rows, cols) for _ in range(5)]
    for i in range(3):
        b[i].upload(host[i])
    h = [x.handle for x in b]
    tr = DeviceBuffer.alloc(dtype, cols, rows)                      # transpose target
    mean, std = DeviceBuffer.alloc(dtype, 1, rows), DeviceBuffer.alloc(dtype, 1, rows)
    cases = {
        "copy": (2, lambda: lib.prad_buf_copy(h[3], h[0])),
        "leakyrelu_bwd": (3, lambda: lib.prad_act_bwd(_lib.ACT_LEAKYRELU, h[0], h[1], h[3], 0.01)),
        "sigmoid_bwd": (3, lambda: lib.prad_act_bwd(_lib.ACT_SIGMOID, h[0], h[1], h[3], 0.0)),
        "tanh_bwd": (3, lambda: lib.prad_act_bwd(_lib.ACT_TANH, h[0], h[1], h[3], 0.0)),
        "gelu_bwd": (3, lambda: lib.prad_act_bwd(_lib.ACT_GELU, h[0], h[1], h[3], 0.0)),
        "hadamard_bwd": (5, lambda: lib.prad_hadamard_bwd(h[0], h[1], h[2], h[3], h[4])),
        "accumulate": (3, lambda: lib.prad_accumulate(h[3], h[1])),
        "clip": (3, lambda: lib.prad_clip(h[1], 4.0, 1e-16 if dtype_name == "f64" else 1e-8)),
        "adam": (7, lambda: lib.prad_adam(h[0], h[3], h[2], h[1], 1e-3, 0.9, 0.999, 1e-8, 1.0)),
        "amplified_sigmoid_bwd": (3, lambda: lib.prad_act_bwd(_lib.ACT_AMPLIFIED_SIGMOID, h[0], h[1], h[3], 0.0)),
        "add": (3, lambda: lib.prad_add(h[0], h[1], h[3])),
        "add_three": (4, lambda: lib.prad_add_three(h[0], h[1], h[2], h[3])),
        "transpose": (2, lambda: lib.prad_transpose(h[0], tr.handle)),
        "layernorm_fwd": (2, lambda: lib.prad_layernorm_fwd(h[0], h[3], mean.handle, std.handle)),
        "layernorm_bwd": (3, lambda: lib.prad_layernorm_bwd(h[0], mean.handle, std.handle, h[1], h[3])),
    }
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.prad_event_create(ctypes.byref(e0)))
    check(lib.prad_event_create(ctypes.byref(e1)))
    out = {}
    for name, (factor, fn) in cases.items():
        if only and name not in only:
            continue
        for _ in range(warmup):
            check(fn())
        check(lib.prad_stream_sync())
        check(lib.prad_event_record(e0))
        for _ in range(steps):
            check(fn())
        check(lib.prad_event_record(e1))
        ms = ctypes.c_float()
        check(lib.prad_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        per = ms.value / steps
        gbs = factor * es * n / (per * 1e-3) / 1e9
        out[name] = {"ms": per, "GB/s": gbs, "frac_of_8TBps": gbs / 8000.0, "bytes_per_element": factor * es}
    return out, n


def matmul_sum_leg(dtype_name, steps, warmup):
    """configs[2]: MatrixMultiplyAndSum, A 512x768, 32 slices of 768x512, forward (MFMA, 12.88 GFLOP) and the
    reference's backward (data movement: read A and B once, write dA and dB once = 103.8 MB in float)."""
    from parallelreverseautodiff_amd import _lib, seeded
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer

    lib = _lib.load()
    CudaBlas.Instance.DeviceId = 0
    CudaBlas.Instance.Initialize()
    dtype = np.float64 if dtype_name == "f64" else np.float32
    M, K, P = 512, 768, 32
    A = DeviceBuffer.alloc(dtype, M, K); B = DeviceBuffer.alloc(dtype, K, M, depth=P)
    out = DeviceBuffer.alloc(dtype, 1, P); dOut = DeviceBuffer.alloc(dtype, 1, P)
    dA = DeviceBuffer.alloc(dtype, M, K); dB = DeviceBuffer.alloc(dtype, K, M, depth=P)
    A.upload(seeded.normal(seeded.DEFAULT_SEED, 1, (M, K), 0.02, dtype))
    B.upload(seeded.normal(seeded.DEFAULT_SEED, 2, (P, K, M), 0.02, dtype))
    dOut.upload(seeded.normal(seeded.DEFAULT_SEED, 3, (1, P), 1.0, dtype))
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.prad_event_create(ctypes.byref(e0)))
    check(lib.prad_event_create(ctypes.byref(e1)))

    def timed(fn):
        for _ in range(warmup):
            check(fn())
        check(lib.prad_stream_sync())
        check(lib.prad_event_record(e0))
        for _ in range(steps):
            check(fn())
        check(lib.prad_event_record(e1))
        ms = ctypes.c_float()
        check(lib.prad_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        return ms.value / steps

    fwd_ms = timed(lambda: lib.prad_matmul_sum_fwd(A.handle, B.handle, out.handle))
    bwd_ms = timed(lambda: lib.prad_matmul_sum_bwd(A.handle, B.handle, dOut.handle, dA.handle, dB.handle))
    es = np.dtype(dtype).itemsize
    flops = 2.0 * M * K * M * P
    bytes_bwd = 2.0 * (M * K + P * K * M) * es
    # The same configuration read as "32 independent products summed into one output plus a broadcast
    # bias": C = sum_q A[q].B[q] + bias, and its backward (dA[q], dB[q], dbias): 12.88 + 25.77 GFLOP.
    A3 = DeviceBuffer.alloc(dtype, M, K, depth=P); dA3 = DeviceBuffer.alloc(dtype, M, K, depth=P)
    A3.upload(seeded.normal(seeded.DEFAULT_SEED, 4, (P, M, K), 0.02, dtype))
    bias = DeviceBuffer.alloc(dtype, 1, M); dbias = DeviceBuffer.alloc(dtype, 1, M)
    C = DeviceBuffer.alloc(dtype, M, M); dC = DeviceBuffer.alloc(dtype, M, M)
    dC.upload(seeded.normal(seeded.DEFAULT_SEED, 5, (M, M), 1.0, dtype))
    bs_fwd_ms = timed(lambda: lib.prad_matmul_batch_sum_fwd(A3.handle, B.handle, bias.handle, C.handle))
    bs_bwd_ms = timed(lambda: lib.prad_matmul_batch_sum_bwd(dC.handle, A3.handle, B.handle, dA3.handle, dB.handle, dbias.handle))
    batch_sum = {"fwd_ms": bs_fwd_ms, "fwd_TFLOPs": flops / (bs_fwd_ms * 1e-3) / 1e12,
                 "fwd_frac_of_mfma_peak": flops / (bs_fwd_ms * 1e-3) / 1e12 / PEAK_TFLOPS[dtype_name],
                 "bwd_ms": bs_bwd_ms, "bwd_TFLOPs": 2 * flops / (bs_bwd_ms * 1e-3) / 1e12,
                 "bwd_frac_of_mfma_peak": 2 * flops / (bs_bwd_ms * 1e-3) / 1e12 / PEAK_TFLOPS[dtype_name]}
    return {"batch_sum_with_bias": batch_sum, "fwd_ms": fwd_ms, "fwd_TFLOPs": flops / (fwd_ms * 1e-3) / 1e12, "fwd_frac_of_mfma_peak": flops / (fwd_ms * 1e-3) / 1e12 / PEAK_TFLOPS[dtype_name],
            "bwd_ms": bwd_ms, "bwd_GBps": bytes_bwd / (bwd_ms * 1e-3) / 1e9, "bwd_frac_of_8TBps": bytes_bwd / (bwd_ms * 1e-3) / 8e12,
            "fwd_flop": flops, "bwd_bytes": bytes_bwd}


def lstm_leg(dtype_name, steps, warmup, with_cpu):
    """configs[3]: one LSTM layer, input 256, hidden 512, batch 128, 64 time steps, fused 4-gate weight,
    MSE on the hidden states, backprop through time, clip, Adam."""
    from parallelreverseautodiff_amd import _lib
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.lstm import LSTMLayer

    lib = _lib.load()
    CudaBlas.Instance.DeviceId = 0
    CudaBlas.Instance.Initialize()
    dtype = np.float64 if dtype_name == "f64" else np.float32
    layer = LSTMLayer(dtype=dtype)
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.prad_event_create(ctypes.byref(e0)))
    check(lib.prad_event_create(ctypes.byref(e1)))

    def timed(fn):
        for _ in range(warmup):
            fn()
        check(lib.prad_stream_sync())
        check(lib.prad_event_record(e0))
        for _ in range(steps):
            fn()
        check(lib.prad_event_record(e1))
        check(lib.prad_stream_sync())
        ms = ctypes.c_float()
        check(lib.prad_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        return ms.value / steps

    eager_ms = timed(layer.step)
    layer.record()
    rec_ms = timed(layer.replay)
    layer.release()
    flops = layer.flops_per_step()
    out = {"eager_ms_per_step": eager_ms, "recorded_ms_per_step": rec_ms, "flop_per_step": flops,
           "TFLOPs": flops / (rec_ms * 1e-3) / 1e12, "loss_after": float(layer.loss.download()[0, 0])}
    if with_cpu:
        from oracle import compose, oracle
        threads = min(16, oracle.hardware_threads() or 1)
        I, H, B, T = layer.input_dim, layer.hidden, layer.batch, layer.steps
        t0 = time.perf_counter()
        compose.lstm_forward_backward(layer.host_W, np.zeros((1, 4 * H), dtype), layer.host_X, layer.host_Y, I, H, B, T, threads=threads)
        secs = time.perf_counter() - t0
        out["cpu"] = {"steps_per_s": 1.0 / secs, "ms_per_step": secs * 1e3, "cores": threads, "steps_timed": 1, "kind": "port",
                      "note": "forward + backward only (no clip/Adam), node-by-node composition of the oracle's operations"}
    return out


def swin_leg(dtype_name, steps, warmup, with_cpu):
    """configs[4]: Swin-style windowed self-attention block, batch 16, 56x56 tokens in 7x7 windows, embed 96, 3 heads,
    MLP x4 with GELU (GELUOperation's own derivative), MSE, full backward, clip, Adam."""
    from parallelreverseautodiff_amd import _lib
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.swin import SwinBlock

    lib = _lib.load()
    CudaBlas.Instance.DeviceId = 0
    CudaBlas.Instance.Initialize()
    dtype = np.float64 if dtype_name == "f64" else np.float32
    blk = SwinBlock(dtype=dtype)
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.prad_event_create(ctypes.byref(e0)))
    check(lib.prad_event_create(ctypes.byref(e1)))

    def timed(fn):
        for _ in range(warmup):
            fn()
        check(lib.prad_stream_sync())
        check(lib.prad_event_record(e0))
        for _ in range(steps):
            fn()
        check(lib.prad_event_record(e1))
        check(lib.prad_stream_sync())
        ms = ctypes.c_float()
        check(lib.prad_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        return ms.value / steps

    eager_ms = timed(blk.step)
    blk.record()
    rec_ms = timed(blk.replay)
    blk.release()
    flops = blk.flops_per_step()
    out = {"eager_ms_per_step": eager_ms, "recorded_ms_per_step": rec_ms, "flop_per_step": flops,
           "TFLOPs": flops / (rec_ms * 1e-3) / 1e12, "loss_after": float(blk.loss.download()[0, 0])}
    if with_cpu:
        from oracle import compose, oracle
        threads = min(16, oracle.hardware_threads() or 1)
        t0 = time.perf_counter()
        compose.swin_block_forward_backward({k: blk.host[k] for k in blk.names}, blk.host["X"], blk.host["T"], blk.nw, blk.wt,
                                            blk.heads, threads=threads)
        secs = time.perf_counter() - t0
        out["cpu"] = {"steps_per_s": 1.0 / secs, "ms_per_step": secs * 1e3, "cores": threads, "steps_timed": 1, "kind": "port",
                      "note": "forward + backward only, node-by-node composition of the oracle's operations (per-window loop in Python)"}
    return out


def oneshot_leg(n, dtype_name, steps):
    """The call-per-operation entry points (jagged host rows in, jagged host rows out, like today's
    GpuMatrixMultiplyOperation): marshalling, PCIe both ways and allocation are inside the timed region."""
    from parallelreverseautodiff_amd import _lib, seeded
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import check

    lib = _lib.load()
    CudaBlas.Instance.DeviceId = 0
    CudaBlas.Instance.Initialize()
    dtype = np.float64 if dtype_name == "f64" else np.float32
    code = _lib.PRAD_F64 if dtype_name == "f64" else _lib.PRAD_F32

    def jag(a):
        rows = [np.array(a[i]) for i in range(a.shape[0])]
        return rows, (ctypes.c_void_p * len(rows))(*[r.ctypes.data for r in rows])

    A, pa = jag(seeded.uniform(1, 1, (n, n), -1, 1, dtype)); B, pb = jag(seeded.uniform(1, 2, (n, n), -1, 1, dtype))
    G, pg = jag(seeded.normal(1, 3, (n, n), 1.0, dtype))
    C, pc = jag(np.zeros((n, n), dtype)); dA, pda = jag(np.zeros((n, n), dtype)); dB, pdb = jag(np.zeros((n, n), dtype))
    check(lib.prad_matmul_fwd_host(code, pa, pb, pc, n, n, n, n))
    t0 = time.perf_counter()
    for _ in range(steps):
        check(lib.prad_matmul_fwd_host(code, pa, pb, pc, n, n, n, n))
        check(lib.prad_matmul_bwd_host(code, pg, pa, pb, pda, pdb, n, n, n))
    secs = (time.perf_counter() - t0) / steps
    return {"n": n, "ms_per_step": secs * 1e3, "TFLOPs": 6.0 * n ** 3 / secs / 1e12,
            "host_bytes_per_step": 8 * n * n * np.dtype(dtype).itemsize}


def mlp_leg(dtype_name, steps, warmup, with_cpu):
    """Feed-forward training step of configs[0]: batch 64, 784-256-128-10, LeakyReLU(0.01), softmax
    cross-entropy, clip, Adam.  Timed launch by launch and as one recorded launch sequence."""
    from parallelreverseautodiff_amd import _lib, seeded
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.feedforward import FeedForwardNetwork

    lib = _lib.load()
    CudaBlas.Instance.DeviceId = 0
    CudaBlas.Instance.Initialize()
    dtype = np.float64 if dtype_name == "f64" else np.float32
    net = FeedForwardNetwork(dtype=dtype)
    X = seeded.uniform(seeded.DEFAULT_SEED, 1, (64, 784), 0.0, 1.0, dtype)
    T = seeded.one_hot_labels(seeded.DEFAULT_SEED, 2, 64, 10, dtype)
    net.set_batch(X, T)
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.prad_event_create(ctypes.byref(e0)))
    check(lib.prad_event_create(ctypes.byref(e1)))

    def timed(fn):
        for _ in range(warmup):
            fn()
        check(lib.prad_stream_sync())
        t0 = time.perf_counter()
        check(lib.prad_event_record(e0))
        for _ in range(steps):
            fn()
        check(lib.prad_event_record(e1))
        check(lib.prad_stream_sync())
        wall = time.perf_counter() - t0
        ms = ctypes.c_float()
        check(lib.prad_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        return ms.value / steps, wall * 1e3 / steps

    eager_ms, eager_wall = timed(net.step)
    net.record()
    graph_ms, graph_wall = timed(net.replay)
    loss = float(net.loss.download()[0, 0])
    net.release()
    out = {"eager_ms_per_step": eager_ms, "eager_wall_ms_per_step": eager_wall, "recorded_ms_per_step": graph_ms,
           "recorded_wall_ms_per_step": graph_wall, "loss_after": loss, "flop_per_step": net.flops_per_step(),
           "parameters": net.parameter_count()}
    if with_cpu:
        out["cpu"] = mlp_cpu_leg(net.host_W, X, T, net.params, dtype)
    return out


def mlp_cpu_leg(W0, X, T, params, dtype, budget_s=15.0):
    """The same step composed from the oracle's restatements of the reference operations, on the host."""
    from oracle import oracle
    threads = min(16, oracle.hardware_threads() or 1)
    alpha = dtype(params.LeakyReLUAlpha)
    W = [w.copy() for w in W0]
    b = [np.zeros((1, w.shape[1]), dtype) for w in W]
    m = [np.zeros_like(x) for x in W + b]
    v = [np.zeros_like(x) for x in W + b]
    L = len(W)

    def step(t):
        nonlocal W, b, m, v
        a, Z, H = X, [], []
        for l in range(L):
            z = oracle.add_broadcast_fwd(oracle.matmul_fwd(a, W[l], threads=threads), b[l])
            Z.append(z)
            a = z if l == L - 1 else oracle.leakyrelu_fwd(z, alpha)
            H.append(a)
        P = oracle.softmax_fwd(Z[-1])
        oracle.cce_fwd(P, T)
        dz = oracle.softmax_bwd(P, oracle.cce_bwd(P, T))
        dW, db = [None] * L, [None] * L
        for l in range(L - 1, -1, -1):
            db[l] = oracle.add_broadcast_bwd_bias(dz)
            dA, dW[l] = oracle.matmul_bwd(dz, X if l == 0 else H[l - 1], W[l], threads=threads)
            if l > 0:
                dz = oracle.leakyrelu_bwd(Z[l - 1], dA, alpha)
        grads = [oracle.clip(g, params.ClipValue, params.MinimumClipValue) for g in dW + db]
        new = [oracle.adam(w, mm, vv, g, params.LearningRate, params.AdamBeta1, params.AdamBeta2, params.AdamEpsilon, float(t))
               for w, mm, vv, g in zip(W + b, m, v, grads)]
        W, b = [n[0] for n in new[:L]], [n[0] for n in new[L:]]
        m, v = [n[1] for n in new], [n[2] for n in new]

    step(1)
    n, t0 = 0, time.perf_counter()
    while n < 200 and time.perf_counter() - t0 < budget_s:
        step(n + 2)
        n += 1
    secs = (time.perf_counter() - t0) / n
    return {"steps_per_s": 1.0 / secs, "ms_per_step": secs * 1e3, "cores": threads, "steps_timed": n, "kind": "port"}


def cpu_leg(budget_s=40.0):
    """Times the CPU restatement of the reference's Parallel.For path (jagged rows, row-parallel scalar
    i-j-k loops) on this host: a bounded sample of the same workload at a smaller N."""
    from oracle import oracle
    threads = min(16, oracle.hardware_threads() or 1)
    n = 1024
    secs = oracle.time_matmul_fwdbwd(n, np.float64, threads=threads, iters=1)
    for bigger in (2048, 4096):  # each doubling costs 8x the work and misses cache more often
        if secs * 9.0 > budget_s:
            break
        n = bigger
        secs = oracle.time_matmul_fwdbwd(n, np.float64, threads=threads, iters=1)
    flops = 6.0 * n ** 3
    return {"value": flops / secs / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "fp64 MatrixMultiplyOperation forward+backward at N=%d (%.1f GFLOP, 1 pass, %.2f s), "
                      "C++ restatement of the reference's Parallel.For loops on jagged rows, -O2, no FMA" % (n, flops / 1e9, secs)}


def load_traffic(n, dtype_name):
    """HBM bytes per launch measured with rocprofv3 --pmc (recorded under profiles/), or None."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get("gemm_%s_n%d" % (dtype_name, n), {}).get("bytes_per_launch")
    except (OSError, ValueError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--n", type=int, default=4096)
    ap.add_argument("--dtype", choices=["f64", "f32"], default="f64")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-also", action="store_true", help="gemm mode: skip the other-precision and MLP legs")
    ap.add_argument("--mode", choices=["gemm", "bandwidth", "mlp", "matmul_sum", "lstm", "swin", "oneshot"], default="gemm",
                    help="gemm: the headline forward+backward step; bandwidth: the elementwise / clip / Adam kernels; "
                         "mlp: the feed-forward training step of configs[0]")
    ap.add_argument("--elems", type=int, default=64 * 1024 * 1024, help="elements per tensor in bandwidth mode")
    ap.add_argument("--only", default="", help="bandwidth mode: comma-separated kernel names")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py measures one GPU: this path has no multi-GPU part (--gpus 1 only)")
    if args.mode == "oneshot":
        res = oneshot_leg(args.n, args.dtype, args.steps)
        print(json.dumps({"metric": "one-shot host-pointer matmul fwd+bwd TFLOP/s (PCIe and marshalling inclusive)", "unit": "TFLOP/s",
                          "value": res["TFLOPs"], "n_gpus": 1, "steps": args.steps, "warmup": 1, "dtype": args.dtype, "data": "synthetic",
                          "higher_is_better": True, "ms_per_step": res["ms_per_step"],
                          "config": {"workload": "prad_matmul_fwd_host + prad_matmul_bwd_host, N=%d, jagged rows" % args.n}, "detail": res}))
        return
    if args.mode == "swin":
        res = swin_leg(args.dtype, args.steps, args.warmup, not args.no_cpu)
        print(json.dumps({"metric": "Swin block train steps/sec", "unit": "steps/s", "value": 1e3 / res["recorded_ms_per_step"],
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": args.dtype, "data": "synthetic",
                          "higher_is_better": True, "ms_per_step": res["recorded_ms_per_step"],
                          "config": {"workload": "configs[4]: windowed self-attention block, 16 x 56x56 tokens, 7x7 windows, embed 96, "
                                                 "3 heads, MLP x4 GELU, MSE, full backward, clip, Adam"},
                          "detail": res}))
        return
    if args.mode == "lstm":
        res = lstm_leg(args.dtype, args.steps, args.warmup, not args.no_cpu)
        print(json.dumps({"metric": "LSTM train steps/sec", "unit": "steps/s", "value": 1e3 / res["recorded_ms_per_step"],
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": args.dtype, "data": "synthetic",
                          "higher_is_better": True, "ms_per_step": res["recorded_ms_per_step"],
                          "config": {"workload": "configs[3]: LSTM layer 256->512, batch 128, 64 steps, fused 4-gate weight, MSE, "
                                                 "BPTT, clip, Adam"},
                          "detail": res}))
        return
    if args.mode == "matmul_sum":
        res = matmul_sum_leg(args.dtype, args.steps, args.warmup)
        print(json.dumps({"metric": "MatrixMultiplyAndSum forward TFLOP/s, backward GB/s", "unit": "TFLOP/s", "value": res["fwd_TFLOPs"],
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": args.dtype, "data": "synthetic",
                          "higher_is_better": True, "ms_per_step": res["fwd_ms"] + res["bwd_ms"],
                          "config": {"workload": "configs[2]: GpuMatrixMultiplyAndSumOperation, A 512x768 ~N(0,0.02), 32 slices 768x512, "
                                                 "reference semantics (out 1x32; backward as written)"},
                          "detail": res}))
        return
    if args.mode == "mlp":
        res = mlp_leg(args.dtype, args.steps, args.warmup, not args.no_cpu)
        print(json.dumps({"metric": "MLP train steps/sec", "unit": "steps/s", "value": 1e3 / res["recorded_ms_per_step"],
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": args.dtype, "data": "synthetic",
                          "higher_is_better": True, "ms_per_step": res["recorded_ms_per_step"],
                          "config": {"workload": "configs[0]: 3-layer MLP 784-256-128-10, batch 64, LeakyReLU(0.01), softmax "
                                                 "cross-entropy, clip(4), Adam(lr 1e-3): forward + backward + update"},
                          "detail": res}))
        return
    if args.mode == "bandwidth":
        res, n = bandwidth_leg(args.elems, args.dtype, args.steps, args.warmup, [x for x in args.only.split(",") if x])
        best = max(res.values(), key=lambda r: r["GB/s"])
        print(json.dumps({"metric": "fused gradient kernels GB/s (% of 8 TB/s HBM)", "unit": "GB/s", "value": best["GB/s"],
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": args.dtype, "data": "synthetic",
                          "higher_is_better": True, "config": {"workload": "elementwise/clip/Adam kernels on %d elements" % n},
                          "kernels": res}))
        return

    ms, wall_ms, spot = gpu_leg(args.n, args.dtype, args.steps, args.warmup)
    flops_per_step = 6.0 * args.n ** 3
    ms_per_step = ms / args.steps
    tflops = flops_per_step / (ms_per_step * 1e-3) / 1e12
    peak = PEAK_TFLOPS[args.dtype]
    # dominant kernel: the MFMA product kernel, three launches per step of 2 N^3 flop each
    launch_ms = ms / (3 * args.steps)
    achieved = 2.0 * args.n ** 3 / (launch_ms * 1e-3) / 1e12
    line = {
        "metric": METRIC, "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "configs[1]: single MatrixMultiplyOperation forward+backward, %s, square M=N=K=%d, "
                               "A,B~U[-1,1], dC~N(0,1), seed %d, device-resident" % (args.dtype, args.n, 20240611),
                   "flop_per_step": flops_per_step, "launches_per_step": 3},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s", "frac": achieved / peak,
                     "traffic": load_traffic(args.n, args.dtype), "kernel": "prad::gemm_kernel<%s> (NN, NT, TN instantiations)" %
                     ("double" if args.dtype == "f64" else "float"), "launch_ms": launch_ms},
        "wall_ms_per_step": wall_ms / args.steps, "spot_check_error": spot,
    }
    if not args.no_also:
        line["also"] = also_legs(args)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_leg()
    print(json.dumps(line))


def also_legs(args):
    """The rest of the metric beside the headline figure, measured in the same run: the product in the other
    precision at the same size, the MLP training step of configs[0] (recorded launch sequence; in double beside its CPU
    restatement on the host cores) and the LSTM training step of configs[3].  A leg
    that fails is reported as its error text and does not touch the headline figures."""
    out = {}
    other = "f32" if args.dtype == "f64" else "f64"
    try:
        ms, _, spot = gpu_leg(args.n, other, args.steps, args.warmup)
        tf = 6.0 * args.n ** 3 / (ms / args.steps * 1e-3) / 1e12
        out["matmul_fwd_bwd_" + other] = {"TFLOPs": tf, "frac_of_mfma_peak": tf / PEAK_TFLOPS[other], "n": args.n,
                                          "ms_per_step": ms / args.steps, "spot_check_error": spot}
    except Exception as e:  # noqa: BLE001 - reported, not hidden
        out["matmul_fwd_bwd_" + other] = {"error": repr(e)}
    for d in ("f64", "f32"):
        try:
            r = mlp_leg(d, 1000, 100, d == "f64" and not args.no_cpu)
            leg = {"value": 1e3 / r["recorded_ms_per_step"], "ms_per_step": r["recorded_ms_per_step"], "loss_after": r["loss_after"]}
            if "cpu" in r:
                leg["cpu_baseline"] = r["cpu"]
            out["mlp_train_steps_per_s_" + d] = leg
        except Exception as e:  # noqa: BLE001
            out["mlp_train_steps_per_s_" + d] = {"error": repr(e)}
    try:
        r = lstm_leg("f32", 10, 2, False)
        out["lstm_train_steps_per_s_f32"] = {"value": 1e3 / r["recorded_ms_per_step"], "ms_per_step": r["recorded_ms_per_step"]}
    except Exception as e:  # noqa: BLE001
        out["lstm_train_steps_per_s_f32"] = {"error": repr(e)}
    return out


if __name__ == "__main__":
    main()
