"""Benchmark of the matrix-multiply forward+backward path on one MI355X.

One step = MatrixMultiplyOperation forward (C = A.B) plus backward (dA = dC.B^T, dB = A^T.dC) on
device-resident square double matrices, N = 4096 by default: three launches of the MFMA product
kernel, 6 N^3 floating-point operations.  The LAST line printed is one compact JSON object (the
figures of the headline leg with its roofline and CPU baseline, under 1800 characters); the line
before it (also written to the file --detail-file names, if any) carries every other leg and the table.

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


def error_metrics(x, ref):
    """The two error figures of a result against the reference's arithmetic: normwise max|x - ref| / max|ref|, and
    elementwise max |x - ref| / max(|ref|, 1e-3 rms(ref)); beside them the measure the parity tests hold to the bar,
    elementwise against max(|ref|, rms(ref))."""
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    diff = np.abs(x - ref)
    rms = float(np.sqrt(np.mean(ref * ref)))
    tiny = np.finfo(np.float64).tiny
    return {"normwise": float(diff.max() / max(float(np.abs(ref).max()), tiny)),
            "elementwise_floor_1e-3_rms": float(np.max(diff / np.maximum(np.abs(ref), max(1e-3 * rms, tiny)))),
            "elementwise_floor_rms": float(np.max(diff / np.maximum(np.abs(ref), max(rms, tiny))))}


def worst_metrics(items):
    out = {}
    for m in items:
        for k, v in m.items():
            out[k] = max(out.get(k, 0.0), v)
    return out


def gemm_sample_errors(A, B, dC, C, dA, dB, dtype, rows=48):
    """Error of the timed buffers against the CPU restatement of MatrixMultiplyOperation (same element type, k-ascending
    sums) on a sample of `rows` rows of each of C, dA and dB; for float also against the products evaluated in double,
    since at K in the thousands the reference's own float loop is further from the exact product than the bar."""
    from oracle import oracle
    n = A.shape[0]
    rng = np.random.default_rng(1)
    idx = np.sort(rng.choice(n, size=min(rows, n), replace=False))
    threads = min(16, oracle.hardware_threads() or 1)
    cont = np.ascontiguousarray
    refs = [(C[idx], oracle.matmul_fwd(cont(A[idx]), B, threads=threads)),                       # C = A.B
            (dA[idx], oracle.matmul_fwd(cont(dC[idx]), cont(B.T), threads=threads)),            # dA = dC.B^T
            (dB[idx], oracle.matmul_fwd(cont(A[:, idx].T), dC, threads=threads))]               # dB = A^T.dC
    out = {"against_reference_arithmetic": worst_metrics(error_metrics(x, r) for x, r in refs), "sampled_rows_per_output": int(len(idx))}
    if dtype == np.float32:
        f = lambda z: np.asarray(z, np.float64)
        exact = [f(A[idx]) @ f(B), f(dC[idx]) @ f(B).T, f(A[:, idx]).T @ f(dC)]
        out["device_against_double"] = worst_metrics(error_metrics(x, e) for (x, _), e in zip(refs, exact))
        out["reference_arithmetic_against_double"] = worst_metrics(error_metrics(r, e) for (_, r), e in zip(refs, exact))
    return out


def gpu_leg(n, dtype_name, steps, warmup, with_errors=True):
    """cfg2: MatrixMultiplyOperation forward + backward on device-resident n x n operands; returns the time of `steps`
    steps (HIP events on the library stream), the wall time, a spot check and the sampled error figures."""
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
    # each of the three launches alone between two events, the stream idle before it: the duration a kernel trace shows
    # for a launch, where back-to-back launches above overlap one launch's drain with the next one's ramp
    isolated = {}
    for name, call in (("NN C=A.B", lambda: lib.prad_gemm(0, 0, h["A"], h["B"], h["C"], 0)),
                       ("NT dA=dC.B^T", lambda: lib.prad_gemm(0, 1, h["dC"], h["B"], h["dA"], 0)),
                       ("TN dB=A^T.dC", lambda: lib.prad_gemm(1, 0, h["A"], h["dC"], h["dB"], 0))):
        total = 0.0
        reps = max(3, min(steps, 10))
        for _ in range(reps):
            check(lib.prad_stream_sync())
            check(lib.prad_event_record(e0))
            check(call())
            check(lib.prad_event_record(e1))
            one = ctypes.c_float()
            check(lib.prad_event_elapsed_ms(e0, e1, ctypes.byref(one)))
            total += one.value
        isolated[name] = total / reps
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
    errors = gemm_sample_errors(A, B, dC, C, bufs["dA"].download(), bufs["dB"].download(), dtype) if with_errors else None
    return {"ms": float(ms.value), "wall_ms": wall_ms, "spot": worst, "errors": errors, "isolated_launch_ms": isolated}


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

    first = None
    if with_cpu:  # forward + backward from the initial weights, kept for the error figures
        layer.step(update=False)
        layer.iteration = 0
        first = {"loss": float(layer.loss.download()[0, 0]), "hidden states": layer.H_out.download(), "dW": layer.dW.download(),
                 "db": layer.db.download(), "dX": layer.dX.download()}
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
        loss, Hout, dW, db, dX = compose.lstm_forward_backward(layer.host_W, np.zeros((1, 4 * H), dtype), layer.host_X, layer.host_Y,
                                                               I, H, B, T, threads=threads)
        secs = time.perf_counter() - t0
        out["cpu"] = {"steps_per_s": 1.0 / secs, "ms_per_step": secs * 1e3, "cores": threads, "steps_timed": 1, "kind": "port",
                      "note": "forward + backward only (no clip/Adam), node-by-node composition of the oracle's operations"}
        out["errors"] = {"against_reference_arithmetic": worst_metrics(
            error_metrics(first[k], r) for k, r in (("hidden states", Hout), ("dW", dW), ("db", db), ("dX", dX))),
            "loss_relative": abs(first["loss"] - loss) / abs(loss)}
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

    first = None
    if with_cpu:  # forward + backward from the initial weights, kept for the error figures
        blk.step(update=False)
        blk.iteration = 0
        first = {"loss": float(blk.loss.download()[0, 0]), "Y2": blk.Y2.download(), "dX": blk.dX.download()}
        first.update({k: blk.g[k].download() for k in blk.names})
        operands = {"W2": (blk.H1, blk.dY2), "W1": (blk.Y1, blk.dZ1), "Wo": (blk.O, blk.dY1), "Wqkv": (blk.X, blk.dQKV)}
        exact = {k: lhs.download().astype(np.float64).T @ rhs.download().astype(np.float64) for k, (lhs, rhs) in operands.items()}
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
        loss, Y2, g, dX = compose.swin_block_forward_backward({k: blk.host[k] for k in blk.names}, blk.host["X"], blk.host["T"],
                                                              blk.nw, blk.wt, blk.heads, threads=threads)
        secs = time.perf_counter() - t0
        out["cpu"] = {"steps_per_s": 1.0 / secs, "ms_per_step": secs * 1e3, "cores": threads, "steps_timed": 1, "kind": "port",
                      "note": "forward + backward only, node-by-node composition of the oracle's operations (per-window loop in Python)"}
        pairs = [("Y2", Y2), ("dX", dX)] + [(k, g[k]) for k in blk.names]
        out["errors"] = {"against_reference_arithmetic": worst_metrics(error_metrics(first[k], r) for k, r in pairs),
                         "loss_relative": abs(first["loss"] - loss) / abs(loss),
                         # the weight gradients are sums over all 50 176 token rows: there the reference's k-ascending
                         # float loop is the less accurate side, so both are also measured against the double product
                         "weight_gradients_device_against_double": worst_metrics(error_metrics(first[k], exact[k]) for k in exact),
                         "weight_gradients_reference_arithmetic_against_double": worst_metrics(error_metrics(g[k], exact[k]) for k in exact)}
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

    first = None
    if with_cpu:  # the first step from the initial weights, kept for the error figures
        net.step()
        first = {"loss": float(net.loss.download()[0, 0]), "grads": [g.download() for g in net._grads],
                 "weights": [w.download() for w in net._weights]}
        net = FeedForwardNetwork(dtype=dtype)
        net.set_batch(X, T)
    eager_ms, eager_wall = timed(net.step)
    net.record()
    graph_ms, graph_wall = timed(net.replay)
    loss = float(net.loss.download()[0, 0])
    net.release()
    out = {"eager_ms_per_step": eager_ms, "eager_wall_ms_per_step": eager_wall, "recorded_ms_per_step": graph_ms,
           "recorded_wall_ms_per_step": graph_wall, "loss_after": loss, "flop_per_step": net.flops_per_step(),
           "parameters": net.parameter_count()}
    if with_cpu:
        out["cpu"], ref = mlp_cpu_leg(net.host_W, X, T, net.params, dtype)
        # clipped gradients of the first step, and in double also the weights after it (in float a gradient entry at
        # rounding-noise level changes sign between two correct summation orders, and the first Adam step moves its
        # weight by the learning rate either way: the float weights are compared operation by operation in the tests)
        pairs = list(zip(first["grads"], ref["grads"])) + (list(zip(first["weights"], ref["weights"])) if dtype_name == "f64" else [])
        out["errors"] = {"against_reference_arithmetic": worst_metrics(error_metrics(x, r) for x, r in pairs),
                         "loss_relative": abs(first["loss"] - ref["loss"]) / abs(ref["loss"])}
    return out


def mlp_ops_leg(dtype_name, steps, warmup):
    """The configs[0] step driven operation by operation through the operation classes, in the reference's order
    (MatrixMultiplyOperation.Forward -> MatrixAddBroadcastingOperation -> LeakyReLUOperation ... -> loss -> the
    Backward chain with accumulate_gradient into the gradient destinations -> GradientClearer / GradientClipper.Clip /
    AdamOptimizer.Optimize): no fused entry point, no recorded sequence, a fresh output Matrix per call.  This is the
    rate an unchanged caller of the operation classes gets; the host side here is Python, so its figure is the wall
    clock of the loop, and the time the device is busy is given beside it."""
    from parallelreverseautodiff_amd import _lib, seeded
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.feedforward import OperationWalkNetwork

    lib = _lib.load()
    CudaBlas.Instance.DeviceId = 0
    CudaBlas.Instance.Initialize()
    dtype = np.float64 if dtype_name == "f64" else np.float32
    net = OperationWalkNetwork(dtype=dtype)
    net.set_batch(seeded.uniform(seeded.DEFAULT_SEED, 1, (64, 784), 0.0, 1.0, dtype),
                  seeded.one_hot_labels(seeded.DEFAULT_SEED, 2, 64, 10, dtype))

    def stats():
        vals = [ctypes.c_int64() for _ in range(5)]
        check(lib.prad_alloc_stats(*[ctypes.byref(v) for v in vals]))
        return [v.value for v in vals]

    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.prad_event_create(ctypes.byref(e0)))
    check(lib.prad_event_create(ctypes.byref(e1)))
    for _ in range(max(warmup, 3)):
        net.step()
    check(lib.prad_stream_sync())
    before = stats()
    t0 = time.perf_counter()
    check(lib.prad_event_record(e0))
    for _ in range(steps):
        net.step()
    check(lib.prad_event_record(e1))
    issue_ms = (time.perf_counter() - t0) * 1e3 / steps      # host time to issue a step (nothing waits for the device)
    check(lib.prad_stream_sync())
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    after = stats()
    ms = ctypes.c_float()
    check(lib.prad_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
    # the same walk driven by compiled code (libprad_hostwalk.so: C ABI calls only), where the host is no interpreter
    compiled = None
    try:
        from parallelreverseautodiff_amd.feedforward import compiled_operation_walk
        c_ms, c_loss, _ = compiled_operation_walk(dtype=dtype, steps=max(steps, 500), warmup=50)
        compiled = {"wall_ms_per_step": c_ms, "steps_per_s": 1e3 / c_ms, "loss_after": c_loss}
    except Exception as e:  # noqa: BLE001 - reported, not hidden
        compiled = {"error": repr(e)}
    return {"wall_ms_per_step": wall_ms, "host_issue_ms_per_step": issue_ms, "device_ms_per_step": ms.value / steps,
            "steps_per_s": 1e3 / wall_ms, "compiled_caller": compiled, "loss_after": float(net.loss.to_numpy()[0, 0]), "flop_per_step": net.flops_per_step(),
            "operations_per_step": 2 * len(net.nodes) + 2, "device_mallocs_in_timed_steps": after[0] - before[0],
            "device_frees_in_timed_steps": after[1] - before[1], "stream_waits_in_timed_steps": after[2] - before[2],
            "pool_hits_in_timed_steps": after[3] - before[3]}


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
        loss = oracle.cce_fwd(P, T)
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
        return {"loss": loss, "grads": grads, "weights": W + b}

    first = step(1)
    n, t0 = 0, time.perf_counter()
    while n < 200 and time.perf_counter() - t0 < budget_s:
        step(n + 2)
        n += 1
    secs = (time.perf_counter() - t0) / n
    return {"steps_per_s": 1.0 / secs, "ms_per_step": secs * 1e3, "cores": threads, "steps_timed": n, "kind": "port"}, first


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
    return {"value": flops / secs / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port", "n": n, "secs": secs,
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
    ap.add_argument("--detail-file", default=None, help="gemm mode: also write the detail line to this file")
    ap.add_argument("--mode", choices=["gemm", "bandwidth", "mlp", "mlp_ops", "matmul_sum", "lstm", "swin", "oneshot"], default="gemm",
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
    if args.mode == "mlp_ops":
        res = mlp_ops_leg(args.dtype, args.steps, args.warmup)
        print(json.dumps({"metric": "MLP train steps/sec, operation by operation", "unit": "steps/s", "value": res["steps_per_s"],
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": args.dtype, "data": "synthetic",
                          "higher_is_better": True, "ms_per_step": res["wall_ms_per_step"],
                          "config": {"workload": "configs[0] driven through the operation classes one Forward / Backward at a time: "
                                                 "fresh outputs per call, accumulate_gradient, GradientClipper.Clip, AdamOptimizer.Optimize"},
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

    head = gpu_leg(args.n, args.dtype, args.steps, args.warmup, with_errors=not args.no_cpu)
    cpu = None if args.no_cpu else cpu_leg()
    ms_per_step = head["ms"] / args.steps
    table = [gemm_row(args.n, args.dtype, ms_per_step, head["errors"], cpu)]
    also = None if args.no_also else also_legs(args, table)
    line, detail = headline_lines(args, head, cpu, also, table)
    text = json.dumps({"detail": detail})
    print(text)
    if args.detail_file:  # the same detail as a file, for runs whose captured output is cut short
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.detail_file)), exist_ok=True)
            with open(args.detail_file, "w") as f:
                f.write(text + "\n")
        except OSError:
            pass
    sys.stdout.flush()
    print(json.dumps(line, separators=(",", ":")))


MAX_LINE_CHARS = 1800  # the harness that runs this keeps the tail of stdout: the last line has to fit in it


def headline_lines(args, head, cpu, also, table):
    """(the compact last line, the detail object) of the headline run from its legs' results.  Everything bulky - the
    error blocks, the other legs with their rooflines, the table - goes into the detail object; the last line holds
    the contract's fields, the roofline and CPU baseline of the headline kernel, and a few scalars of the other legs."""
    n, steps = args.n, args.steps
    flops_per_step = 6.0 * n ** 3
    ms_per_step = head["ms"] / steps
    tflops = flops_per_step / (ms_per_step * 1e-3) / 1e12
    peak = PEAK_TFLOPS[args.dtype]
    # dominant kernel: the MFMA product kernel, three products per step of 2 N^3 flop each (three launches at N = 4096;
    # below N = 2600 both gradient products share one launch)
    launch_ms = head["ms"] / (3 * steps)
    achieved = 2.0 * n ** 3 / (launch_ms * 1e-3) / 1e12
    iso = head.get("isolated_launch_ms") or {}
    iso_mean = sum(iso.values()) / len(iso) if iso else None
    sig = lambda x, d=5: None if x is None else float("%.*g" % (d, x))
    line = {
        "metric": METRIC, "value": sig(tflops), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": sig(ms_per_step), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "configs[1]: MatrixMultiplyOperation forward+backward, %s, M=N=K=%d, A,B~U[-1,1], dC~N(0,1), seed %d, "
                               "device-resident, 3 products, 6N^3 flop/step" % (args.dtype, n, 20240611)},
        "roofline": {"bound": "mfma", "achieved": sig(achieved), "peak": peak, "unit": "TFLOP/s", "frac": sig(achieved / peak, 4),
                     "traffic": load_traffic(n, args.dtype), "kernel": "prad::gemm_kernel<%s> NN/NT/TN" % ("double" if args.dtype == "f64" else "float"),
                     "launch_ms": sig(launch_ms), "launch_ms_isolated": sig(iso_mean),
                     "frac_isolated": None if not iso_mean else sig(2.0 * n ** 3 / (iso_mean * 1e-3) / 1e12 / peak, 4)},
    }
    if cpu is not None:
        line["cpu_baseline"] = {"value": sig(cpu["value"]), "unit": cpu["unit"], "cores": cpu["cores"], "kind": cpu["kind"],
                                "sample": "fp64 fwd+bwd at N=%d, 1 pass, %.1f s" % (cpu["n"], cpu["secs"])}
    detail = {"headline": {"wall_ms_per_step": head["wall_ms"] / steps, "spot_check_error": head["spot"], "errors": head["errors"],
                           "isolated_launch_ms": iso, "flop_per_step": flops_per_step, "products_per_step": 3},
              "cpu_baseline": cpu, "also": also, "table": table}
    if head["errors"] is not None:
        line["err_vs_reference_arithmetic"] = sig(head["errors"]["against_reference_arithmetic"]["elementwise_floor_rms"], 3)
    extras = summary_scalars(also) if also else {}
    for key, value in extras.items():  # scalars of the other legs, as many as fit
        line.setdefault("also", {})[key] = value
        if len(json.dumps(line, separators=(",", ":"))) > MAX_LINE_CHARS:
            del line["also"][key]
            break
    return line, detail


def summary_scalars(also):
    """A few scalars of the other legs for the last line (their full results are in the detail object)."""
    out = {}
    sig = lambda x: float("%.4g" % x)

    def put(key, leg, *path):
        try:
            v = also[leg]
            for k in path:
                v = v[k]
            out[key] = sig(v)
        except (KeyError, TypeError):
            pass
    for leg in also:
        if leg.startswith("matmul_fwd_bwd_"):
            put(leg.replace("matmul_fwd_bwd_", "") + "_frac", leg, "roofline", "frac")
    put("mlp_f64_steps_s", "mlp_train_steps_per_s_f64", "value")
    put("mlp_f64_cpu_steps_s", "mlp_train_steps_per_s_f64", "cpu_baseline", "steps_per_s")
    put("mlp_ops_f64_steps_s", "mlp_operation_walk_f64", "value")
    put("mlp_ops_compiled_f64_steps_s", "mlp_operation_walk_f64", "detail", "compiled_caller", "steps_per_s")
    put("mlp_f32_steps_s", "mlp_train_steps_per_s_f32", "value")
    put("mlp_ops_f32_steps_s", "mlp_operation_walk_f32", "value")
    put("mlp_ops_compiled_f32_steps_s", "mlp_operation_walk_f32", "detail", "compiled_caller", "steps_per_s")
    put("lstm_f32_steps_s", "lstm_train_steps_per_s_f32", "value")
    put("lstm_f32_frac", "lstm_train_steps_per_s_f32", "roofline", "frac")
    put("swin_f32_steps_s", "swin_block_train_steps_per_s_f32", "value")
    put("swin_f32_frac", "swin_block_train_steps_per_s_f32", "roofline", "frac")
    put("matmulsum_fwd_frac", "matmul_and_sum_f32", "forward", "roofline", "frac")
    put("matmulsum_bwd_hbm_frac", "matmul_and_sum_f32", "backward", "roofline", "frac")
    for d in ("f64", "f32"):
        leg = also.get("gradient_kernels_64Mi_" + d)
        if isinstance(leg, dict) and "error" not in leg:
            fr = {k: v["roofline"]["frac"] for k, v in leg.items()}
            out["adam_%s_hbm_frac" % d] = sig(fr.get("adam", 0.0))
            out["min_act_bwd_%s_hbm_frac" % d] = sig(min(v for k, v in fr.items() if k.endswith("_bwd")))
    failed = [k for k, v in also.items() if isinstance(v, dict) and "error" in v]
    if failed:
        out["failed_legs"] = len(failed)
    return out


def mfma_roofline(flops, ms, dtype_name, kernel, traffic=None):
    achieved = flops / (ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": achieved, "peak": PEAK_TFLOPS[dtype_name], "unit": "TFLOP/s",
            "frac": achieved / PEAK_TFLOPS[dtype_name], "traffic": traffic, "kernel": kernel}


def hbm_roofline(nbytes, ms, kernel):
    achieved = nbytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": achieved, "peak": 8000.0, "unit": "GB/s", "frac": achieved / 8000.0, "traffic": None, "kernel": kernel}


def flat_errors(errors):
    """The two error columns of a table row from an `errors` block (None where the leg had no CPU side)."""
    if not errors:
        return {"err_normwise": None, "err_elementwise_floor_1e-3_rms": None}
    m = errors["against_reference_arithmetic"]
    return {"err_normwise": m["normwise"], "err_elementwise_floor_1e-3_rms": m["elementwise_floor_1e-3_rms"],
            "err_elementwise_floor_rms": m["elementwise_floor_rms"]}


def gemm_row(n, dtype_name, ms_per_step, errors, cpu):
    """Table row of the square product; the CPU columns are filled where the CPU sample ran at this very size."""
    tf = 6.0 * n ** 3 / (ms_per_step * 1e-3) / 1e12
    row = {"config": "configs[1] MatrixMultiply fwd+bwd N=%d" % n, "precision": dtype_name, "gpu_ms": ms_per_step, "rate": tf,
           "unit": "TFLOP/s", "bound": "mfma", "frac_of_peak": tf / PEAK_TFLOPS[dtype_name], "cpu_ms": None, "cpu_cores": None, "speedup": None}
    if cpu is not None and dtype_name == "f64" and cpu.get("n") == n:
        row.update({"cpu_ms": cpu["secs"] * 1e3, "cpu_cores": cpu["cores"], "speedup": cpu["secs"] * 1e3 / ms_per_step})
    row.update(flat_errors(errors))
    return row


def step_row(config, dtype_name, r):
    """Table row of a training step (MLP, LSTM, attention block) from its leg's result."""
    ms = r["recorded_ms_per_step"]
    tf = r["flop_per_step"] / (ms * 1e-3) / 1e12
    row = {"config": config, "precision": dtype_name, "gpu_ms": ms, "rate": 1e3 / ms, "unit": "steps/s", "bound": "mfma",
           "frac_of_peak": tf / PEAK_TFLOPS[dtype_name], "cpu_ms": None, "cpu_cores": None, "speedup": None}
    if "cpu" in r:
        row.update({"cpu_ms": r["cpu"]["ms_per_step"], "cpu_cores": r["cpu"]["cores"], "speedup": r["cpu"]["ms_per_step"] / ms})
    row.update(flat_errors(r.get("errors")))
    return row


def also_legs(args, table):
    """The rest of the metric beside the headline figure, measured in the same run, each with the roofline that bounds
    it: the product in the other precision at the same size and both precisions at the smaller sizes of the
    configuration, the MLP training step (recorded launch sequence; beside its CPU restatement on the host cores), the
    LSTM and attention-block steps, MatrixMultiplyAndSum, and the bandwidth-bound gradient kernels on 64 Mi elements.
    Every leg also adds its row to `table`.  A leg that fails is reported as its error text and does not touch the
    headline figures."""
    out = {}
    with_cpu = not args.no_cpu
    other = "f32" if args.dtype == "f64" else "f64"
    for n, d, steps in [(args.n, other, args.steps)] + [(m, dt, 60) for m in (2048, 1024, 512) if m < args.n for dt in ("f64", "f32")]:
        key = "matmul_fwd_bwd_%s_n%d" % (d, n)
        try:
            r = gpu_leg(n, d, steps, args.warmup, with_errors=with_cpu)
            per = r["ms"] / steps
            out[key] = {"TFLOPs": 6.0 * n ** 3 / (per * 1e-3) / 1e12, "n": n, "ms_per_step": per, "spot_check_error": r["spot"],
                        "roofline": mfma_roofline(2.0 * n ** 3, per / 3, d, "prad::gemm_kernel<%s>" % ("double" if d == "f64" else "float"),
                                                  traffic=load_traffic(n, d)),
                        "isolated_launch_ms": r["isolated_launch_ms"], "errors": r["errors"]}
            table.append(gemm_row(n, d, per, r["errors"], None))
        except Exception as e:  # noqa: BLE001 - reported, not hidden
            out[key] = {"error": repr(e)}
    for d in ("f64", "f32"):
        try:
            r = mlp_leg(d, 1000, 100, with_cpu)
            leg = {"value": 1e3 / r["recorded_ms_per_step"], "unit": "steps/s", "ms_per_step": r["recorded_ms_per_step"],
                   "loss_after": r["loss_after"], "errors": r.get("errors"),
                   "roofline": mfma_roofline(r["flop_per_step"], r["recorded_ms_per_step"], d,
                                             "whole step: 9 dependent launches (products on 32x32 tiles, softmax + cross-entropy, clip + Adam)")}
            if "cpu" in r:
                leg["cpu_baseline"] = r["cpu"]
            out["mlp_train_steps_per_s_" + d] = leg
            table.append(step_row("configs[0] MLP 784-256-128-10 batch 64 step", d, r))
        except Exception as e:  # noqa: BLE001
            out["mlp_train_steps_per_s_" + d] = {"error": repr(e)}
    for d in ("f64", "f32"):
        try:
            r = mlp_ops_leg(d, 300, 20)
            out["mlp_operation_walk_" + d] = {"value": r["steps_per_s"], "unit": "steps/s", "ms_per_step": r["wall_ms_per_step"], "detail": r,
                                               "roofline": mfma_roofline(r["flop_per_step"], r["wall_ms_per_step"], d,
                                                                         "whole step, one launch per operation (%d operations)" % r["operations_per_step"])}
            if "steps_per_s" in (r.get("compiled_caller") or {}):
                c = r["compiled_caller"]
                table.append({"config": "configs[0] MLP step, operation by operation, compiled caller of the C ABI", "precision": d,
                              "gpu_ms": c["wall_ms_per_step"], "rate": c["steps_per_s"], "unit": "steps/s", "bound": "mfma",
                              "frac_of_peak": r["flop_per_step"] / (c["wall_ms_per_step"] * 1e-3) / 1e12 / PEAK_TFLOPS[d],
                              "cpu_ms": None, "cpu_cores": None, "speedup": None, "err_normwise": None, "err_elementwise_floor_1e-3_rms": None})
            table.append({"config": "configs[0] MLP step, operation by operation through the operation classes", "precision": d,
                          "gpu_ms": r["wall_ms_per_step"], "rate": r["steps_per_s"], "unit": "steps/s", "bound": "mfma",
                          "frac_of_peak": r["flop_per_step"] / (r["wall_ms_per_step"] * 1e-3) / 1e12 / PEAK_TFLOPS[d],
                          "cpu_ms": None, "cpu_cores": None, "speedup": None, "err_normwise": None, "err_elementwise_floor_1e-3_rms": None})
        except Exception as e:  # noqa: BLE001
            out["mlp_operation_walk_" + d] = {"error": repr(e)}
    for name, fn, config, kernel in (
            ("lstm_train_steps_per_s_f32", lstm_leg, "configs[3] LSTM 256->512 batch 128 T=64 step",
             "whole step: 2 x 64 recurrent launches + 5 large products"),
            ("swin_block_train_steps_per_s_f32", swin_leg, "configs[4] windowed attention block 16x56x56 embed 96 step",
             "whole step: 12 dense products, 6 batched window products, softmax, column sums")):
        try:
            r = fn("f32", 50, 10, with_cpu)
            leg = {"value": 1e3 / r["recorded_ms_per_step"], "unit": "steps/s", "ms_per_step": r["recorded_ms_per_step"],
                   "errors": r.get("errors"), "roofline": mfma_roofline(r["flop_per_step"], r["recorded_ms_per_step"], "f32", kernel)}
            if "cpu" in r:
                leg["cpu_baseline"] = r["cpu"]
            out[name] = leg
            table.append(step_row(config, "f32", r))
        except Exception as e:  # noqa: BLE001
            out[name] = {"error": repr(e)}
    try:
        r = matmul_sum_leg("f32", 100, 10)
        out["matmul_and_sum_f32"] = {
            "forward": {"ms": r["fwd_ms"], "roofline": mfma_roofline(r["fwd_flop"], r["fwd_ms"], "f32", "prad::gemm_kernel<float> with the per-tile sum epilogue")},
            "backward": {"ms": r["bwd_ms"], "roofline": hbm_roofline(r["bwd_bytes"], r["bwd_ms"], "prad::sum_bwd_kernel<float>")}}
        table.append({"config": "configs[2] MatrixMultiplyAndSum forward 512x768 x 32 slices", "precision": "f32", "gpu_ms": r["fwd_ms"],
                      "rate": r["fwd_TFLOPs"], "unit": "TFLOP/s", "bound": "mfma", "frac_of_peak": r["fwd_frac_of_mfma_peak"],
                      "cpu_ms": None, "cpu_cores": None, "speedup": None, "err_normwise": None, "err_elementwise_floor_1e-3_rms": None})
        table.append({"config": "configs[2] MatrixMultiplyAndSum backward (as the reference writes it)", "precision": "f32", "gpu_ms": r["bwd_ms"],
                      "rate": r["bwd_GBps"], "unit": "GB/s", "bound": "hbm", "frac_of_peak": r["bwd_frac_of_8TBps"],
                      "cpu_ms": None, "cpu_cores": None, "speedup": None, "err_normwise": None, "err_elementwise_floor_1e-3_rms": None})
    except Exception as e:  # noqa: BLE001
        out["matmul_and_sum_f32"] = {"error": repr(e)}
    for d in ("f64", "f32"):
        try:
            res, n = bandwidth_leg(64 * 1024 * 1024, d, 10, 2,
                                   ["leakyrelu_bwd", "sigmoid_bwd", "tanh_bwd", "gelu_bwd", "hadamard_bwd", "accumulate", "clip", "adam"])
            es = 8 if d == "f64" else 4
            out["gradient_kernels_64Mi_" + d] = {
                k: {"ms": v["ms"], "roofline": hbm_roofline(v["bytes_per_element"] * n, v["ms"], k)} for k, v in res.items()}
            for k, v in res.items():
                table.append({"config": "%s on 64 Mi elements" % k, "precision": d, "gpu_ms": v["ms"], "rate": v["GB/s"], "unit": "GB/s",
                              "bound": "hbm", "frac_of_peak": v["frac_of_8TBps"], "cpu_ms": None, "cpu_cores": None, "speedup": None,
                              "err_normwise": None, "err_elementwise_floor_1e-3_rms": None})
        except Exception as e:  # noqa: BLE001
            out["gradient_kernels_64Mi_" + d] = {"error": repr(e)}
    return out


if __name__ == "__main__":
    main()
