"""The feed-forward training step (config: batch 64, 784-256-128-10, LeakyReLU, softmax cross-entropy, clip,
Adam) against the oracle's composition of the same reference operations."""
import numpy as np
import pytest

from conftest import assert_parity
from parallelreverseautodiff_amd import seeded
from parallelreverseautodiff_amd.feedforward import FeedForwardNetwork
from parallelreverseautodiff_amd.matrix import Matrix
from parallelreverseautodiff_amd.operations import CategoricalCrossEntropyLossOperation, SoftmaxOperation

pytestmark = pytest.mark.gpu
DTYPES = [np.float64, np.float32]


def oracle_step(oracle, W, b, m, v, X, T, params, t, dtype, adam_grads=None):
    """Forward, loss, backward, clip, Adam with the oracle's restatements, layer by layer.  `adam_grads`
    replaces the oracle's own clipped gradients as Adam's input (see the float case below)."""
    alpha = dtype(params.LeakyReLUAlpha)
    L = len(W)
    a, Z, H = X, [], []
    for l in range(L):
        z = oracle.add_broadcast_fwd(oracle.matmul_fwd(a, W[l], threads=8), b[l])
        Z.append(z)
        a = z if l == L - 1 else oracle.leakyrelu_fwd(z, alpha)
        H.append(a)
    P = oracle.softmax_fwd(Z[-1])
    loss = oracle.cce_fwd(P, T)
    dz = oracle.softmax_bwd(P, oracle.cce_bwd(P, T))
    dW, db = [None] * L, [None] * L
    for l in range(L - 1, -1, -1):
        inp = X if l == 0 else H[l - 1]
        db[l] = oracle.add_broadcast_bwd_bias(dz)
        dA, dW[l] = oracle.matmul_bwd(dz, inp, W[l], threads=8)
        if l > 0:
            dz = oracle.leakyrelu_bwd(Z[l - 1], dA, alpha)
    grads = [oracle.clip(g, params.ClipValue, params.MinimumClipValue) for g in dW + db]
    new = [oracle.adam(w, mm, vv, g, params.LearningRate, params.AdamBeta1, params.AdamBeta2, params.AdamEpsilon, float(t))
           for w, mm, vv, g in zip(W + b, m, v, adam_grads or grads)]
    return loss, dW + db, grads, new


@pytest.mark.parametrize("dtype", DTYPES)
def test_training_steps_match_oracle(gpu, oracle, dtype):
    net = FeedForwardNetwork(dtype=dtype)
    X = seeded.uniform(seeded.DEFAULT_SEED, 1, (64, 784), 0.0, 1.0, dtype)
    T = seeded.one_hot_labels(seeded.DEFAULT_SEED, 2, 64, 10, dtype)
    net.set_batch(X, T)
    W = [w.copy() for w in net.host_W]
    b = [np.zeros((1, s), dtype) for s in net.sizes[1:]]
    m = [np.zeros_like(x) for x in W + b]
    v = [np.zeros_like(x) for x in W + b]
    for t in (1, 2, 3):
        net.step()
        # In float, Adam's early steps are close to lr * sign(g): entries whose gradient is at rounding-noise
        # level (and the clipper's +-1e-8 floor, which turns that noise into a sign) move a weight by up to
        # lr either way, so end-to-end weight parity is ill-conditioned there.  Gradients are compared
        # end to end; Adam is then checked as an operation, on the gradients the device actually used.
        dev_grads = [g.download() for g in net._grads] if dtype == np.float32 else None
        loss, raw, clipped, new = oracle_step(oracle, W, b, m, v, X, T, net.params, t, dtype, adam_grads=dev_grads)
        assert abs(float(net.loss.download()[0, 0]) - loss) <= (1e-12 if dtype == np.float64 else 1e-5) * abs(loss)
        L = len(W)
        for i, (g_dev, g_ref) in enumerate(zip(net._grads, clipped)):
            assert_parity(g_dev.download(), g_ref, dtype, "clipped gradient %d step %d" % (i, t))
        W = [n[0] for n in new[:L]]; b = [n[0] for n in new[L:]]
        m = [n[1] for n in new]; v = [n[2] for n in new]
        for i, (w_dev, w_ref) in enumerate(zip(net._weights, W + b)):
            assert_parity(w_dev.download(), w_ref, dtype, "weight %d step %d" % (i, t))
        for i, (m_dev, m_ref) in enumerate(zip(net._m, m)):
            assert_parity(m_dev.download(), m_ref, dtype, "first moment %d step %d" % (i, t))


def test_recorded_step_equals_eager_step(gpu):
    """Replays of the recorded launch sequence, with eager work and synchronisation in between, must give
    exactly what the launch-by-launch step gives from the same state."""
    X = seeded.uniform(3, 1, (64, 784), 0.0, 1.0)
    T = seeded.one_hot_labels(3, 2, 64, 10)
    eager, rec = FeedForwardNetwork(), FeedForwardNetwork()
    for net in (eager, rec):
        net.set_batch(X, T)
    # warm-up step on both (sizes shared workspace), then record the next step; AdamIteration advances on both sides
    eager.step(); rec.step()
    rec.record()
    for replay in range(4):
        eager.step()
        rec.replay()
        gpu.Synchronize()
        junk = FeedForwardNetwork(sizes=(32, 16, 4), batch=8)  # unrelated eager work between replays
        junk.set_batch(np.ones((8, 32)), np.eye(8, 4)); junk.step()
        for a, b2 in zip(eager._weights + eager._grads + eager._m + eager._v, rec._weights + rec._grads + rec._m + rec._v):
            assert np.array_equal(a.download(), b2.download()), "replay %d differs" % replay
        assert np.array_equal(eager.loss.download(), rec.loss.download())
    rec.release()


@pytest.mark.parametrize("dtype", DTYPES)
def test_softmax_and_cross_entropy_operations(gpu, oracle, dtype):
    x = seeded.normal(5, 1, (64, 10), 2.0, dtype)
    t = seeded.one_hot_labels(5, 2, 64, 10, dtype)
    sm = SoftmaxOperation.Instantiate(None)
    p = sm.Forward(Matrix.from_numpy(x))
    rp = oracle.softmax_fwd(x)
    assert_parity(p.to_numpy(), rp, dtype, "softmax")
    ce = CategoricalCrossEntropyLossOperation.Instantiate(None)
    loss = ce.Forward(p, Matrix.from_numpy(t)).to_numpy()[0, 0]
    assert abs(loss - oracle.cce_fwd(rp, t)) <= (1e-12 if dtype == np.float64 else 1e-5) * abs(loss)
    dp = ce.Backward(p).Item1
    assert_parity(dp.to_numpy(), oracle.cce_bwd(rp, t), dtype, "cce backward")
    dx = sm.Backward(dp).Item1.to_numpy()
    assert_parity(dx, oracle.softmax_bwd(rp, oracle.cce_bwd(rp, t)), dtype, "softmax backward")
    wide = seeded.normal(5, 3, (3, 1000), 3.0, dtype)  # more columns than a wavefront
    assert_parity(SoftmaxOperation().Forward(Matrix.from_numpy(wide)).to_numpy(), oracle.softmax_fwd(wide), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_recorded_steps_equal_eager_steps_with_advancing_adam_iteration(gpu, dtype):
    """N replays of a recorded step give, bit for bit, what N eager steps with AdamIteration 2, 3, ... give (the
    reference's caller advances AdamIteration every step, src/RMAD/AdamOptimizer.cs:204-207); the fused launches give
    the bits of the operation-by-operation step throughout.  Eager work runs between the replays."""
    X = seeded.uniform(7, 1, (64, 784), 0.0, 1.0, dtype)
    T = seeded.one_hot_labels(7, 2, 64, 10, dtype)
    seq = FeedForwardNetwork(dtype=dtype, fused=False)   # one reference operation per launch
    fus = FeedForwardNetwork(dtype=dtype, fused=True)
    rec = FeedForwardNetwork(dtype=dtype, fused=True)
    for net in (seq, fus, rec):
        net.set_batch(X, T)
        net.step()
    rec.record()
    assert rec.iteration == 1
    for replay in range(4):
        for net in (seq, fus):
            net.step()
        rec.replay()
        gpu.Synchronize()
        assert seq.iteration == fus.iteration == rec.iteration == replay + 2
        for name in ("_weights", "_grads", "_m", "_v"):
            for a, f, c in zip(getattr(seq, name), getattr(fus, name), getattr(rec, name)):
                ref = a.download()
                assert np.array_equal(ref, f.download()), "%s differs (fused launches, pass %d)" % (name, replay)
                assert np.array_equal(ref, c.download()), "%s differs (recorded step, pass %d)" % (name, replay)
        for other in (fus, rec):
            assert np.array_equal(seq.loss.download(), other.loss.download())
    # a replay can be told which AdamIteration it stands for
    from parallelreverseautodiff_amd.exceptions import check
    check(rec.lib.prad_graph_set_adam_iteration(rec._graph, 9.0))
    rec.iteration = 8
    fus.iteration = 8
    fus.step(); rec.replay()
    gpu.Synchronize()
    for a, c in zip(fus._weights, rec._weights):
        assert np.array_equal(a.download(), c.download())
    rec.release()


def test_recording_refuses_other_threads_and_host_traffic(gpu):
    """While one thread records, an enqueueing call from another thread is refused instead of being recorded
    (the reference calls Backward from pool threads, src/RMAD/OperationNeuralNetworkVisitor.cs:303-306), and the
    recording thread itself cannot allocate, free, copy to or from the host or wait for the device."""
    import ctypes
    import threading
    from parallelreverseautodiff_amd import _lib
    from parallelreverseautodiff_amd.exceptions import InvalidOperationException, check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    a, b, c = (DeviceBuffer.alloc(np.float64, 32, 32) for _ in range(3))
    a.upload(np.ones((32, 32))); b.upload(np.full((32, 32), 2.0))
    check(lib.prad_matmul_fwd(a.handle, b.handle, c.handle))          # eager once
    check(lib.prad_graph_begin())
    status = {}
    try:
        def other():
            status["matmul"] = lib.prad_matmul_fwd(a.handle, b.handle, c.handle)
            status["message"] = lib.prad_last_error().decode()
            status["end"] = lib.prad_graph_end(ctypes.byref(ctypes.c_void_p()))
        th = threading.Thread(target=other)
        th.start(); th.join()
        assert status["matmul"] == _lib.PRAD_ERR_RECORDING and "another thread" in status["message"]
        assert status["end"] == _lib.PRAD_ERR_RECORDING
        extra = ctypes.c_void_p()
        assert lib.prad_buf_alloc(_lib.PRAD_F64, 4, 4, ctypes.byref(extra)) == _lib.PRAD_ERR_RECORDING
        host = np.zeros((32, 32))
        assert lib.prad_buf_download(c.handle, host.ctypes.data_as(ctypes.c_void_p), 32) == _lib.PRAD_ERR_RECORDING
        assert lib.prad_stream_sync() == _lib.PRAD_ERR_RECORDING
        assert lib.prad_graph_begin() == _lib.PRAD_ERR_RECORDING
        with pytest.raises(InvalidOperationException):
            check(lib.prad_buf_upload(c.handle, host.ctypes.data_as(ctypes.c_void_p), 32))
        check(lib.prad_matmul_fwd(a.handle, b.handle, c.handle))      # the recording thread records
    finally:
        g = ctypes.c_void_p()
        check(lib.prad_graph_end(ctypes.byref(g)))
    check(lib.prad_buf_zero(c.handle))
    check(lib.prad_graph_launch(g))
    assert np.array_equal(c.download(), np.full((32, 32), 64.0))      # exactly one product was recorded
    assert lib.prad_graph_launch(ctypes.c_void_p(a.handle.value)) == _lib.PRAD_ERR_BAD_HANDLE
    check(lib.prad_graph_destroy(g))


def test_workspace_growth_while_a_recorded_sequence_is_alive(gpu, oracle):
    """A recorded split product keeps the workspace address it was recorded with.  An eager call that needs a larger
    workspace afterwards must not free that block under it: the replay still gives the recorded product's bits, and
    growing the workspace during a recording is refused."""
    import ctypes
    from parallelreverseautodiff_amd import _lib
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    dtype = np.float64
    M, K, N = 64, 4096, 64                      # few tiles, long K: runs split along K through the workspace
    A = seeded.uniform(3, 1, (M, K), -1, 1, dtype)
    B = seeded.uniform(3, 2, (K, N), -1, 1, dtype)
    a, b, c = DeviceBuffer.alloc(dtype, M, K), DeviceBuffer.alloc(dtype, K, N), DeviceBuffer.alloc(dtype, M, N)
    a.upload(A); b.upload(B)
    check(lib.prad_matmul_fwd(a.handle, b.handle, c.handle))
    eager = c.download()
    check(lib.prad_graph_begin())
    try:
        check(lib.prad_matmul_fwd(a.handle, b.handle, c.handle))
    finally:
        g = ctypes.c_void_p()
        check(lib.prad_graph_end(ctypes.byref(g)))
    # eager work that outgrows the workspace: a taller split product (same kernels, 16x the partial tiles)
    M2 = 1024
    a2, c2 = DeviceBuffer.alloc(dtype, M2, K), DeviceBuffer.alloc(dtype, M2, N)
    a2.upload(seeded.uniform(3, 4, (M2, K), -1, 1, dtype))
    check(lib.prad_matmul_fwd(a2.handle, b.handle, c2.handle))
    check(lib.prad_buf_zero(c.handle))
    for _ in range(3):
        check(lib.prad_graph_launch(g))
        check(lib.prad_matmul_fwd(a2.handle, b.handle, c2.handle))   # eager work in between, on the new workspace
        gpu.Synchronize()
        assert np.array_equal(c.download(), eager)
    check(lib.prad_graph_destroy(g))
    # growth during a recording is refused with a message that says what to do: a sum of 16 products whose partial
    # results (16 x 1536 x 1536 doubles = 288 MiB) outgrow everything above and whatever tests run before this one left
    P, m, k, n = 16, 1536, 64, 1536
    da, db, dc = DeviceBuffer.alloc(dtype, m, k, depth=P), DeviceBuffer.alloc(dtype, k, n, depth=P), DeviceBuffer.alloc(dtype, m, n)
    check(lib.prad_graph_begin())
    try:
        st = lib.prad_matmul_batch_sum_fwd(da.handle, db.handle, None, dc.handle)
        msg = lib.prad_last_error().decode()
    finally:
        g = ctypes.c_void_p()
        check(lib.prad_graph_end(ctypes.byref(g)))
    assert st == _lib.PRAD_ERR_RECORDING and "once before recording" in msg
    check(lib.prad_graph_destroy(g))
    check(lib.prad_matmul_batch_sum_fwd(da.handle, db.handle, None, dc.handle))   # eagerly it grows and runs
    gpu.Synchronize()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(64, 10), (5, 200), (1, 1), (700, 12)])
def test_fused_softmax_cross_entropy_equals_separate_launches(gpu, dtype, shape):
    from parallelreverseautodiff_amd import _lib
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    x = seeded.normal(9, 1, shape, 2.0, dtype)
    t = seeded.one_hot_labels(9, 2, shape[0], shape[1], dtype)
    bx, bt = DeviceBuffer.alloc(dtype, *shape), DeviceBuffer.alloc(dtype, *shape)
    bx.upload(x); bt.upload(t)
    p1, dp1, dx1, p2, dp2, dx2 = (DeviceBuffer.alloc(dtype, *shape) for _ in range(6))
    l1, l2 = DeviceBuffer.alloc(dtype, 1, 1), DeviceBuffer.alloc(dtype, 1, 1)
    check(lib.prad_softmax_fwd(bx.handle, p1.handle))
    check(lib.prad_cce_fwd(p1.handle, bt.handle, l1.handle))
    check(lib.prad_cce_bwd(p1.handle, bt.handle, dp1.handle))
    check(lib.prad_softmax_bwd(p1.handle, dp1.handle, dx1.handle))
    check(lib.prad_softmax_cce(bx.handle, bt.handle, p2.handle, l2.handle, dp2.handle, dx2.handle))
    for a, b2 in ((p1, p2), (dp1, dp2), (dx1, dx2), (l1, l2)):
        assert np.array_equal(a.download(), b2.download())
    check(lib.prad_softmax_cce(bx.handle, bt.handle, p2.handle, None, dp2.handle, dx2.handle))   # loss is optional
    assert np.array_equal(dx1.download(), dx2.download())


def _alloc_stats():
    import ctypes
    from parallelreverseautodiff_amd import _lib
    vals = [ctypes.c_int64() for _ in range(5)]
    assert _lib.load().prad_alloc_stats(*[ctypes.byref(v) for v in vals]) == 0
    return dict(zip(("mallocs", "frees", "syncs", "pool_hits", "pooled_bytes"), (v.value for v in vals)))


@pytest.mark.parametrize("multiply", ["MatrixMultiplyOperation", "GpuMatrixMultiplyOperation", "CudaMatrixMultiplyOperation"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_operation_by_operation_walk(gpu, oracle, dtype, multiply):
    """The step driven through the operation classes one Forward / Backward at a time (fresh output Matrix per call,
    results added into the gradient destinations, then GradientClipper and AdamOptimizer over the layers) against the
    oracle's composition, and against the fused launch sequence: same arithmetic per operation, so the same bits."""
    from parallelreverseautodiff_amd.feedforward import OperationWalkNetwork
    X = seeded.uniform(seeded.DEFAULT_SEED, 1, (64, 784), 0.0, 1.0, dtype)
    T = seeded.one_hot_labels(seeded.DEFAULT_SEED, 2, 64, 10, dtype)
    walk, fused = OperationWalkNetwork(dtype=dtype, multiply=multiply), FeedForwardNetwork(dtype=dtype)
    walk.set_batch(X, T); fused.set_batch(X, T)
    W = [w.copy() for w in walk.host_W]
    b = [np.zeros((1, s), dtype) for s in walk.sizes[1:]]
    m = [np.zeros_like(x) for x in W + b]
    v = [np.zeros_like(x) for x in W + b]
    for t in (1, 2, 3):
        walk.step(); fused.step()
        dev_grads = [g.to_numpy() for g in walk.dW + walk.db]
        loss, raw, clipped, new = oracle_step(oracle, W, b, m, v, X, T, walk.Parameters, t, dtype,
                                              adam_grads=dev_grads if dtype == np.float32 else None)
        assert abs(float(walk.loss.to_numpy()[0, 0]) - loss) <= (1e-12 if dtype == np.float64 else 1e-5) * abs(loss)
        for i, (g_dev, g_ref) in enumerate(zip(dev_grads, clipped)):
            assert_parity(g_dev, g_ref, dtype, "clipped gradient %d step %d" % (i, t))
        L = len(W)
        W = [n[0] for n in new[:L]]; b = [n[0] for n in new[L:]]
        m = [n[1] for n in new]; v = [n[2] for n in new]
        for i, (w_dev, w_ref) in enumerate(zip(walk.W + walk.b, W + b)):
            assert_parity(w_dev.to_numpy(), w_ref, dtype, "weight %d step %d" % (i, t))
        for i, (w_walk, w_fused) in enumerate(zip(walk.W + walk.b, fused._weights)):
            assert np.array_equal(w_walk.to_numpy(), w_fused.download()), "weight %d step %d: walk and fused sequence differ" % (i, t)


def test_operation_walk_steady_state_allocates_nothing(gpu):
    """After the first steps the walk takes every output block from the library's pool: no hipMalloc, no hipFree and
    no wait for the stream per step, although every operation returns a fresh Matrix."""
    from parallelreverseautodiff_amd.feedforward import OperationWalkNetwork
    net = OperationWalkNetwork()
    net.set_batch(seeded.uniform(5, 1, (64, 784), 0.0, 1.0), seeded.one_hot_labels(5, 2, 64, 10))
    for _ in range(3):
        net.step()
    before = _alloc_stats()
    for _ in range(5):
        net.step()
    after = _alloc_stats()
    assert after["mallocs"] == before["mallocs"] and after["frees"] == before["frees"] and after["syncs"] == before["syncs"], (before, after)
    assert after["pool_hits"] - before["pool_hits"] >= 5 * 20
    assert np.isfinite(net.loss.to_numpy()[0, 0])


@pytest.mark.parametrize("dtype", DTYPES)
def test_compiled_operation_walk_equals_the_python_walk(gpu, dtype):
    """The step walked by compiled code through the C ABI (one call per operation) gives the bits of the Python walk
    through the operation classes: same entry points in the same order."""
    from parallelreverseautodiff_amd.feedforward import OperationWalkNetwork, compiled_operation_walk
    X = seeded.uniform(seeded.DEFAULT_SEED, 1, (64, 784), 0.0, 1.0, dtype)
    T = seeded.one_hot_labels(seeded.DEFAULT_SEED, 2, 64, 10, dtype)
    walk = OperationWalkNetwork(dtype=dtype)
    walk.set_batch(X, T)
    for _ in range(4):
        walk.step()
    ms, loss, weights = compiled_operation_walk(dtype=dtype, steps=3, warmup=1)
    assert ms > 0
    assert loss == float(walk.loss.to_numpy()[0, 0])
    for got, ref in zip(weights, walk.W):
        assert np.array_equal(got, ref.to_numpy())
