"""Device-resident training step of the feed-forward configuration: the call sequence the reference's
training loop makes (forward walk over the operation list, loss, backward visitor with gradient
accumulation, clip, Adam: examples/feedforward/ParallelReverseAutoDiff.FeedForwardExample/FeedForwardNeuralNetwork.cs:212-358)
replayed on pre-allocated device buffers, either launch by launch or as one recorded submission.

Network: X (batch x n0) -> [MatrixMultiply(W_l) -> MatrixAddBroadcasting(b_l) -> LeakyReLU] x (L-1)
         -> MatrixMultiply(W_L) -> MatrixAddBroadcasting(b_L) -> Softmax -> CategoricalCrossEntropy.
Per layer the product, the bias add and the activation are one launch (fused epilogue), and the
activation's Backward is the epilogue of the next layer's dA product.  A step of this size costs what
its chain of dependent launches costs, so fused=True (the default) uses the entry points that cover
several reference operations per launch (softmax + cross-entropy forward and backward; the bias gradient
next to the weight gradient; clip + Adam).  The arithmetic of every operation is the same in both variants
and the results are bit for bit equal.
"""
import ctypes

import numpy as np

from . import _lib, seeded
from .exceptions import check
from .matrix import DeviceBuffer
from .operations import _ensure_initialized, handle_array
from .optim import NeuralNetworkParameters


class FeedForwardNetwork:
    def __init__(self, sizes=(784, 256, 128, 10), batch=64, dtype=np.float64, seed=seeded.DEFAULT_SEED, parameters=None, fused=True):
        _ensure_initialized()
        self.lib = _lib.load()
        self.dtype = np.dtype(dtype)
        self.sizes, self.batch = tuple(sizes), batch
        self.params = parameters or NeuralNetworkParameters(lite=self.dtype == np.float32)
        L = len(sizes) - 1
        alloc = lambda r, c: DeviceBuffer.alloc(self.dtype, r, c)
        # weights Xavier-uniform, biases zero (Matrix.InitializeXavier, src/RMAD/Matrix.cs:1037-1046)
        self.host_W = [seeded.xavier(seed, 10 + l, sizes[l], sizes[l + 1], self.dtype) for l in range(L)]
        self.W = [alloc(sizes[l], sizes[l + 1]) for l in range(L)]
        self.b = [alloc(1, sizes[l + 1]) for l in range(L)]
        for w, h in zip(self.W, self.host_W):
            w.upload(h)
        self.dW = [alloc(sizes[l], sizes[l + 1]) for l in range(L)]
        self.db = [alloc(1, sizes[l + 1]) for l in range(L)]
        self.mW = [alloc(sizes[l], sizes[l + 1]) for l in range(L)]
        self.vW = [alloc(sizes[l], sizes[l + 1]) for l in range(L)]
        self.mb = [alloc(1, sizes[l + 1]) for l in range(L)]
        self.vb = [alloc(1, sizes[l + 1]) for l in range(L)]
        self.X = alloc(batch, sizes[0])
        self.T = alloc(batch, sizes[-1])
        self.Z = [alloc(batch, sizes[l + 1]) for l in range(L)]      # pre-activations (what LeakyReLU caches)
        self.H = [alloc(batch, sizes[l + 1]) for l in range(L - 1)]  # activations
        self.P = alloc(batch, sizes[-1])                             # softmax output
        self.loss = alloc(1, 1)
        self.dP = alloc(batch, sizes[-1])
        self.dZ = [alloc(batch, sizes[l + 1]) for l in range(L)]
        self.dX = alloc(batch, sizes[0])
        self.iteration = 0
        self.fused = fused
        self._graph = None
        self._weights = self.W + self.b
        self._grads = self.dW + self.db
        self._m = self.mW + self.mb
        self._v = self.vW + self.vb

    def set_batch(self, X, T):
        self.X.upload(X)
        self.T.upload(T)

    # ---- one step, launch by launch ------------------------------------------------------------
    def _enqueue_forward(self, layers=None):
        lib, L, alpha = self.lib, len(self.W), float(self.params.LeakyReLUAlpha)
        a = self.X
        for l in range(L if layers is None else layers):
            last = l == L - 1
            out = self.Z[l] if last else self.H[l]
            z = None if last else self.Z[l].handle
            check(lib.prad_matmul_fwd_fused(a.handle, self.W[l].handle, self.b[l].handle, z, out.handle,
                                            _lib.ACT_NONE if last else _lib.ACT_LEAKYRELU, alpha))
            a = out

    def _enqueue_forward_backward(self):
        lib, L, alpha = self.lib, len(self.W), float(self.params.LeakyReLUAlpha)
        head = self.fused and L >= 2  # output layer, loss and the layer's backward in one call
        self._enqueue_forward(L - 1 if head else None)
        if head:
            check(lib.prad_dense_softmax_cce(self.H[L - 2].handle, self.W[-1].handle, self.b[-1].handle, self.T.handle,
                                             self.Z[-1].handle, self.P.handle, self.loss.handle, self.dP.handle, self.dZ[-1].handle,
                                             self.dZ[L - 2].handle, self.dW[-1].handle, self.db[-1].handle, 0,
                                             _lib.ACT_LEAKYRELU, self.Z[L - 2].handle, alpha))
        elif self.fused:
            check(lib.prad_softmax_cce(self.Z[-1].handle, self.T.handle, self.P.handle, self.loss.handle, self.dP.handle,
                                       self.dZ[-1].handle))
        else:
            check(lib.prad_softmax_fwd(self.Z[-1].handle, self.P.handle))
            check(lib.prad_cce_fwd(self.P.handle, self.T.handle, self.loss.handle))
            check(lib.prad_cce_bwd(self.P.handle, self.T.handle, self.dP.handle))
            check(lib.prad_softmax_bwd(self.P.handle, self.dP.handle, self.dZ[-1].handle))
        for l in range(L - 2 if head else L - 1, -1, -1):
            inp = self.X if l == 0 else self.H[l - 1]
            # MatrixMultiplyOperation.Backward always forms both gradients, also for the network input (l == 0)
            dA = self.dX if l == 0 else self.dZ[l - 1]
            act, src = (_lib.ACT_NONE, None) if l == 0 else (_lib.ACT_LEAKYRELU, self.Z[l - 1].handle)
            if self.fused:
                check(lib.prad_matmul_bias_bwd(self.dZ[l].handle, inp.handle, self.W[l].handle, dA.handle, self.dW[l].handle,
                                               self.db[l].handle, 0, act, src, alpha))
                continue
            check(lib.prad_add_broadcast_bwd_bias(self.dZ[l].handle, self.db[l].handle))
            if l == 0:
                check(lib.prad_matmul_bwd(self.dZ[0].handle, inp.handle, self.W[0].handle, self.dX.handle, self.dW[0].handle, 0, 0))
            else:
                check(lib.prad_matmul_bwd_fused(self.dZ[l].handle, inp.handle, self.W[l].handle, dA.handle,
                                                self.dW[l].handle, 0, act, src, alpha))

    def _enqueue_update(self, t):
        p = self.params
        n = len(self._grads)
        if self.fused:
            check(self.lib.prad_clip_adam_multi(handle_array(self._weights), handle_array(self._m), handle_array(self._v),
                                                handle_array(self._grads), n, float(p.ClipValue), float(p.MinimumClipValue),
                                                float(p.LearningRate), float(p.AdamBeta1), float(p.AdamBeta2),
                                                float(p.AdamEpsilon), float(t)))
            return
        check(self.lib.prad_clip_multi(handle_array(self._grads), n, float(p.ClipValue), float(p.MinimumClipValue)))
        check(self.lib.prad_adam_multi(handle_array(self._weights), handle_array(self._m), handle_array(self._v),
                                       handle_array(self._grads), n, float(p.LearningRate), float(p.AdamBeta1),
                                       float(p.AdamBeta2), float(p.AdamEpsilon), float(t)))

    def step(self):
        """Forward, loss, backward, clip, Adam (AdamIteration = step number, as the reference's caller sets it)."""
        self.iteration += 1
        self._enqueue_forward_backward()
        self._enqueue_update(self.iteration)

    # ---- one step as a recorded launch sequence ------------------------------------------------
    def record(self, adam_iteration=None):
        """Records one step; one eager step must have run before so that the shared workspace is already sized.
        The recording stands for the step after the last one taken (AdamIteration = iteration + 1) unless
        `adam_iteration` says otherwise; every replay advances AdamIteration by one, as step() does."""
        lib = self.lib
        self._recorded_from = float(self.iteration + 1 if adam_iteration is None else adam_iteration)
        self.iteration = int(self._recorded_from) - 1
        check(lib.prad_graph_begin())
        try:
            self._enqueue_forward_backward()
            self._enqueue_update(self._recorded_from)
        finally:
            g = ctypes.c_void_p()
            check(lib.prad_graph_end(ctypes.byref(g)))
        self._graph = g
        return g

    def replay(self):
        """One recorded step; AdamIteration advances by one per replay."""
        check(self.lib.prad_graph_launch(self._graph))
        self.iteration += 1

    def release(self):
        if self._graph is not None:
            check(self.lib.prad_graph_destroy(self._graph))
            self._graph = None

    def flops_per_step(self):
        fwd = sum(2.0 * self.batch * self.sizes[l] * self.sizes[l + 1] for l in range(len(self.W)))
        return 3.0 * fwd

    def parameter_count(self):
        return sum(self.sizes[l] * self.sizes[l + 1] + self.sizes[l + 1] for l in range(len(self.W)))


class OperationWalkNetwork:
    """The same network and step, driven the way the reference's own loop drives it and with nothing fused: one
    operation object per graph node, Forward called node by node in graph order, the loss, Backward called node by node
    in reverse with each node's results added into its gradient destinations (OperationBase.AccumulateGradient,
    src/RMAD/OperationBase.cs:273-304), then GradientClearer / GradientClipper / AdamOptimizer over the layers
    (examples/feedforward/ParallelReverseAutoDiff.FeedForwardExample/FeedForwardNeuralNetwork.cs:212-303,
    src/RMAD/OperationNeuralNetworkVisitor.cs:198-215, :287-329).  Every Forward / Backward returns a fresh output
    Matrix, as in the reference; those come from the library's block pool, so a step in its steady state allocates
    nothing on the device and never waits for it.  This is what an unchanged caller of the operation classes gets."""

    def __init__(self, sizes=(784, 256, 128, 10), batch=64, dtype=np.float64, seed=seeded.DEFAULT_SEED, parameters=None,
                 multiply="MatrixMultiplyOperation"):
        from . import operations as ops
        from .matrix import Matrix
        from .optim import AdamOptimizer, GradientClearer, GradientClipper, ModelLayer
        _ensure_initialized()
        self.dtype = np.dtype(dtype)
        self.sizes, self.batch = tuple(sizes), batch
        self.Parameters = parameters or NeuralNetworkParameters(lite=self.dtype == np.float32)
        L = len(sizes) - 1
        self.host_W = [seeded.xavier(seed, 10 + l, sizes[l], sizes[l + 1], self.dtype) for l in range(L)]
        self.W = [Matrix.from_numpy(w) for w in self.host_W]
        self.b = [Matrix(1, sizes[l + 1], self.dtype) for l in range(L)]
        self.layers = []
        for l in range(L):
            layer = ModelLayer().AddModelElementGroup("W", self.W[l]).AddModelElementGroup("B", self.b[l])
            self.layers.append(layer)
        self.dW = [layer["W", "Gradient"] for layer in self.layers]
        self.db = [layer["B", "Gradient"] for layer in self.layers]
        for m in self.dW + self.db + [layer[i, e] for layer in self.layers for i in ("W", "B") for e in ("FirstMoment", "SecondMoment")]:
            m.device()
        # the graph: [multiply -> add bias -> LeakyReLU] x (L - 1) -> multiply -> add bias -> softmax; loss = cross-entropy
        multiply_type = getattr(ops, multiply)
        self.nodes = []   # (operation, names of its inputs, gradient destinations per result)
        for l in range(L):
            self.nodes.append((multiply_type.Instantiate(self), ("prev", ("W", l)), (None, self.dW[l])))
            self.nodes.append((ops.MatrixAddBroadcastingOperation.Instantiate(self), ("prev", ("b", l)), (None, self.db[l])))
            self.nodes.append((ops.LeakyReLUOperation.Instantiate(self) if l < L - 1 else ops.SoftmaxOperation.Instantiate(self),
                               ("prev",), (None,)))
        self.loss_op = ops.CategoricalCrossEntropyLossOperation.Instantiate(self)
        self._accumulate = ops.accumulate_gradient
        self.clearer, self.clipper, self.adam = GradientClearer(), GradientClipper(self), AdamOptimizer(self)
        self.iteration = 0
        self.Input = self.Target = self.Output = self.loss = None

    def set_batch(self, X, T):
        from .matrix import Matrix
        self.Input, self.Target = Matrix.from_numpy(np.asarray(X, self.dtype)), Matrix.from_numpy(np.asarray(T, self.dtype))
        self.Input.device(); self.Target.device()

    def step(self):
        self.iteration += 1
        self.Parameters.AdamIteration = float(self.iteration)
        self.clearer.Clear(self.layers)
        value = self.Input
        for op, inputs, _ in self.nodes:                                   # forward walk, graph order
            args = [value if name == "prev" else (self.W if name[0] == "W" else self.b)[name[1]] for name in inputs]
            value = op.Forward(*args)
        self.Output = value
        self.loss = self.loss_op.Forward(self.Output, self.Target)
        grad = self.loss_op.Backward(self.Output).Item1
        for op, _, destinations in reversed(self.nodes):                   # backward walk
            results = op.Backward(grad).Results
            for dest, result in zip(destinations, results):
                if dest is not None:
                    self._accumulate(dest, result)
            grad = results[0]
        self.clipper.Clip(self.layers)
        self.adam.Optimize(self.layers)

    def flops_per_step(self):
        return 3.0 * sum(2.0 * self.batch * self.sizes[l] * self.sizes[l + 1] for l in range(len(self.W)))


def compiled_operation_walk(sizes=(784, 256, 128, 10), batch=64, dtype=np.float64, seed=seeded.DEFAULT_SEED, parameters=None,
                            steps=1, warmup=0, X=None, T=None):
    """The same operation-by-operation step as OperationWalkNetwork, driven by compiled code instead of Python
    (libprad_hostwalk.so, csrc/host_walk.cpp: nothing but C ABI calls, one per operation): what the boundary costs a
    compiled caller such as the reference's C# classes.  Runs `warmup` + `steps` steps from the seeded initial weights
    and returns (wall-clock ms per timed step, last loss, final weight matrices)."""
    import os
    _ensure_initialized()
    _lib.load()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libprad_hostwalk.so")
    if not os.path.exists(path):
        raise ImportError("libprad_hostwalk.so is not built (python -m parallelreverseautodiff_amd.build)")
    walk = ctypes.CDLL(path).prad_hostwalk_mlp
    walk.restype = ctypes.c_int32
    dtype = np.dtype(dtype)
    p = parameters or NeuralNetworkParameters(lite=dtype == np.float32)
    L = len(sizes) - 1
    W = [np.ascontiguousarray(seeded.xavier(seed, 10 + l, sizes[l], sizes[l + 1], dtype)) for l in range(L)]
    X = np.ascontiguousarray(seeded.uniform(seed, 1, (batch, sizes[0]), 0.0, 1.0, dtype) if X is None else np.asarray(X, dtype))
    T = np.ascontiguousarray(seeded.one_hot_labels(seed, 2, batch, sizes[-1], dtype) if T is None else np.asarray(T, dtype))
    out = [np.empty_like(w) for w in W]
    ptrs = lambda arrays: (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
    ms, loss = ctypes.c_double(), ctypes.c_double()
    d = ctypes.c_double
    check(walk(ctypes.c_int32(_lib.PRAD_F64 if dtype == np.float64 else _lib.PRAD_F32), ctypes.c_int32(batch), ctypes.c_int32(L),
               (ctypes.c_int64 * (L + 1))(*sizes), ptrs(W), ctypes.c_void_p(X.ctypes.data), ctypes.c_void_p(T.ctypes.data),
               ctypes.c_int32(steps), ctypes.c_int32(warmup), d(p.LeakyReLUAlpha), d(p.ClipValue), d(p.MinimumClipValue),
               d(p.LearningRate), d(p.AdamBeta1), d(p.AdamBeta2), d(p.AdamEpsilon), ctypes.byref(ms), ctypes.byref(loss), ptrs(out)))
    return ms.value, loss.value, out
