"""Device-resident training step of a Swin-style windowed self-attention block (shape specification:
examples/swin/SwinExample/SwinTransformerTools.cs:325-411 for the attention, :157-190 for the MLP).

Tokens arrive window-major: rows [w*49, (w+1)*49) of X are the 7 x 7 tokens of window w.  The block is
  QKV = X . Wqkv + b            per window w and head h (32 columns each):
  S   = Q_wh . K_wh^T * 1/sqrt(32)   (MatrixMultiply, MatrixMultiplyScalar)
  P   = softmax rows(S)              (SoftmaxOperation; the reference example uses its SymmetricSoftmax variant)
  O_wh = P . V_wh
  Y1 = O . Wo + bo ;  Y2 = GELU(Y1 . W1 + b1) . W2 + b2   (GELUOperation, with the reference's own derivative)
  loss = MSE(Y2, target)
and the backward of every node in reverse order, then clip and Adam.  The 3 x windows small products of a kind
are one launch over windows x heads (two-level strided batch over the columns of the shared QKV / gradient
matrices, no gather).
"""
import ctypes

import numpy as np

from . import _lib, seeded
from .exceptions import check
from .matrix import DeviceBuffer
from .operations import _ensure_initialized, handle_array
from .optim import NeuralNetworkParameters


class SwinBlock:
    def __init__(self, images=16, side=56, window=7, embed=96, heads=3, mlp_ratio=4, dtype=np.float32,
                 seed=seeded.DEFAULT_SEED, parameters=None, fused_attention=None):
        _ensure_initialized()
        self.lib = _lib.load()
        self.dtype = np.dtype(dtype)
        self.params = parameters or NeuralNetworkParameters(lite=self.dtype == np.float32)
        self.C, self.heads, self.hd = embed, heads, embed // heads
        self.wt = window * window                                  # tokens per window
        self.nw = images * (side // window) ** 2                   # windows
        self.tokens = self.nw * self.wt
        self.hidden = mlp_ratio * embed
        C, Hd, N = self.C, self.hidden, self.tokens
        alloc = lambda r, c: DeviceBuffer.alloc(self.dtype, r, c)
        shapes = {"Wqkv": (C, 3 * C), "bqkv": (1, 3 * C), "Wo": (C, C), "bo": (1, C), "W1": (C, Hd), "b1": (1, Hd),
                  "W2": (Hd, C), "b2": (1, C)}
        self.names = list(shapes)
        self.host = {}
        for i, (k, shp) in enumerate(shapes.items()):
            self.host[k] = (seeded.normal(seed, 40 + i, shp, 0.02, self.dtype) if k.startswith("W")
                            else np.zeros(shp, self.dtype))
        self.host["X"] = seeded.normal(seed, 60, (N, C), 1.0, self.dtype)
        self.host["T"] = seeded.normal(seed, 61, (N, C), 1.0, self.dtype)
        self.w = {k: alloc(*shapes[k]) for k in shapes}
        self.g = {k: alloc(*shapes[k]) for k in shapes}
        self.m = {k: alloc(*shapes[k]) for k in shapes}
        self.v = {k: alloc(*shapes[k]) for k in shapes}
        for k in shapes:
            self.w[k].upload(self.host[k])
        self.X, self.T = alloc(N, C), alloc(N, C)
        self.X.upload(self.host["X"]); self.T.upload(self.host["T"])
        self.QKV, self.dQKV = alloc(N, 3 * C), alloc(N, 3 * C)
        srows = heads * self.nw * self.wt
        self.S, self.P, self.dP, self.dS = alloc(srows, self.wt), alloc(srows, self.wt), alloc(srows, self.wt), alloc(srows, self.wt)
        self.O, self.dO = alloc(N, C), alloc(N, C)
        self.Y1, self.dY1 = alloc(N, C), alloc(N, C)
        self.Z1, self.H1, self.dZ1 = alloc(N, Hd), alloc(N, Hd), alloc(N, Hd)
        self.Y2, self.dY2, self.dX = alloc(N, C), alloc(N, C), alloc(N, C)
        self.loss = alloc(1, 1)
        self.scale = 1.0 / float(np.sqrt(self.hd))
        self.iteration = 0
        self._graph = None
        supported = bool(self.lib.prad_window_attention_supported(_lib.PRAD_F32 if self.dtype == np.float32 else _lib.PRAD_F64, self.wt, self.hd))
        self.fused_attention = supported if fused_attention is None else bool(fused_attention) and supported
        self._batched = (self.lib.prad_gemm_strided_batched_2d_f64 if self.dtype == np.float64
                         else self.lib.prad_gemm_strided_batched_2d_f32)

    def _ptr(self, buf, elem_offset):
        return ctypes.c_void_p(buf.ptr + elem_offset * self.dtype.itemsize)

    def _all_heads(self, tA, tB, M, N, K, A, a_off, lda, sA, hA, B, b_off, ldb, sB, hB, Cb, c_off, ldc, sC, hC):
        """One launch over windows x heads: s* are the element strides between windows, h* between heads."""
        check(self._batched(tA, tB, M, N, K, self._ptr(A, a_off), lda, sA, hA, self._ptr(B, b_off), ldb, sB, hB,
                            self._ptr(Cb, c_off), ldc, sC, hC, self.nw, self.heads, 0))

    def _enqueue_forward_backward(self):
        lib, C, wt, hd, nw = self.lib, self.C, self.wt, self.hd, self.nw
        w, g = self.w, self.g
        q3 = 3 * C
        fused = lib.prad_matmul_fwd_fused
        check(fused(self.X.handle, w["Wqkv"].handle, w["bqkv"].handle, None, self.QKV.handle, _lib.ACT_NONE, 0.0))
        hs = nw * wt * wt                 # scores are stored head-major: [head][window][wt][wt]
        if self.fused_attention:
            # scores, softmax and P . V of every window and head in one launch; the scores never reach memory
            check(lib.prad_window_attention_fwd(self.QKV.handle, self.P.handle, self.O.handle, nw, self.heads, wt, self.scale))
        else:
            # S = Q . K^T per window and head
            self._all_heads(0, 1, wt, wt, hd, self.QKV, 0, q3, wt * q3, hd, self.QKV, C, q3, wt * q3, hd, self.S, 0, wt, wt * wt, hs)
            check(lib.prad_softmax_scaled_fwd(self.S.handle, self.scale, self.P.handle))   # P = softmax(S / sqrt(head dim))
            # O = P . V per window, written into each head's columns of O
            self._all_heads(0, 0, wt, hd, wt, self.P, 0, wt, wt * wt, hs, self.QKV, 2 * C, q3, wt * q3, hd, self.O, 0, C, wt * C, hd)
        check(fused(self.O.handle, w["Wo"].handle, w["bo"].handle, None, self.Y1.handle, _lib.ACT_NONE, 0.0))
        check(fused(self.Y1.handle, w["W1"].handle, w["b1"].handle, self.Z1.handle, self.H1.handle, _lib.ACT_GELU, 0.0))
        check(fused(self.H1.handle, w["W2"].handle, w["b2"].handle, None, self.Y2.handle, _lib.ACT_NONE, 0.0))
        check(lib.prad_mse(self.Y2.handle, self.T.handle, self.loss.handle, self.dY2.handle))   # loss and its gradient
        # ---- backward ----
        # (a layer's input, weight and bias gradients in one call: in float the weight gradient of these tall batches is
        # one pass over the layer's input and dZ, and the bias gradient - the column sums of dZ - is taken in that pass)
        check(lib.prad_matmul_bias_bwd(self.dY2.handle, self.H1.handle, w["W2"].handle, self.dZ1.handle, g["W2"].handle, g["b2"].handle, 0,
                                       _lib.ACT_GELU, self.Z1.handle, 0.0))
        check(lib.prad_matmul_bias_bwd(self.dZ1.handle, self.Y1.handle, w["W1"].handle, self.dY1.handle, g["W1"].handle, g["b1"].handle, 0,
                                       _lib.ACT_NONE, None, 0.0))
        check(lib.prad_matmul_bias_bwd(self.dY1.handle, self.O.handle, w["Wo"].handle, self.dO.handle, g["Wo"].handle, g["bo"].handle, 0,
                                       _lib.ACT_NONE, None, 0.0))
        if self.fused_attention:
            # dP, dV, the softmax's backward, dQ and dK of every window and head in one launch; dP and dS never reach memory
            check(lib.prad_window_attention_bwd(self.QKV.handle, self.P.handle, self.dO.handle, self.dQKV.handle, nw, self.heads, wt, self.scale))
        else:
            # dP = dO . V^T ; dV = P^T . dO
            self._all_heads(0, 1, wt, wt, hd, self.dO, 0, C, wt * C, hd, self.QKV, 2 * C, q3, wt * q3, hd, self.dP, 0, wt, wt * wt, hs)
            self._all_heads(1, 0, wt, hd, wt, self.P, 0, wt, wt * wt, hs, self.dO, 0, C, wt * C, hd, self.dQKV, 2 * C, q3, wt * q3, hd)
            check(lib.prad_softmax_scaled_bwd(self.P.handle, self.dP.handle, self.scale, self.dS.handle))
            # dQ = dS . K ; dK = dS^T . Q
            self._all_heads(0, 0, wt, hd, wt, self.dS, 0, wt, wt * wt, hs, self.QKV, C, q3, wt * q3, hd, self.dQKV, 0, q3, wt * q3, hd)
            self._all_heads(1, 0, wt, hd, wt, self.dS, 0, wt, wt * wt, hs, self.QKV, 0, q3, wt * q3, hd, self.dQKV, C, q3, wt * q3, hd)
        check(lib.prad_matmul_bias_bwd(self.dQKV.handle, self.X.handle, w["Wqkv"].handle, self.dX.handle, g["Wqkv"].handle, g["bqkv"].handle, 0,
                                       _lib.ACT_NONE, None, 0.0))

    def _enqueue_update(self, t):
        p, n = self.params, len(self.names)
        arr = lambda d: handle_array([d[k] for k in self.names])
        check(self.lib.prad_clip_adam_multi(arr(self.w), arr(self.m), arr(self.v), arr(self.g), n, float(p.ClipValue),
                                            float(p.MinimumClipValue), float(p.LearningRate), float(p.AdamBeta1),
                                            float(p.AdamBeta2), float(p.AdamEpsilon), float(t)))

    def step(self, update=True):
        self.iteration += 1
        self._enqueue_forward_backward()
        if update:
            self._enqueue_update(self.iteration)

    def record(self, adam_iteration=None):
        self._recorded_from = float(self.iteration + 1 if adam_iteration is None else adam_iteration)
        self.iteration = int(self._recorded_from) - 1
        check(self.lib.prad_graph_begin())
        try:
            self._enqueue_forward_backward()
            self._enqueue_update(self._recorded_from)
        finally:
            gr = ctypes.c_void_p()
            check(self.lib.prad_graph_end(ctypes.byref(gr)))
        self._graph = gr

    def replay(self):
        """One recorded step; AdamIteration advances by one per replay."""
        check(self.lib.prad_graph_launch(self._graph))
        self.iteration += 1

    def release(self):
        if self._graph is not None:
            check(self.lib.prad_graph_destroy(self._graph))
            self._graph = None

    def flops_per_step(self):
        N, C, Hd, wt, hd = self.tokens, self.C, self.hidden, self.wt, self.hd
        fwd = 2.0 * N * C * 3 * C + 2.0 * N * C * C + 2.0 * 2.0 * N * C * Hd + 2.0 * 2.0 * self.nw * self.heads * wt * wt * hd
        return 3.0 * fwd
