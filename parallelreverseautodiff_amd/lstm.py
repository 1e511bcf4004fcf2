"""Device-resident training step of one LSTM layer with a fused 4-gate weight.

The reference unrolls a sequence into per-time-step operation nodes (src/RMAD/ComputationGraph.cs:808-849) and
runs, per step, separate MatrixMultiplyOperation / MatrixAddBroadcasting / Sigmoid / Tanh / HadamardProduct /
MatrixAdd nodes (examples/lstm/.../architecture/SelfAttentionMultiLayerLSTMArchitectureAmplified.json).  Here:

  * the input half of every step's product is one large product over the whole sequence,
    G_all = X_all . W_x + b  (rows = steps*batch), so only h_{t-1} . W_h stays inside the time loop,
    accumulated into step t's rows of G_all by the product's own epilogue;
  * the ten pointwise nodes of a step are one kernel each way (prad_lstm_cell_fwd / _bwd);
  * backward keeps only dh_{t-1} = dG_t . W_h^T in the loop; dW = [X_all | H_prev_all]^T . dG_all, the bias
    gradient and dX_all are three large products / one column sum after it.

  * where the shape allows it (float, batch a multiple of 16, hidden a multiple of 64 up to 512, one workgroup per
    compute unit) the time loop itself runs inside one kernel each way (prad_lstm_sequence_fwd / _bwd), the recurrent
    weight staying in registers for the whole sequence; otherwise one launch per time step each way.

Every value equals the node-by-node evaluation up to the order of the floating-point sums.
W is steps-independent: (input + hidden) x 4*hidden, gate blocks [i | f | g | o].
"""
import ctypes

import numpy as np

from . import _lib, seeded
from .exceptions import ArgumentException, check
from .matrix import DeviceBuffer
from .operations import _ensure_initialized, handle_array
from .optim import NeuralNetworkParameters


class LSTMLayer:
    def __init__(self, input_dim=256, hidden=512, batch=128, steps=64, dtype=np.float32, seed=seeded.DEFAULT_SEED,
                 parameters=None, fused=True, sequence=None):
        _ensure_initialized()
        self.lib = _lib.load()
        self.dtype = np.dtype(dtype)
        self.input_dim, self.hidden, self.batch, self.steps = input_dim, hidden, batch, steps
        self.params = parameters or NeuralNetworkParameters(lite=self.dtype == np.float32)
        I, H, B, T = input_dim, hidden, batch, steps
        alloc = lambda r, c: DeviceBuffer.alloc(self.dtype, r, c)
        bound = 1.0 / np.sqrt(hidden)
        self.host_W = seeded.uniform(seed, 31, (I + H, 4 * H), -bound, bound, self.dtype)
        self.host_X = seeded.normal(seed, 32, (T * B, I), 1.0, self.dtype)
        self.host_Y = seeded.normal(seed, 33, (T * B, H), 1.0, self.dtype)
        self.W, self.b = alloc(I + H, 4 * H), alloc(1, 4 * H)
        self.W.upload(self.host_W)
        self.Wx, self.Wh = self.W.view_rows(0, I), self.W.view_rows(I, H)
        self.dW, self.db = alloc(I + H, 4 * H), alloc(1, 4 * H)
        self.dWx, self.dWh = self.dW.view_rows(0, I), self.dW.view_rows(I, H)
        self.mW, self.vW, self.mb, self.vb = alloc(I + H, 4 * H), alloc(I + H, 4 * H), alloc(1, 4 * H), alloc(1, 4 * H)
        self.X, self.Y = alloc(T * B, I), alloc(T * B, H)
        self.X.upload(self.host_X)
        self.Y.upload(self.host_Y)
        self.G = alloc(T * B, 4 * H)                 # pre-activations, then activated gates, all steps
        self.C = alloc((T + 1) * B, H)               # c_0 = 0 in the first block
        self.Hs = alloc((T + 1) * B, H)              # h_0 = 0 in the first block
        self.TC = alloc(T * B, H)                    # tanh(c_t)
        self.dG, self.dHl, self.dX = alloc(T * B, 4 * H), alloc(T * B, H), alloc(T * B, I)
        self.dh = [alloc(B, H), alloc(B, H)]
        self.dc = [alloc(B, H), alloc(B, H)]
        self.loss = alloc(1, 1)
        v = lambda buf, t: buf.view_rows(t * B, B)
        self.G_t = [v(self.G, t) for t in range(T)]
        self.C_t = [v(self.C, t) for t in range(T + 1)]
        self.H_t = [v(self.Hs, t) for t in range(T + 1)]
        self.TC_t = [v(self.TC, t) for t in range(T)]
        self.dG_t = [v(self.dG, t) for t in range(T)]
        self.dHl_t = [v(self.dHl, t) for t in range(T)]
        self.H_prev_all = self.Hs.view_rows(0, T * B)
        self.H_out = self.Hs.view_rows(B, T * B)
        self.iteration = 0
        self._graph = None
        self.fused = fused   # one launch per time step each way (cell arithmetic as the recurrent product's epilogue)
        # the whole time loop in one launch each way where the shape allows it (sequence=False: never; True: required)
        supported = bool(self.lib.prad_lstm_sequence_supported(_lib.PRAD_F32 if self.dtype == np.float32 else _lib.PRAD_F64, B, H, T))
        if sequence and not supported:
            raise ArgumentException("the sequence kernels do not take this shape (float, batch % 16 == 0, hidden % 64 == 0, hidden <= 512)")
        self.sequence = supported and fused if sequence is None else bool(sequence)

    def _enqueue_forward_backward(self):
        lib, T = self.lib, self.steps
        check(lib.prad_matmul_fwd_fused(self.X.handle, self.Wx.handle, self.b.handle, None, self.G.handle, _lib.ACT_NONE, 0.0))
        if self.sequence:
            check(lib.prad_lstm_sequence_fwd(self.Wh.handle, self.G.handle, self.C.handle, self.Hs.handle, self.TC.handle, T))
        for t in range(0 if self.sequence else T):
            if self.fused:
                check(lib.prad_lstm_step_fwd(self.H_t[t].handle, self.Wh.handle, self.G_t[t].handle, self.C_t[t].handle,
                                             self.C_t[t + 1].handle, self.TC_t[t].handle, self.H_t[t + 1].handle))
                continue
            check(lib.prad_gemm(0, 0, self.H_t[t].handle, self.Wh.handle, self.G_t[t].handle, 1))  # G_t += h_{t-1} . W_h
            check(lib.prad_lstm_cell_fwd(self.G_t[t].handle, self.C_t[t].handle, self.C_t[t + 1].handle, self.TC_t[t].handle,
                                         self.H_t[t + 1].handle))
        check(lib.prad_mse(self.H_out.handle, self.Y.handle, self.loss.handle, self.dHl.handle))   # loss and its gradient
        if self.sequence:
            check(lib.prad_lstm_sequence_bwd(self.Wh.handle, self.G.handle, self.C.handle, self.TC.handle, self.dHl.handle, self.dG.handle, T))
        for t in range(-1 if self.sequence else T - 1, -1, -1):
            last = t == T - 1
            rec, dc_in, dc_out = self.dh[t % 2], self.dc[t % 2], self.dc[(t + 1) % 2]
            if self.fused and not last:
                # dh_t = dHl_t + dG_{t+1} . W_h^T and the cell's backward in one launch
                check(lib.prad_lstm_step_bwd(self.dG_t[t + 1].handle, self.Wh.handle, self.G_t[t].handle, self.C_t[t].handle,
                                             self.TC_t[t].handle, self.dHl_t[t].handle, dc_in.handle, self.dG_t[t].handle,
                                             dc_out.handle, rec.handle))
                continue
            check(lib.prad_lstm_cell_bwd(self.G_t[t].handle, self.C_t[t].handle, self.TC_t[t].handle, self.dHl_t[t].handle,
                                         None if last else rec.handle, None if last else dc_in.handle,
                                         self.dG_t[t].handle, dc_out.handle))
            if not self.fused:
                # dh_{t-1} = dG_t . W_h^T (formed for t = 0 too: MatrixMultiplyOperation.Backward always returns both gradients)
                check(lib.prad_gemm(0, 1, self.dG_t[t].handle, self.Wh.handle, self.dh[(t + 1) % 2].handle, 0))
        if self.fused or self.sequence:
            check(lib.prad_gemm(0, 1, self.dG_t[0].handle, self.Wh.handle, self.dh[1].handle, 0))   # dh_{-1}, as above
        check(lib.prad_gemm(1, 0, self.X.handle, self.dG.handle, self.dWx.handle, 0))
        check(lib.prad_gemm(1, 0, self.H_prev_all.handle, self.dG.handle, self.dWh.handle, 0))
        check(lib.prad_add_broadcast_bwd_bias(self.dG.handle, self.db.handle))
        check(lib.prad_gemm(0, 1, self.dG.handle, self.Wx.handle, self.dX.handle, 0))

    def _enqueue_update(self, t):
        p = self.params
        check(self.lib.prad_clip_adam_multi(handle_array([self.W, self.b]), handle_array([self.mW, self.mb]),
                                            handle_array([self.vW, self.vb]), handle_array([self.dW, self.db]), 2,
                                            float(p.ClipValue), float(p.MinimumClipValue), float(p.LearningRate),
                                            float(p.AdamBeta1), float(p.AdamBeta2), float(p.AdamEpsilon), float(t)))

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
            g = ctypes.c_void_p()
            check(self.lib.prad_graph_end(ctypes.byref(g)))
        self._graph = g

    def replay(self):
        """One recorded step; AdamIteration advances by one per replay."""
        check(self.lib.prad_graph_launch(self._graph))
        self.iteration += 1

    def release(self):
        if self._graph is not None:
            check(self.lib.prad_graph_destroy(self._graph))
            self._graph = None

    def flops_per_step(self):
        return 3.0 * 2.0 * self.steps * self.batch * (self.input_dim + self.hidden) * 4 * self.hidden
