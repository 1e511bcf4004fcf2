"""Compositions of the oracle's per-operation restatements into whole training steps, node by node as the
reference's graph would run them.  TEST INFRASTRUCTURE ONLY (same rule as oracle.py): used by tests and by
the benchmark's cpu_baseline leg.  Both compositions are pinned by tests/test_oracle_compose.py: forward against an
independent numpy statement, gradients against central differences of it, a hand-worked single step."""
import numpy as np

from . import oracle


def lstm_forward_backward(W, b, X, Y, I, H, B, T, threads=8):
    """One LSTM layer over T steps with MSE on the stacked hidden states: returns loss, hidden states, dW, db, dX."""
    dt = W.dtype
    h, c = np.zeros((B, H), dt), np.zeros((B, H), dt)
    cache = []
    hs = []
    for t in range(T):
        xh = np.ascontiguousarray(np.concatenate([X[t * B:(t + 1) * B], h], axis=1))
        G = oracle.add_broadcast_fwd(oracle.matmul_fwd(xh, W, threads=threads), b)
        i_, f_ = oracle.sigmoid_fwd(np.ascontiguousarray(G[:, :H])), oracle.sigmoid_fwd(np.ascontiguousarray(G[:, H:2 * H]))
        g_, o_ = oracle.tanh_fwd(np.ascontiguousarray(G[:, 2 * H:3 * H])), oracle.sigmoid_fwd(np.ascontiguousarray(G[:, 3 * H:]))
        c_new = oracle.hadamard_fwd(f_, c) + oracle.hadamard_fwd(i_, g_)
        tc = oracle.tanh_fwd(c_new)
        h_new = oracle.hadamard_fwd(o_, tc)
        cache.append((xh, i_, f_, g_, o_, c, tc))
        h, c = h_new, c_new
        hs.append(h)
    Hout = np.concatenate(hs, axis=0)
    loss = oracle.mse_fwd(Hout, Y)
    dH = oracle.mse_bwd(Hout, Y)
    dW, db = np.zeros_like(W), np.zeros_like(b)
    dh_rec, dc_next = None, None
    dX = np.zeros_like(X)
    for t in range(T - 1, -1, -1):
        xh, i_, f_, g_, o_, c_prev, tc = cache[t]
        dh = dH[t * B:(t + 1) * B] if dh_rec is None else dH[t * B:(t + 1) * B] + dh_rec
        d_o, d_tc = oracle.hadamard_bwd(o_, tc, dh)          # h = o . tanh(c)
        dc = oracle.tanh_bwd(tc, d_tc)
        if dc_next is not None:
            dc = dc + dc_next
        d_f, dc_prev = oracle.hadamard_bwd(f_, c_prev, dc)   # f . c_prev
        d_i, d_g = oracle.hadamard_bwd(i_, g_, dc)           # i . g
        dG = np.concatenate([oracle.sigmoid_bwd(i_, d_i), oracle.sigmoid_bwd(f_, d_f), oracle.tanh_bwd(g_, d_g),
                             oracle.sigmoid_bwd(o_, d_o)], axis=1)
        dG = np.ascontiguousarray(dG)
        db = db + oracle.add_broadcast_bwd_bias(dG)
        dxh, dWt = oracle.matmul_bwd(dG, xh, W, threads=threads)
        dW = dW + dWt                                        # OperationBase.AccumulateGradient over the time steps
        dX[t * B:(t + 1) * B] = dxh[:, :I]
        dh_rec, dc_next = np.ascontiguousarray(dxh[:, I:]), dc_prev
    return loss, Hout, dW, db, dX


def swin_block_forward_backward(p, X, T, nw, wt, heads, threads=8):
    """Windowed self-attention block + MLP (see parallelreverseautodiff_amd/swin.py for the wiring), node by node.
    p: dict of Wqkv, bqkv, Wo, bo, W1, b1, W2, b2.  Returns loss, Y2 and the gradients of every parameter and of X."""
    dt = X.dtype
    C = X.shape[1]
    hd = C // heads
    scale = dt.type(1.0 / np.sqrt(hd))
    mm = lambda a, b: oracle.matmul_fwd(np.ascontiguousarray(a), np.ascontiguousarray(b), threads=threads)
    QKV = oracle.add_broadcast_fwd(mm(X, p["Wqkv"]), p["bqkv"])
    O = np.zeros_like(X)
    P_all = {}
    for w in range(nw):
        r = slice(w * wt, (w + 1) * wt)
        for h in range(heads):
            Q, K, V = (np.ascontiguousarray(QKV[r, o + h * hd:o + (h + 1) * hd]) for o in (0, C, 2 * C))
            S = oracle.matmul_fwd(Q, np.ascontiguousarray(K.T)) * scale
            P = oracle.softmax_fwd(np.ascontiguousarray(S))
            P_all[(w, h)] = P
            O[r, h * hd:(h + 1) * hd] = oracle.matmul_fwd(P, V)
    Y1 = oracle.add_broadcast_fwd(mm(O, p["Wo"]), p["bo"])
    Z1 = oracle.add_broadcast_fwd(mm(Y1, p["W1"]), p["b1"])
    H1 = oracle.gelu_fwd(Z1)
    Y2 = oracle.add_broadcast_fwd(mm(H1, p["W2"]), p["b2"])
    loss = oracle.mse_fwd(Y2, T)
    g = {}
    dY2 = oracle.mse_bwd(Y2, T)
    g["b2"] = oracle.add_broadcast_bwd_bias(dY2)
    dH1, g["W2"] = oracle.matmul_bwd(dY2, H1, p["W2"], threads=threads)
    dZ1 = oracle.gelu_bwd(Z1, dH1)
    g["b1"] = oracle.add_broadcast_bwd_bias(dZ1)
    dY1, g["W1"] = oracle.matmul_bwd(dZ1, Y1, p["W1"], threads=threads)
    g["bo"] = oracle.add_broadcast_bwd_bias(dY1)
    dO, g["Wo"] = oracle.matmul_bwd(dY1, O, p["Wo"], threads=threads)
    dQKV = np.zeros_like(QKV)
    for w in range(nw):
        r = slice(w * wt, (w + 1) * wt)
        for h in range(heads):
            Q, K, V = (np.ascontiguousarray(QKV[r, o + h * hd:o + (h + 1) * hd]) for o in (0, C, 2 * C))
            P = P_all[(w, h)]
            dOh = np.ascontiguousarray(dO[r, h * hd:(h + 1) * hd])
            dP, dV = oracle.matmul_bwd(dOh, P, V)                       # O = P . V
            dS = oracle.softmax_bwd(P, dP) * scale
            dQ, dKt = oracle.matmul_bwd(np.ascontiguousarray(dS), Q, np.ascontiguousarray(K.T))   # S = Q . K^T
            dQKV[r, h * hd:(h + 1) * hd] = dQ
            dQKV[r, C + h * hd:C + (h + 1) * hd] = dKt.T
            dQKV[r, 2 * C + h * hd:2 * C + (h + 1) * hd] = dV
    g["bqkv"] = oracle.add_broadcast_bwd_bias(dQKV)
    dX, g["Wqkv"] = oracle.matmul_bwd(dQKV, X, p["Wqkv"], threads=threads)
    return loss, Y2, g, dX
