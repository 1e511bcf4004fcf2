"""Windowed self-attention block step against the oracle's node-by-node composition (reduced sizes; the
strided-batched entry point is also checked on its own)."""
import ctypes

import numpy as np
import pytest

from conftest import assert_long_sum_parity, assert_parity, norm_err, strict_err
from oracle import compose
from parallelreverseautodiff_amd import _lib, seeded
from parallelreverseautodiff_amd.matrix import DeviceBuffer
from parallelreverseautodiff_amd.swin import SwinBlock

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,cfg", [(np.float64, (1, 14, 32, 2)), (np.float32, (1, 14, 32, 2)), (np.float32, (2, 28, 96, 3))])
def test_swin_block_matches_node_by_node_oracle(gpu, oracle, dtype, cfg):
    images, side, embed, heads = cfg
    blk = SwinBlock(images=images, side=side, embed=embed, heads=heads, dtype=dtype)
    blk.step(update=False)
    params = {k: blk.host[k] for k in blk.names}
    loss, Y2, g, dX = compose.swin_block_forward_backward(params, blk.host["X"], blk.host["T"], blk.nw, blk.wt, heads)
    tol = 1e-12 if dtype == np.float64 else 1e-5
    assert abs(float(blk.loss.download()[0, 0]) - loss) <= tol * abs(loss)
    assert_parity(blk.Y2.download(), Y2, dtype, "block output")
    for k in blk.names:
        assert_parity(blk.g[k].download(), g[k], dtype, "gradient of " + k)
    assert_parity(blk.dX.download(), dX, dtype, "dX")


def test_swin_block_with_separate_attention_launches(gpu, oracle):
    """The float block with the attention nodes as separate launches (strided-batched products, scaled softmax and its
    backward) instead of one launch each way: against the oracle, and against the block as it runs by default."""
    cfg = dict(images=2, side=28, embed=96, heads=3, dtype=np.float32)
    apart, fused = SwinBlock(fused_attention=False, **cfg), SwinBlock(**cfg)
    assert not apart.fused_attention and fused.fused_attention
    apart.step(update=False); fused.step(update=False)
    params = {k: apart.host[k] for k in apart.names}
    loss, Y2, g, dX = compose.swin_block_forward_backward(params, apart.host["X"], apart.host["T"], apart.nw, apart.wt, 3)
    assert abs(float(apart.loss.download()[0, 0]) - loss) <= 1e-5 * abs(loss)
    assert_parity(apart.Y2.download(), Y2, np.float32, "block output")
    assert_parity(apart.dX.download(), dX, np.float32, "dX")
    for k in apart.names:
        assert_parity(apart.g[k].download(), g[k], np.float32, "gradient of " + k)
        assert_parity(fused.g[k].download(), apart.g[k].download(), np.float32, "gradient of %s, one launch against separate ones" % k)
    assert_parity(fused.dQKV.download(), apart.dQKV.download(), np.float32, "dQKV, one launch against separate ones")


def test_swin_benchmark_configuration_full_size(gpu, oracle):
    """The configuration the benchmark times, at its full size: 16 images of 56 x 56 tokens in 7 x 7 windows, embed 96,
    3 heads, float (50 176 token rows, 1024 windows).  The four weight gradients are sums over all 50 176 rows: see
    assert_long_sum_parity (the reference's k-ascending float loop is the less accurate side there)."""
    blk = SwinBlock(images=16, side=56, embed=96, heads=3, dtype=np.float32)
    assert blk.nw == 1024 and blk.wt == 49
    blk.step(update=False)
    params = {k: blk.host[k] for k in blk.names}
    loss, Y2, g, dX = compose.swin_block_forward_backward(params, blk.host["X"], blk.host["T"], blk.nw, blk.wt, 3, threads=16)
    assert abs(float(blk.loss.download()[0, 0]) - loss) <= 1e-5 * abs(loss)
    for what, got, ref in [("block output", blk.Y2, Y2), ("dX", blk.dX, dX)] + [("gradient of " + k, blk.g[k], g[k]) for k in blk.names if k.startswith("b")]:
        x = got.download()
        err = assert_parity(x, ref, np.float32, what)
        print("Swin 16/56/96/3 float %s: relative %.2e, normwise %.2e, floor 1e-3 rms %.2e" % (what, err, norm_err(x, ref), strict_err(x, ref)))
    operands = {"W2": (blk.H1, blk.dY2), "W1": (blk.Y1, blk.dZ1), "Wo": (blk.O, blk.dY1), "Wqkv": (blk.X, blk.dQKV)}
    for k, (lhs, rhs) in operands.items():
        errs = assert_long_sum_parity(blk.g[k].download(), g[k], lhs.download(), rhs.download(), np.float32, "gradient of " + k)
        print("Swin 16/56/96/3 float gradient of %s (K = 50176): against the reference %.2e; against the double product: device %.2e, "
              "reference arithmetic %.2e" % ((k,) + errs))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_strided_batched_products_on_column_blocks(gpu, oracle, dtype):
    """49 x 32 blocks taken out of a wide matrix by leading dimension and stride, all three orientations."""
    lib = _lib.load()
    from parallelreverseautodiff_amd.exceptions import check
    fn = lib.prad_gemm_strided_batched_f64 if dtype == np.float64 else lib.prad_gemm_strided_batched_f32
    nb, m, k, ld = 7, 49, 32, 96
    A = seeded.normal(9, 1, (nb * m, ld), 1.0, dtype)
    B = seeded.normal(9, 2, (nb * m, ld), 1.0, dtype)
    dA, dB = DeviceBuffer.alloc(dtype, nb * m, ld), DeviceBuffer.alloc(dtype, nb * m, ld)
    dA.upload(A); dB.upload(B)
    es = np.dtype(dtype).itemsize
    S = DeviceBuffer.alloc(dtype, nb * m, m)
    check(fn(0, 1, m, m, k, ctypes.c_void_p(dA.ptr + 32 * es), ld, m * ld, ctypes.c_void_p(dB.ptr + 64 * es), ld, m * ld,
             ctypes.c_void_p(S.ptr), m, m * m, nb, 0))
    got = S.download()
    for b in range(nb):
        a_blk = np.ascontiguousarray(A[b * m:(b + 1) * m, 32:64]); b_blk = np.ascontiguousarray(B[b * m:(b + 1) * m, 64:96])
        assert_parity(got[b * m:(b + 1) * m], oracle.matmul_fwd(a_blk, np.ascontiguousarray(b_blk.T)), dtype, "Q.K^T")
    O = DeviceBuffer.alloc(dtype, nb * m, ld)
    check(fn(1, 0, m, k, m, ctypes.c_void_p(S.ptr), m, m * m, ctypes.c_void_p(dB.ptr), ld, m * ld, ctypes.c_void_p(O.ptr + 32 * es),
             ld, m * ld, nb, 0))
    out = O.download()
    for b in range(nb):
        ref = oracle.matmul_fwd(np.ascontiguousarray(got[b * m:(b + 1) * m].T), np.ascontiguousarray(B[b * m:(b + 1) * m, 0:32]))
        assert_parity(out[b * m:(b + 1) * m, 32:64], ref, dtype, "S^T.B")
    assert not out[:, :32].any() and not out[:, 64:].any()  # neighbouring column blocks untouched
    assert fn(0, 0, m, k, m, ctypes.c_void_p(S.ptr), m, m * m, ctypes.c_void_p(dB.ptr), ld, m * ld, ctypes.c_void_p(O.ptr), ld, 10, nb, 0) \
        == _lib.PRAD_ERR_ARG  # overlapping outputs


@pytest.mark.parametrize("cfg", [(64, 3, 49), (5, 2, 64), (7, 4, 16), (33, 1, 33), (3, 3, 1), (9, 2, 52), (4, 2, 50)])
def test_attention_of_all_windows_and_heads_in_one_launch(gpu, oracle, cfg):
    """Scores, scaling, softmax and P . V per window and head in one launch (float, head dimension 32): P and O against
    the three launches they stand for (strided-batched products and the scaled softmax) and against numpy in double;
    windows that fill the 64-token tile, the 49 of the benchmark, small and odd ones."""
    import ctypes
    from parallelreverseautodiff_amd import _lib, seeded
    from parallelreverseautodiff_amd.exceptions import ArgumentException, check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    nw, heads, wt = cfg
    hd, dtype = 32, np.float32
    C = heads * hd
    assert lib.prad_window_attention_supported(_lib.PRAD_F32, wt, hd) == 1
    assert lib.prad_window_attention_supported(_lib.PRAD_F64, wt, hd) == 0 and lib.prad_window_attention_supported(_lib.PRAD_F32, 65, hd) == 0
    QKV = seeded.normal(77, 1, (nw * wt, 3 * C), 1.0, dtype)
    scale = 1.0 / np.sqrt(hd)
    bQKV = DeviceBuffer.alloc(dtype, *QKV.shape); bQKV.upload(QKV)
    P1, O1 = DeviceBuffer.alloc(dtype, heads * nw * wt, wt), DeviceBuffer.alloc(dtype, nw * wt, C)
    check(lib.prad_window_attention_fwd(bQKV.handle, P1.handle, O1.handle, nw, heads, wt, scale))
    # the three launches
    S, P2, O2 = DeviceBuffer.alloc(dtype, heads * nw * wt, wt), DeviceBuffer.alloc(dtype, heads * nw * wt, wt), DeviceBuffer.alloc(dtype, nw * wt, C)
    ptr = lambda b, off: ctypes.c_void_p(b.ptr + off * 4)
    q3, hs = 3 * C, nw * wt * wt
    check(lib.prad_gemm_strided_batched_2d_f32(0, 1, wt, wt, hd, ptr(bQKV, 0), q3, wt * q3, hd, ptr(bQKV, C), q3, wt * q3, hd,
                                               ptr(S, 0), wt, wt * wt, hs, nw, heads, 0))
    check(lib.prad_softmax_scaled_fwd(S.handle, scale, P2.handle))
    check(lib.prad_gemm_strided_batched_2d_f32(0, 0, wt, hd, wt, ptr(P2, 0), wt, wt * wt, hs, ptr(bQKV, 2 * C), q3, wt * q3, hd,
                                               ptr(O2, 0), C, wt * C, hd, nw, heads, 0))
    gP, gO = P1.download(), O1.download()
    assert_parity(gP, P2.download(), dtype, "P against the separate launches")
    assert_parity(gO, O2.download(), dtype, "O against the separate launches")
    # numpy in double
    X = QKV.astype(np.float64).reshape(nw, wt, 3, heads, hd)
    Sd = np.einsum("wihd,wjhd->hwij", X[:, :, 0], X[:, :, 1]) * scale
    Pd = np.exp(Sd - Sd.max(axis=-1, keepdims=True)); Pd /= Pd.sum(axis=-1, keepdims=True)
    Od = np.einsum("hwij,wjhd->wihd", Pd, X[:, :, 2]).reshape(nw * wt, C)
    assert_parity(gP, Pd.reshape(heads * nw * wt, wt).astype(dtype), dtype, "P against numpy")
    assert_parity(gO, Od.astype(dtype), dtype, "O against numpy")
    with pytest.raises(ArgumentException):
        check(lib.prad_window_attention_fwd(bQKV.handle, P1.handle, O1.handle, nw, heads, wt + 1, scale))   # rows do not match


@pytest.mark.parametrize("cfg", [(64, 3, 49), (5, 2, 64), (7, 4, 16), (33, 1, 33), (3, 3, 1), (9, 2, 52)])
def test_attention_backward_of_all_windows_and_heads_in_one_launch(gpu, oracle, cfg):
    """dQ, dK and dV of every window and head from dO and the forward's P in one launch, against the five launches it
    stands for (four strided-batched products and the scaled softmax's backward) and against numpy in double; the
    gradient buffer starts out full of NaN, so a cell the launch leaves unwritten shows."""
    import ctypes
    from parallelreverseautodiff_amd import _lib, seeded
    from parallelreverseautodiff_amd.exceptions import ArgumentException, check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    nw, heads, wt = cfg
    hd, dtype = 32, np.float32
    C = heads * hd
    QKV = seeded.normal(78, 1, (nw * wt, 3 * C), 1.0, dtype)
    dO = seeded.normal(78, 2, (nw * wt, C), 1.0, dtype)
    scale = 1.0 / np.sqrt(hd)
    alloc = lambda r, c: DeviceBuffer.alloc(dtype, r, c)
    bQKV, bdO = alloc(*QKV.shape), alloc(*dO.shape)
    bQKV.upload(QKV); bdO.upload(dO)
    P, O = alloc(heads * nw * wt, wt), alloc(nw * wt, C)
    check(lib.prad_window_attention_fwd(bQKV.handle, P.handle, O.handle, nw, heads, wt, scale))
    d1, d2 = alloc(nw * wt, 3 * C), alloc(nw * wt, 3 * C)
    d1.upload(np.full((nw * wt, 3 * C), np.nan, dtype))
    check(lib.prad_window_attention_bwd(bQKV.handle, P.handle, bdO.handle, d1.handle, nw, heads, wt, scale))
    # the five launches
    dP, dS = alloc(heads * nw * wt, wt), alloc(heads * nw * wt, wt)
    ptr = lambda b, off: ctypes.c_void_p(b.ptr + off * 4)
    q3, hs = 3 * C, nw * wt * wt
    bat = lib.prad_gemm_strided_batched_2d_f32
    check(bat(0, 1, wt, wt, hd, ptr(bdO, 0), C, wt * C, hd, ptr(bQKV, 2 * C), q3, wt * q3, hd, ptr(dP, 0), wt, wt * wt, hs, nw, heads, 0))
    check(bat(1, 0, wt, hd, wt, ptr(P, 0), wt, wt * wt, hs, ptr(bdO, 0), C, wt * C, hd, ptr(d2, 2 * C), q3, wt * q3, hd, nw, heads, 0))
    check(lib.prad_softmax_scaled_bwd(P.handle, dP.handle, scale, dS.handle))
    check(bat(0, 0, wt, hd, wt, ptr(dS, 0), wt, wt * wt, hs, ptr(bQKV, C), q3, wt * q3, hd, ptr(d2, 0), q3, wt * q3, hd, nw, heads, 0))
    check(bat(1, 0, wt, hd, wt, ptr(dS, 0), wt, wt * wt, hs, ptr(bQKV, 0), q3, wt * q3, hd, ptr(d2, C), q3, wt * q3, hd, nw, heads, 0))
    g1 = d1.download()
    assert np.isfinite(g1).all(), "cells left unwritten"
    assert_parity(g1, d2.download(), dtype, "dQKV against the separate launches")
    # numpy in double, from the same P
    X = QKV.astype(np.float64).reshape(nw, wt, 3, heads, hd)
    G = dO.astype(np.float64).reshape(nw, wt, heads, hd)
    Pd = P.download().astype(np.float64).reshape(heads, nw, wt, wt)
    dPd = np.einsum("wihd,wjhd->hwij", G, X[:, :, 2])
    dSd = Pd * (dPd - (dPd * Pd).sum(axis=-1, keepdims=True)) * scale
    ref = np.empty((nw, wt, 3, heads, hd))
    ref[:, :, 0] = np.einsum("hwij,wjhd->wihd", dSd, X[:, :, 1])
    ref[:, :, 1] = np.einsum("hwij,wihd->wjhd", dSd, X[:, :, 0])
    ref[:, :, 2] = np.einsum("hwij,wihd->wjhd", Pd, G)
    assert_parity(g1, ref.reshape(nw * wt, 3 * C).astype(dtype), dtype, "dQKV against numpy")
    with pytest.raises(ArgumentException):
        check(lib.prad_window_attention_bwd(bQKV.handle, P.handle, bdO.handle, bQKV.handle, nw, heads, wt, scale))   # output over an input
    with pytest.raises(ArgumentException):
        check(lib.prad_window_attention_bwd(bQKV.handle, P.handle, O.handle, d1.handle, nw, heads, wt + 1, scale))  # rows do not match
