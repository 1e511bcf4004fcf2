"""The classifier's output layer with softmax, cross-entropy and the layer's backward in one call
(prad_dense_softmax_cce): every output equals, bit for bit, what the three calls it stands for give
(prad_matmul_fwd_fused, prad_softmax_cce, prad_matmul_bias_bwd), for shapes that run as one launch and for shapes that
fall back to the separate launches; and the values are those of the oracle's operations."""
import numpy as np
import pytest

from conftest import TOL, rel_err
from parallelreverseautodiff_amd import _lib, seeded
from parallelreverseautodiff_amd.exceptions import ArgumentException, InvalidOperationException, check
from parallelreverseautodiff_amd.matrix import DeviceBuffer

pytestmark = pytest.mark.gpu

ACTS = {"none": _lib.ACT_NONE, "leakyrelu": _lib.ACT_LEAKYRELU, "tanh": _lib.ACT_TANH, "gelu": _lib.ACT_GELU}


def dev(a):
    b = DeviceBuffer.alloc(a.dtype.type, a.shape[0], a.shape[1])
    b.upload(a)
    return b


def operands(dtype, B, H, C, seed):
    A = seeded.normal(seed, 1, (B, H), 1.0, dtype)
    W = seeded.normal(seed, 2, (H, C), 0.3, dtype)
    b = seeded.normal(seed, 3, (1, C), 0.2, dtype)
    S = seeded.normal(seed, 4, (B, H), 1.0, dtype)             # what the activation below cached
    T = np.zeros((B, C), dtype)
    T[np.arange(B), (np.arange(B) * 7 + seed) % C] = 1
    if B > 2:
        T[2] = 0                                               # a row without a class: sums of zeros of either sign
    dW0 = seeded.normal(seed, 5, (H, C), 1.0, dtype)           # what dW holds before an accumulating call
    return A, W, b, S, T, dW0


def run(lib, one_call, dtype, A, W, b, S, T, dW0, act, accumulate, alpha=0.01):
    B, H = A.shape
    C = W.shape[1]
    dA_, dW_, db_, dS_, dT_ = dev(A), dev(W), dev(b), dev(S), dev(T)
    alloc = lambda r, c: DeviceBuffer.alloc(dtype, r, c)
    Z, P, loss, dP, dZ, gA, gb = alloc(B, C), alloc(B, C), alloc(1, 1), alloc(B, C), alloc(B, C), alloc(B, H), alloc(1, C)
    gW = dev(dW0)
    src = dS_.handle if act != _lib.ACT_NONE else None
    if one_call:
        check(lib.prad_dense_softmax_cce(dA_.handle, dW_.handle, db_.handle, dT_.handle, Z.handle, P.handle, loss.handle, dP.handle,
                                         dZ.handle, gA.handle, gW.handle, gb.handle, accumulate, act, src, alpha))
    else:
        check(lib.prad_matmul_fwd_fused(dA_.handle, dW_.handle, db_.handle, None, Z.handle, _lib.ACT_NONE, alpha))
        check(lib.prad_softmax_cce(Z.handle, dT_.handle, P.handle, loss.handle, dP.handle, dZ.handle))
        check(lib.prad_matmul_bias_bwd(dZ.handle, dA_.handle, dW_.handle, gA.handle, gW.handle, gb.handle, accumulate, act, src, alpha))
    return {k: v.download() for k, v in dict(Z=Z, P=P, loss=loss, dP=dP, dZ=dZ, dA=gA, dW=gW, db=gb).items()}


# (batch, inputs, classes): the benchmark's output layer; ragged everything; one row; 16, 17 and 64 classes (row segments of
# 16, 32 and 64 lanes); inputs that are no multiple of the vector length; a batch beyond one pass of the softmax rows
SHAPES = [(64, 128, 10), (37, 50, 7), (1, 16, 3), (64, 64, 16), (48, 96, 17), (20, 40, 64), (130, 33, 5), (256, 24, 2)]


@pytest.mark.parametrize("dtype", [np.float64, np.float32], ids=["f64", "f32"])
@pytest.mark.parametrize("B,H,C", SHAPES)
def test_one_call_gives_the_bits_of_the_three_calls(gpu, dtype, B, H, C):
    lib = _lib.load()
    ops = operands(dtype, B, H, C, 5)
    for act, accumulate in (("leakyrelu", 0), ("none", 0), ("tanh", 1), ("gelu", 0)):
        one = run(lib, True, dtype, *ops, ACTS[act], accumulate)
        three = run(lib, False, dtype, *ops, ACTS[act], accumulate)
        for k in one:
            assert np.array_equal(one[k], three[k], equal_nan=True), (k, act, np.max(np.abs(one[k] - three[k])))


@pytest.mark.parametrize("dtype", [np.float64, np.float32], ids=["f64", "f32"])
def test_values_are_the_oracles(gpu, oracle, dtype):
    lib = _lib.load()
    B, H, C = 64, 128, 10
    A, W, b, S, T, dW0 = operands(dtype, B, H, C, 9)
    T[2, 3] = 1
    got = run(lib, True, dtype, A, W, b, S, T, dW0, _lib.ACT_LEAKYRELU, 0)
    tol = TOL[np.dtype(dtype)]
    Z = oracle.add_broadcast_fwd(oracle.matmul_fwd(A, W), b)
    P = oracle.softmax_fwd(Z)
    loss = oracle.cce_fwd(P, T)
    dP = oracle.cce_bwd(P, T)
    dZ = oracle.softmax_bwd(P, dP)
    dA, dW = oracle.matmul_bwd(dZ, A, W)
    dA = oracle.leakyrelu_bwd(S, dA, 0.01)
    db = oracle.add_broadcast_bwd_bias(dZ)
    for name, ref in dict(Z=Z, P=P, dP=dP, dZ=dZ, dA=dA, dW=dW, db=db).items():
        assert rel_err(got[name], ref) <= tol, name
    assert abs(float(got["loss"][0, 0]) - float(loss)) <= tol * abs(float(loss))


def test_shapes_beyond_one_workgroup_run_as_the_three_launches(gpu):
    """More than 64 classes, or operands beyond the compute unit's LDS: same entry point, same values."""
    lib = _lib.load()
    for dtype, (B, H, C) in ((np.float64, (32, 64, 100)), (np.float32, (128, 1024, 10)), (np.float64, (64, 512, 10))):
        ops = operands(dtype, B, H, C, 3)
        one = run(lib, True, dtype, *ops, _lib.ACT_LEAKYRELU, 0)
        three = run(lib, False, dtype, *ops, _lib.ACT_LEAKYRELU, 0)
        for k in one:
            assert np.array_equal(one[k], three[k]), k


def test_argument_checks(gpu):
    lib = _lib.load()
    f = np.float64
    A, W, b, S, T, dW0 = operands(f, 8, 16, 4, 1)
    bufs = dict(A=dev(A), W=dev(W), b=dev(b), T=dev(T), Z=DeviceBuffer.alloc(f, 8, 4), P=DeviceBuffer.alloc(f, 8, 4),
                loss=DeviceBuffer.alloc(f, 1, 1), dP=DeviceBuffer.alloc(f, 8, 4), dZ=DeviceBuffer.alloc(f, 8, 4),
                dA=DeviceBuffer.alloc(f, 8, 16), dW=DeviceBuffer.alloc(f, 16, 4), db=DeviceBuffer.alloc(f, 1, 4))

    def call(**over):
        h = {k: v.handle for k, v in bufs.items()}
        h.update(over)
        return lib.prad_dense_softmax_cce(h["A"], h["W"], h["b"], h["T"], h["Z"], h["P"], h["loss"], h["dP"], h["dZ"], h["dA"], h["dW"],
                                          h["db"], 0, over.get("act", _lib.ACT_NONE), over.get("src"), 0.01)

    check(call())
    with pytest.raises((ArgumentException, InvalidOperationException)):
        check(call(act=_lib.ACT_LEAKYRELU))                                  # an activation without its cached operand
    with pytest.raises((ArgumentException, InvalidOperationException)):
        check(call(T=DeviceBuffer.alloc(f, 8, 5).handle))                    # target of another shape
    with pytest.raises((ArgumentException, InvalidOperationException)):
        check(call(dW=DeviceBuffer.alloc(np.float32, 16, 4).handle))         # mixed element types
    with pytest.raises((ArgumentException, InvalidOperationException)):
        check(call(act=99))
