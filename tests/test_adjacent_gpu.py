"""Operations next to the matrix products in the reference's example graphs (MatrixAdd, MatrixAddThree,
MatrixTranspose, LayerNormalization, AmplifiedSigmoid) against the oracle, through the operation classes."""
import numpy as np
import pytest

from conftest import assert_parity
from parallelreverseautodiff_amd import _lib, seeded
from parallelreverseautodiff_amd.exceptions import ArgumentException, check
from parallelreverseautodiff_amd.matrix import DeviceBuffer, Matrix
from parallelreverseautodiff_amd.operations import (AmplifiedSigmoidOperation, LayerNormalizationOperation, MatrixAddOperation,
                                                    MatrixAddThreeOperation, MatrixTransposeOperation)

pytestmark = pytest.mark.gpu
DTYPES = [np.float64, np.float32]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 1), (7, 13), (64, 1000), (300, 257)])
def test_add_and_add_three_are_exact(gpu, oracle, dtype, shape):
    a, b, c = (seeded.normal(101, i, shape, 2.0, dtype) for i in range(3))
    op = MatrixAddOperation.Instantiate(None)
    y = op.Forward(Matrix.from_numpy(a), Matrix.from_numpy(b))
    assert np.array_equal(y.to_numpy(), oracle.matrix_add(a, b))
    g = Matrix.from_numpy(c)
    res = op.Backward(g)
    assert res.HasMultipleInputs and len(res.Results) == 2 and all(np.array_equal(r.to_numpy(), c) for r in res.Results)
    op3 = MatrixAddThreeOperation.Instantiate(None)
    y3 = op3.Forward(Matrix.from_numpy(a), Matrix.from_numpy(b), Matrix.from_numpy(c))
    assert np.array_equal(y3.to_numpy(), oracle.matrix_add_three(a, b, c))
    assert len(op3.Backward(g).Results) == 3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 1), (1, 100), (100, 1), (64, 64), (65, 127), (300, 1000), (128, 200), (1000, 36), (4, 4)])
def test_transpose(gpu, oracle, dtype, shape):
    x = seeded.normal(102, 1, shape, 1.0, dtype)
    op = MatrixTransposeOperation.Instantiate(None)
    y = op.Forward(Matrix.from_numpy(x))
    assert (y.Rows, y.Cols) == (shape[1], shape[0])
    assert np.array_equal(y.to_numpy(), oracle.matrix_transpose(x))
    back = op.Backward(y).Item1
    assert np.array_equal(back.to_numpy(), x)
    lib = _lib.load()
    bx = DeviceBuffer.alloc(dtype, 3, 5)
    with pytest.raises(ArgumentException):
        check(lib.prad_transpose(bx.handle, bx.handle))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(3, 4), (1, 1), (64, 1000), (33, 1024), (5, 1025), (9, 3000)])
def test_layer_normalization(gpu, oracle, dtype, shape):
    x = seeded.normal(103, 1, shape, 2.0, dtype) + dtype(0.5)
    if shape[0] > 2:
        x[1, :] = 5.0                                   # zero deviation: output 0 / 1e-9 = 0
    dy = seeded.normal(103, 2, shape, 1.0, dtype)
    op = LayerNormalizationOperation.Instantiate(None)
    y = op.Forward(Matrix.from_numpy(x))
    ry, rmean, rstd = oracle.layernorm_fwd(x)
    assert_parity(y.to_numpy(), ry, dtype, "layer norm forward")
    assert_parity(op.mean.download().reshape(-1), rmean, dtype, "row means")
    assert_parity(op.stdDev.download().reshape(-1), rstd, dtype, "row deviations")
    if shape[0] > 2:
        assert np.array_equal(y.to_numpy()[1], np.zeros(shape[1], dtype))
    dx = op.Backward(Matrix.from_numpy(dy)).Item1
    keep = np.ones(shape[0], bool)
    if shape[0] > 2:
        keep[1] = False                                 # 1 / (0 + 1e-9)^3 overflows float: inf in both, compared apart
    rdx = oracle.layernorm_bwd(x, rmean, rstd, dy)
    assert_parity(dx.to_numpy()[keep], rdx[keep], dtype, "layer norm backward")
    if shape[0] > 2:
        got, want = dx.to_numpy()[1], rdx[1]
        assert np.array_equal(np.isfinite(got), np.isfinite(want))
        fin = np.isfinite(want)
        assert np.allclose(got[fin], want[fin], rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_amplified_sigmoid(gpu, oracle, dtype):
    x = seeded.normal(104, 1, (37, 91), 4.0, dtype)
    x[0, :4] = [0.0, 1.0, -1.0, 30.0]
    dy = seeded.normal(104, 2, (37, 91), 1.0, dtype)
    op = AmplifiedSigmoidOperation.Instantiate(None)
    y = op.Forward(Matrix.from_numpy(x))
    assert_parity(y.to_numpy(), oracle.amplified_sigmoid_fwd(x), dtype, "amplified sigmoid")
    assert y.to_numpy()[0, 0] == dtype(0.5)
    dx = op.Backward(Matrix.from_numpy(dy)).Item1
    assert_parity(dx.to_numpy(), oracle.amplified_sigmoid_bwd(x, dy), dtype, "amplified sigmoid backward")
    assert dx.to_numpy()[0, 0] == dtype(0.25) * dy[0, 0]    # as written: no ln(b) factor


@pytest.mark.parametrize("dtype", DTYPES)
def test_amplified_sigmoid_in_fused_product(gpu, oracle, dtype):
    """The activation is also available as an epilogue of the product (forward) and of the dA product (backward)."""
    lib = _lib.load()
    A = seeded.normal(105, 1, (40, 64), 1.0, dtype)
    B = seeded.normal(105, 2, (64, 48), 0.3, dtype)
    bias = seeded.normal(105, 3, (1, 48), 1.0, dtype)
    up = lambda a: (lambda b: (b.upload(a), b)[1])(DeviceBuffer.alloc(dtype, *a.shape))
    bA, bB, bb = up(A), up(B), up(bias)
    Z, H = DeviceBuffer.alloc(dtype, 40, 48), DeviceBuffer.alloc(dtype, 40, 48)
    check(lib.prad_matmul_fwd_fused(bA.handle, bB.handle, bb.handle, Z.handle, H.handle, _lib.ACT_AMPLIFIED_SIGMOID, 0.0))
    rZ = oracle.add_broadcast_fwd(oracle.matmul_fwd(A, B), bias)
    assert_parity(Z.download(), rZ, dtype, "pre-activation")
    assert_parity(H.download(), oracle.amplified_sigmoid_fwd(rZ), dtype, "fused amplified sigmoid")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(37, 49), (5000, 49), (4100, 32), (4097, 64), (6000, 7), (2049, 1), (9, 200)])
def test_scaled_softmax_forward_and_backward(gpu, oracle, dtype, shape):
    """y = softmax(alpha x), dx = alpha J^T dy against the oracle's scale-then-softmax; few rows (a wavefront
    per row), thousands of short rows (a lane per row, staged through LDS: even, odd and single-column pitches,
    a last workgroup that is not full), rows wider than a wavefront; and bit for bit against the separate launches."""
    lib = _lib.load()
    rows, cols = shape
    alpha = 1.0 / np.sqrt(32.0)
    x = seeded.normal(31, 1, shape, 3.0, dtype)
    dy = seeded.normal(31, 2, shape, 1.0, dtype)
    X, Y, DY, DX = (DeviceBuffer.alloc(dtype, rows, cols) for _ in range(4))
    X.upload(x); DY.upload(dy)
    check(lib.prad_softmax_scaled_fwd(X.handle, alpha, Y.handle))
    check(lib.prad_softmax_scaled_bwd(Y.handle, DY.handle, alpha, DX.handle))
    y, dx = Y.download(), DX.download()
    xs = x * dtype(alpha)                                  # MatrixMultiplyScalarOperation.Forward
    ry = oracle.softmax_fwd(xs)
    assert_parity(y, ry, dtype, "softmax(alpha x)")
    assert np.all(np.abs(y.astype(np.float64).sum(axis=1) - 1.0) <= cols * np.finfo(dtype).eps * 4)
    rdx = oracle.softmax_bwd(y, dy) * dtype(alpha)         # softmax backward, then the scalar's backward
    assert_parity(dx, rdx, dtype, "alpha J^T dy")
    # the separate launches
    S, Y2, DX2 = (DeviceBuffer.alloc(dtype, rows, cols) for _ in range(3))
    check(lib.prad_scale(X.handle, S.handle, alpha))
    check(lib.prad_softmax_fwd(S.handle, Y2.handle))
    assert np.array_equal(Y2.download(), y)
    check(lib.prad_softmax_bwd(Y.handle, DY.handle, DX2.handle))
    check(lib.prad_scale(DX2.handle, DX2.handle, alpha))
    assert np.array_equal(DX2.download(), dx)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 1), (7, 13), (128, 512), (3000, 97), (2500, 1000)])
def test_mean_squared_error_loss_and_gradient(gpu, oracle, dtype, shape):
    """MeanSquaredErrorLossOperation Forward and Backward against the oracle, separately and in one pass
    (prad_mse: the same values as the two launches, bit for bit)."""
    lib = _lib.load()
    y = seeded.normal(51, 1, shape, 1.0, dtype)
    t = seeded.normal(51, 2, shape, 1.0, dtype)
    Y, T, D1, D2 = (DeviceBuffer.alloc(dtype, *shape) for _ in range(4))
    L1, L2 = DeviceBuffer.alloc(dtype, 1, 1), DeviceBuffer.alloc(dtype, 1, 1)
    Y.upload(y); T.upload(t)
    check(lib.prad_mse_fwd(Y.handle, T.handle, L1.handle))
    check(lib.prad_mse_bwd(Y.handle, T.handle, D1.handle))
    check(lib.prad_mse(Y.handle, T.handle, L2.handle, D2.handle))
    loss = float(L1.download()[0, 0])
    ref = oracle.mse_fwd(y, t)
    assert abs(loss - ref) <= (1e-12 if dtype == np.float64 else 1e-5) * abs(ref)
    assert_parity(D1.download(), oracle.mse_bwd(y, t), dtype, "mse backward")
    assert np.array_equal(L2.download(), L1.download()) and np.array_equal(D2.download(), D1.download())
    if shape != (1, 1):
        assert lib.prad_mse(Y.handle, T.handle, D1.handle, D2.handle) == _lib.PRAD_ERR_ARG     # loss must be 1 x 1
