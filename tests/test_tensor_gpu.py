"""The tape engine's products (Tensor.MatrixMultiply, TensorReverse.MatrixMultiplyReverse) on flat row-major arrays.
The reference hands these arrays to MKL, whose summation order its tests do not pin; the bar here is the same
as for MatrixMultiplyOperation: the oracle's k-ascending product within tolerance."""
import ctypes

import numpy as np
import pytest

from conftest import assert_parity, dot_bound
from parallelreverseautodiff_amd import _lib, seeded
from parallelreverseautodiff_amd.exceptions import ArgumentException, InvalidOperationException, check
from parallelreverseautodiff_amd.tensor import Tensor, TensorReverse

pytestmark = pytest.mark.gpu
DTYPES = [np.float64, np.float32]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 1, 1), (5, 7, 3), (64, 96, 50), (130, 257, 65)])
def test_tensor_product_and_reverse(gpu, oracle, dtype, shape):
    m, k, n = shape
    A = seeded.uniform(111, 1, (m, k), -1.0, 1.0, dtype)
    B = seeded.uniform(111, 2, (k, n), -1.0, 1.0, dtype)
    dC = seeded.normal(111, 3, (m, n), 1.0, dtype)
    ta, tb = Tensor([m, k], A.reshape(-1)), Tensor([k, n], B.reshape(-1))
    tc = ta.MatrixMultiply(tb)
    assert tc.Shape == [m, n]
    rC = oracle.matmul_fwd(A, B)
    assert_parity(tc.to_numpy(), rC, dtype, "tensor product", bound=dot_bound(A, B, dtype))
    half = ta.MatrixMultiply(tb, alpha=0.5)
    assert np.array_equal(half.to_numpy(), tc.to_numpy() * dtype(0.5))
    gA, gB = TensorReverse([ta, tb]).MatrixMultiplyReverse(Tensor([m, n], dC.reshape(-1)))
    rA, rB = oracle.matmul_bwd(dC, A, B)
    assert_parity(gA.to_numpy(), rA, dtype, "dA", bound=dot_bound(dC, B.T, dtype))
    assert_parity(gB.to_numpy(), rB, dtype, "dB", bound=dot_bound(A.T, dC, dtype))
    flat = tc.Data                       # the flat array, as the reference exposes it
    assert flat.shape == (m * n,) and np.array_equal(flat.reshape(m, n), tc.to_numpy())
    flat[0] = 42.0                       # callers write into Data; the next product must see it
    again = Tensor([1, m], np.eye(1, m, dtype=dtype).reshape(-1)).MatrixMultiply(tc)
    assert again.to_numpy()[0, 0] == dtype(42.0)


def test_tensor_errors(gpu):
    a, b = Tensor([2, 3]), Tensor([4, 2])
    with pytest.raises(ArgumentException, match="Incompatible shapes"):
        a.MatrixMultiply(b)
    with pytest.raises(ArgumentException, match="only supported for 2D"):
        Tensor([4]).MatrixMultiply(b)
    # the reference's own methods take two-dimensional tensors only (src/PRAD/Tensor.cs:574-577, TensorReverse.cs:96-110)
    with pytest.raises(ArgumentException, match="only supported for 2D"):
        Tensor([2, 3, 4]).MatrixMultiply(Tensor([2, 4, 2]))
    with pytest.raises(ArgumentException, match="only supported for 2D"):
        TensorReverse([Tensor([2, 3, 4]), Tensor([2, 4, 2])]).MatrixMultiplyReverse(Tensor([2, 3, 2]))
    with pytest.raises(ArgumentException, match="Incompatible shapes"):
        Tensor([2, 3, 4]).BatchMatrixMultiply(Tensor([3, 4, 2]))      # leading dimensions differ
    with pytest.raises(ArgumentException, match="Incompatible shapes"):
        Tensor([2, 3, 4]).BatchMatrixMultiply(Tensor([2, 5, 2]))      # inner dimensions differ
    with pytest.raises(InvalidOperationException):
        TensorReverse([a]).MatrixMultiplyReverse(a)
    with pytest.raises(ArgumentException):
        Tensor([2, 2], np.zeros(3))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ["scores", "context", "small"])
def test_batched_tensor_product_and_reverse(gpu, oracle, dtype, case):
    """Products of tensors of more than two dimensions, which the windowed-attention example of the reference needs
    (examples/swin/SwinExample/SwinTransformerTools.cs:372-389) and its Tensor.MatrixMultiply rejects
    (src/PRAD/Tensor.cs:574-577), under names of their own: one product per leading index, checked slice by slice against the oracle's
    MatrixMultiplyOperation.  "scores" and "context" are the shapes of that example at 1024 windows x 3 heads:
    [1024, 3, 49, 32] . [1024, 3, 32, 49] and [1024, 3, 49, 49] . [1024, 3, 49, 32]."""
    lead, m, k, n = {"scores": ([1024, 3], 49, 32, 49), "context": ([1024, 3], 49, 49, 32), "small": ([2, 1, 3], 5, 7, 4)}[case]
    L = int(np.prod(lead))
    A = seeded.uniform(113, 1, (L, m, k), -1.0, 1.0, dtype)
    B = seeded.uniform(113, 2, (L, k, n), -1.0, 1.0, dtype)
    dC = seeded.normal(113, 3, (L, m, n), 1.0, dtype)
    ta, tb, tg = Tensor(lead + [m, k], A.reshape(-1)), Tensor(lead + [k, n], B.reshape(-1)), Tensor(lead + [m, n], dC.reshape(-1))
    tc = ta.BatchMatrixMultiply(tb)
    assert tc.Shape == lead + [m, n]
    gA, gB = TensorReverse([ta, tb]).BatchMatrixMultiplyReverse(tg)
    assert gA.Shape == lead + [m, k] and gB.Shape == lead + [k, n]
    C, dA, dB = tc.to_numpy().reshape(L, m, n), gA.to_numpy().reshape(L, m, k), gB.to_numpy().reshape(L, k, n)
    for s in range(L):
        assert_parity(C[s], oracle.matmul_fwd(A[s], B[s]), dtype, "slice %d" % s, bound=dot_bound(A[s], B[s], dtype))
        rA, rB = oracle.matmul_bwd(dC[s], A[s], B[s])
        assert_parity(dA[s], rA, dtype, "dA of slice %d" % s, bound=dot_bound(dC[s], B[s].T, dtype))
        assert_parity(dB[s], rB, dtype, "dB of slice %d" % s, bound=dot_bound(A[s].T, dC[s], dtype))
    half = ta.BatchMatrixMultiply(tb, alpha=0.5)
    assert np.array_equal(half.to_numpy(), tc.to_numpy() * dtype(0.5))


@pytest.mark.parametrize("dtype", DTYPES)
def test_tensor_product_with_a_shared_right_operand(gpu, oracle, dtype):
    """[windows, tokens, C] . [C, 3C] (the QKV projection of the same example, SwinTransformerTools.cs:348-349): the left
    operand is one (windows * tokens) x C matrix as it lies in memory; the gradient of the shared operand adds up over
    all windows."""
    lead, m, k, n = [6, 2], 49, 96, 288
    L = int(np.prod(lead))
    A = seeded.uniform(114, 1, (L * m, k), -1.0, 1.0, dtype)
    B = seeded.uniform(114, 2, (k, n), -1.0, 1.0, dtype)
    dC = seeded.normal(114, 3, (L * m, n), 1.0, dtype)
    ta, tb, tg = Tensor(lead + [m, k], A.reshape(-1)), Tensor([k, n], B.reshape(-1)), Tensor(lead + [m, n], dC.reshape(-1))
    tc = ta.BatchMatrixMultiply(tb)
    assert tc.Shape == lead + [m, n]
    assert_parity(tc.to_numpy().reshape(L * m, n), oracle.matmul_fwd(A, B), dtype, "shared product", bound=dot_bound(A, B, dtype))
    gA, gB = TensorReverse([ta, tb]).BatchMatrixMultiplyReverse(tg)
    assert gA.Shape == lead + [m, k] and gB.Shape == [k, n]
    rA, rB = oracle.matmul_bwd(dC, A, B)
    assert_parity(gA.to_numpy().reshape(L * m, k), rA, dtype, "dA", bound=dot_bound(dC, B.T, dtype))
    assert_parity(gB.to_numpy(), rB, dtype, "dB summed over the windows", bound=dot_bound(A.T, dC, dtype))
    # a right operand with leading dimensions of one is the same product; results feed the next product from the device
    tb1 = Tensor([1, 1, k, n], B.reshape(-1))
    assert np.array_equal(ta.BatchMatrixMultiply(tb1).to_numpy(), tc.to_numpy())
    chained = tc.BatchMatrixMultiply(Tensor([n, 8], np.ones(n * 8, dtype)))
    assert chained.Shape == lead + [m, 8]
    assert_parity(chained.to_numpy().reshape(L * m, 8), oracle.matmul_fwd(tc.to_numpy().reshape(L * m, n), np.ones((n, 8), dtype)), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_host_entry_points_on_flat_arrays(gpu, oracle, dtype):
    lib = _lib.load()
    code = _lib.PRAD_F64 if dtype == np.float64 else _lib.PRAD_F32
    m, k, n = 33, 70, 19
    A = seeded.uniform(112, 1, (m, k), -1.0, 1.0, dtype)
    B = seeded.uniform(112, 2, (k, n), -1.0, 1.0, dtype)
    dC = seeded.normal(112, 3, (m, n), 1.0, dtype)
    C, dA, dB = np.empty((m, n), dtype), np.empty((m, k), dtype), np.empty((k, n), dtype)
    p = lambda a: ctypes.c_void_p(a.ctypes.data)
    check(lib.prad_tensor_matmul_host(code, p(A), p(B), p(C), m, k, k, n, 2.0))
    assert_parity(C, oracle.matmul_fwd(A, B) * dtype(2.0), dtype, "flat host product")
    check(lib.prad_tensor_matmul_reverse_host(code, p(dC), p(A), p(B), p(dA), p(dB), m, k, n))
    rA, rB = oracle.matmul_bwd(dC, A, B)
    assert_parity(dA, rA, dtype, "flat host dA")
    assert_parity(dB, rB, dtype, "flat host dB")
    assert lib.prad_tensor_matmul_host(code, p(A), p(B), p(C), m, k, k + 1, n, 1.0) == _lib.PRAD_ERR_SHAPE


def test_the_layer_of_the_references_own_tape_test(gpu):
    """The operands of the one tape-engine test that multiplies matrices (test/ParallelReverseAutoDiff.Test/PRAD/
    PradOpTests.cs:4151-4171: a 1 x 4 input, 4 x 3 weights; the test asserts no values).  The products are small enough
    to be written down: 0.7, 0.8, 0.9 forward; with an upstream gradient of ones the input gradient is the row sums of
    the weights and the weight gradient repeats the input along its rows."""
    x = Tensor([1, 4], np.array([0.1, 0.2, 0.3, 0.4]))
    w = Tensor([4, 3], np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 0.7, 0.8, 0.9, 1.0, 1.1, 1.2]))
    y = x.MatrixMultiply(w)
    np.testing.assert_allclose(y.to_numpy(), [[0.7, 0.8, 0.9]], rtol=1e-15, atol=0)
    gx, gw = TensorReverse([x, w]).MatrixMultiplyReverse(Tensor([1, 3], np.ones(3)))
    np.testing.assert_allclose(gx.to_numpy(), [[0.6, 1.5, 2.4, 3.3]], rtol=1e-15, atol=0)
    assert np.array_equal(gw.to_numpy(), np.repeat(np.array([[0.1], [0.2], [0.3], [0.4]]), 3, axis=1))
