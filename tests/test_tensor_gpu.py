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
        Tensor([2, 3, 4]).MatrixMultiply(b)
    with pytest.raises(InvalidOperationException):
        TensorReverse([a]).MatrixMultiplyReverse(a)
    with pytest.raises(ArgumentException):
        Tensor([2, 2], np.zeros(3))


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
