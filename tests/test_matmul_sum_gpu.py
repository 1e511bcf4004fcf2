"""Parity of MatrixMultiplyAndSum forward/backward with the oracle (reference semantics as written)."""
import numpy as np
import pytest

from conftest import TOL, assert_parity
from parallelreverseautodiff_amd import seeded
from parallelreverseautodiff_amd.exceptions import InvalidOperationException
from parallelreverseautodiff_amd.matrix import DeepMatrix, Matrix
from parallelreverseautodiff_amd.operations import (BatchGpuMatrixMultiplyAndSumOperation, BatchMatrixMultiplyAndSumOperation,
                                                   GpuMatrixMultiplyAndSumOperation, MatrixMultiplyAndSumOperation)

pytestmark = pytest.mark.gpu
DTYPES = [np.float64, np.float32]


def check_forward(out, A, B, ref, dtype):
    """out[q] is a sum of M*N products of mixed sign; the error that matters is relative to the magnitude
    of what is summed (sum_ij |(A.B[q])_ij|), for the oracle's sequential sums as much as for the GPU's."""
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    exact = np.array([[np.sum(A64 @ B64[q]) for q in range(B.shape[0])]])
    scale = np.array([[np.sum(np.abs(A64 @ B64[q])) for q in range(B.shape[0])]])
    tol = TOL[np.dtype(dtype)]
    assert np.all(np.abs(out - exact) <= tol * scale)
    assert np.all(np.abs(out - ref) <= 2 * tol * scale)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(6, 9, 3), (64, 96, 5), (130, 70, 4), (128, 256, 8), (100, 36, 9), (68, 200, 13),
                                   (64, 96, 31), (32, 48, 47), (16, 32, 63), (64, 64, 32), (8, 16, 1)])
def test_forward_backward(gpu, oracle, dtype, shape):
    M, K, P = shape
    A = seeded.normal(81, 1, (M, K), 1.0, dtype)
    B = seeded.normal(81, 2, (P, K, M), 1.0, dtype)
    dOut = seeded.normal(81, 3, (1, P), 1.0, dtype)
    op = GpuMatrixMultiplyAndSumOperation.Instantiate(None)
    out = op.Forward(Matrix.from_numpy(A), DeepMatrix.from_numpy(B))
    assert (out.Rows, out.Cols) == (1, P)
    check_forward(out.to_numpy(), A, B, oracle.matmul_sum_fwd(A, B, threads=8), dtype)
    res = op.Backward(Matrix.from_numpy(dOut))
    assert res.HasMultipleInputs and len(res.Results) == 1 + P
    rdA, rdB = oracle.matmul_sum_bwd(A, B, dOut)
    assert np.array_equal(res.Item1.to_numpy(), rdA)  # same products, same q-ascending sums: bit exact
    for q in range(P):
        assert np.array_equal(res.Results[1 + q].to_numpy(), rdB[q])


def test_benchmark_configuration_shape_fp32(gpu, oracle):
    """A 512x768, 32 slices of 768x512 (N(0, 0.02)), upstream gradient N(0, 1)."""
    M, K, P = 512, 768, 32
    A = seeded.normal(82, 1, (M, K), 0.02, np.float32)
    B = seeded.normal(82, 2, (P, K, M), 0.02, np.float32)
    dOut = seeded.normal(82, 3, (1, P), 1.0, np.float32)
    op = GpuMatrixMultiplyAndSumOperation.Instantiate(None)
    out = op.Forward(Matrix.from_numpy(A), DeepMatrix.from_numpy(B)).to_numpy()
    check_forward(out, A, B, oracle.matmul_sum_fwd(A, B, threads=16), np.float32)
    res = op.Backward(Matrix.from_numpy(dOut))
    rdA, rdB = oracle.matmul_sum_bwd(A, B, dOut)
    assert np.array_equal(res.Item1.to_numpy(), rdA)
    for q in (0, 13, 31):
        assert np.array_equal(res.Results[1 + q].to_numpy(), rdB[q])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cls", [BatchGpuMatrixMultiplyAndSumOperation, BatchMatrixMultiplyAndSumOperation])
@pytest.mark.parametrize("shape", [(3, 6, 9, 4), (8, 64, 96, 5), (5, 130, 70, 3), (2, 100, 36, 1), (1, 32, 48, 7)])
def test_per_sample_wrappers(gpu, oracle, dtype, cls, shape):
    """BatchMatrixMultiplyAndSumOperation / BatchGpuMatrixMultiplyAndSumOperation
    (src/RMAD/BatchGpuMatrixMultiplyAndSumOperation.cs:51-74): sample i is MatrixMultiplyAndSum(input1[i], input2); the
    results per sample are those of the single operation (backward bit for bit)."""
    S, M, K, P = shape
    A = seeded.normal(83, 1, (S, M, K), 1.0, dtype)
    B = seeded.normal(83, 2, (P, K, M), 1.0, dtype)
    dOut = seeded.normal(83, 3, (S, 1, P), 1.0, dtype)
    op = cls.Instantiate(None)
    out = op.Forward(DeepMatrix.from_numpy(A), DeepMatrix.from_numpy(B))
    assert op.GetDeepOutput() is out and out.Depth == S and (out.Rows, out.Cols) == (1, P)
    for i in range(S):
        check_forward(out[i].to_numpy(), A[i], B, oracle.matmul_sum_fwd(A[i], B), dtype)
    results = op.Backward(DeepMatrix.from_numpy(dOut))
    assert len(results) == S
    for i, res in enumerate(results):
        assert res.HasMultipleInputs and len(res.Results) == 1 + P
        rdA, rdB = oracle.matmul_sum_bwd(A[i], B, dOut[i])
        assert np.array_equal(res.Item1.to_numpy(), rdA), "dA of sample %d" % i
        for q in range(P):
            assert np.array_equal(res.Results[1 + q].to_numpy(), rdB[q]), "dB[%d] of sample %d" % (q, i)
    # the single operation on one sample gives the bits of that sample in the batch
    single = GpuMatrixMultiplyAndSumOperation.Instantiate(None)
    assert np.array_equal(single.Forward(Matrix.from_numpy(A[S - 1]), DeepMatrix.from_numpy(B)).to_numpy(), out[S - 1].to_numpy())
    # Store / Restore keep the per-sample inputs (IOperationBase.Store, src/RMAD/IOperationBase.cs:188-194)
    op.Store("a")
    op.Forward(DeepMatrix.from_numpy(A[::-1].copy()), DeepMatrix.from_numpy(B))
    op.Restore("a")
    again = op.Backward(DeepMatrix.from_numpy(dOut))
    assert np.array_equal(again[0].Item1.to_numpy(), results[0].Item1.to_numpy())


def test_per_sample_wrapper_errors(gpu):
    op = BatchGpuMatrixMultiplyAndSumOperation.Instantiate(None)
    with pytest.raises(InvalidOperationException, match="compatible for multiplication"):
        op.Forward(DeepMatrix(3, 4, 5), DeepMatrix(2, 6, 4))
    from parallelreverseautodiff_amd.exceptions import ArgumentException
    with pytest.raises(ArgumentException):
        op.Forward(Matrix(4, 5), DeepMatrix(2, 5, 4))
    op.Forward(DeepMatrix(3, 4, 5), DeepMatrix(2, 5, 4))
    with pytest.raises(ArgumentException):
        op.Backward(DeepMatrix(2, 1, 2))          # one upstream matrix per sample


def test_ones_closed_form_and_cpu_name(gpu):
    op = MatrixMultiplyAndSumOperation.Instantiate(None)
    out = op.Forward(Matrix.from_numpy(np.ones((4, 5))), DeepMatrix.from_numpy(np.ones((2, 5, 4)))).to_numpy()
    assert np.array_equal(out, np.full((1, 2), 80.0))


def test_shape_errors(gpu):
    op = GpuMatrixMultiplyAndSumOperation.Instantiate(None)
    with pytest.raises(InvalidOperationException, match="compatible for multiplication"):
        op.Forward(Matrix(4, 5), DeepMatrix(2, 6, 4))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4, 64, 96, 64), (3, 33, 50, 17), (32, 128, 192, 128), (1, 40, 24, 56)])
def test_batch_of_products_summed_with_bias(gpu, oracle, dtype, shape):
    """C = sum_q A[q].B[q] + bias against the oracle's composition: MatrixMultiplyOperation.Forward per slice,
    the products added in slice order, MatrixAddBroadcasting; and its backward against matmul_bwd per slice.
    (The reference has no single operation of this form, so the composition is the bar.)"""
    from conftest import dot_bound
    from parallelreverseautodiff_amd.operations import BatchMatrixMultiplySumOperation
    P, M, K, N = shape
    A = seeded.normal(83, 1, (P, M, K), 1.0, dtype)
    B = seeded.normal(83, 2, (P, K, N), 1.0, dtype)
    bias = seeded.normal(83, 3, (1, N), 1.0, dtype)
    dC = seeded.normal(83, 4, (M, N), 1.0, dtype)
    ref = np.zeros((M, N), dtype)
    for q in range(P):
        ref = ref + oracle.matmul_fwd(A[q], B[q], threads=4)
    ref = oracle.add_broadcast_fwd(ref, bias)
    op = BatchMatrixMultiplySumOperation.Instantiate(None)
    C = op.Forward(DeepMatrix.from_numpy(A), DeepMatrix.from_numpy(B), Matrix.from_numpy(bias))
    bound = sum(dot_bound(A[q], B[q], dtype) for q in range(P)) + P * np.finfo(dtype).eps * np.abs(ref)
    assert_parity(C.to_numpy(), ref, dtype, "sum of products + bias", bound=bound)
    res = op.Backward(Matrix.from_numpy(dC))
    dA, dB, db = res.Results
    for q in range(P):
        rA, rB = oracle.matmul_bwd(dC, A[q], B[q], threads=4)
        assert_parity(dA.to_numpy()[q], rA, dtype, "dA[%d]" % q)
        assert_parity(dB.to_numpy()[q], rB, dtype, "dB[%d]" % q)
    assert_parity(db.to_numpy(), oracle.add_broadcast_bwd_bias(dC), dtype, "bias gradient")
    with pytest.raises(InvalidOperationException):
        BatchMatrixMultiplySumOperation().Forward(DeepMatrix.from_numpy(A), DeepMatrix.from_numpy(A))
