"""Host-side logic that needs no GPU: jagged Matrix / DeepMatrix containers, result builder,
status-code to exception mapping, seeded generator."""
import numpy as np
import pytest

from parallelreverseautodiff_amd import _lib, exceptions, seeded
from parallelreverseautodiff_amd.matrix import DeepMatrix, Matrix
from parallelreverseautodiff_amd.operations import BackwardResultBuilder, GpuMatrixMultiplyOperation
from parallelreverseautodiff_amd.cudablas import CudaBlas


def test_matrix_is_jagged_and_zeroed():
    m = Matrix(3, 4)
    assert (m.Rows, m.Cols, m.Length, len(m)) == (3, 4, 3, 3)
    rows = m.ToArray()
    assert len(rows) == 3 and all(r.shape == (4,) and not r.any() for r in rows)
    assert rows[0].base is None and rows[0] is not rows[1]  # one allocation per row
    m[1][2] = 5.0
    assert m[1, 2] == 5.0 and m.to_numpy()[1, 2] == 5.0
    m[2] = np.arange(4.0)  # row replacement, as GradientClearer does
    assert m.to_numpy()[2].tolist() == [0, 1, 2, 3]


def test_matrix_ids_are_unique_and_adopted_rows_are_live():
    r = [np.array([1.0, 2.0]), np.array([3.0, 4.0])]
    a, b = Matrix(r), Matrix(2, 2)
    assert a.UniqueId != b.UniqueId
    r[0][1] = 9.0
    assert a[0, 1] == 9.0
    f = Matrix.from_numpy(np.ones((2, 3), np.float32))
    assert f.dtype == np.float32


def test_matrix_rows_are_contiguous_and_of_the_matrix_type():
    """What the device copies read from a row is cols contiguous elements of the matrix's type: a strided view or a
    row of another type is copied on adoption (also through Replace and row assignment) instead of being read past."""
    base = np.arange(12.0).reshape(3, 4)
    m = Matrix([base[:, 0], base[:, 1]])                     # column views: stride of 32 bytes
    assert all(r.flags["C_CONTIGUOUS"] and r.dtype == np.float64 for r in m.ToArray())
    assert np.array_equal(m.to_numpy(), base[:, :2].T)
    m.Replace([np.arange(3, dtype=np.float32), base[0, ::2][:3] if False else np.array([7, 8, 9])])
    assert all(r.dtype == np.float64 and r.flags["C_CONTIGUOUS"] for r in m.ToArray()) and m.Cols == 3
    m[1] = base[:, 3]
    assert m.ToArray()[1].flags["C_CONTIGUOUS"] and np.array_equal(m.ToArray()[1], [3.0, 7.0, 11.0])
    live = np.zeros(3)
    m[0] = live                                              # a conforming array is adopted, not copied
    live[2] = 5.0
    assert m[0, 2] == 5.0


def test_matrix_rejects_bad_arguments():
    with pytest.raises(exceptions.ArgumentException):
        Matrix(0, 3)
    with pytest.raises(exceptions.ArgumentException):
        Matrix(2, 2, dtype=np.int32)


def test_deep_matrix():
    d = DeepMatrix(3, 2, 5, np.float32)
    assert (d.Depth, d.Rows, d.Cols) == (3, 2, 5)
    d[1][0][4] = 2.0
    assert d.to_numpy()[1, 0, 4] == 2.0
    e = DeepMatrix.from_numpy(np.arange(24.0).reshape(2, 3, 4))
    assert e[1][2][3] == 23.0


def test_backward_result_builder_order_and_flag():
    a, b, bias = Matrix(1, 1), Matrix(1, 1), Matrix(1, 1)
    r = BackwardResultBuilder().AddInputGradient(a).AddInputGradient(b).Build()
    assert r.Results == [a, b] and r.HasMultipleInputs and r.Item1 is a and r.Item2 is b
    r1 = BackwardResultBuilder().AddInputGradient(a).AddBiasGradient(bias).Build()
    assert r1.Results == [a, bias] and not r1.HasMultipleInputs
    deep = DeepMatrix(2, 1, 1)
    r2 = BackwardResultBuilder().AddInputGradient(a).AddInputGradientArray(deep).Build()
    assert r2.Results == [a, deep[0], deep[1]] and r2.HasMultipleInputs


def test_status_codes_map_to_reference_exceptions(monkeypatch):
    assert exceptions._BY_CODE[_lib.PRAD_ERR_SHAPE] is exceptions.InvalidOperationException
    assert exceptions._BY_CODE[_lib.PRAD_ERR_ARG] is exceptions.ArgumentException
    assert exceptions._BY_CODE[_lib.PRAD_ERR_NOT_RECTANGULAR] is exceptions.InvalidOperationException
    exceptions.check(_lib.PRAD_OK)
    with pytest.raises(exceptions.CudaNotInitializedException):
        exceptions.check(_lib.PRAD_ERR_NOT_INITIALIZED)


def test_gpu_operation_before_initialize_raises():
    if CudaBlas.Instance.IsInitialized:
        pytest.skip("library already initialised in this process")
    op = GpuMatrixMultiplyOperation.Instantiate(None)
    with pytest.raises(exceptions.CudaNotInitializedException):
        op.Forward(Matrix(2, 2), Matrix(2, 2))


def test_seeded_generator_properties():
    a = seeded.uniform(1, 7, (1000,), -1, 1)
    assert -1 <= a.min() and a.max() < 1 and abs(a.mean()) < 0.1
    assert np.array_equal(a, seeded.uniform(1, 7, (1000,), -1, 1))
    assert not np.array_equal(a, seeded.uniform(1, 8, (1000,), -1, 1))
    n = seeded.normal(1, 9, (20000,), 2.0)
    assert abs(n.mean()) < 0.05 and abs(n.std() - 2.0) < 0.05
    x = seeded.xavier(1, 3, 784, 256)
    assert np.abs(x).max() <= np.sqrt(6.0 / (784 + 256))
    t = seeded.one_hot_labels(1, 4, 64, 10)
    assert t.shape == (64, 10) and np.array_equal(t.sum(axis=1), np.ones(64))
    assert seeded.uniform(1, 1, (8,), dtype=np.float32).dtype == np.float32
