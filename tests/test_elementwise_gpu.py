"""Parity of the bandwidth kernels (activations, Hadamard, accumulate, bias broadcast) with the oracle."""
import numpy as np
import pytest

from conftest import assert_parity
from parallelreverseautodiff_amd import seeded
from parallelreverseautodiff_amd.exceptions import ArgumentException
from parallelreverseautodiff_amd.matrix import Matrix
from parallelreverseautodiff_amd.operations import (GELUOperation, HadamardProductOperation, LeakyReLUOperation,
                                                   MatrixAddBroadcastingOperation, SigmoidOperation, TanhOperation)

pytestmark = pytest.mark.gpu
DTYPES = [np.float64, np.float32]
SHAPES = [(1, 1), (1, 3), (7, 5), (64, 256), (129, 1031), (300, 1000)]


def data(dtype, shape, sigma=1.5):
    x = seeded.normal(41, 1, shape, sigma, dtype)
    x.reshape(-1)[0] = 0.0  # LeakyReLU'(0) must take alpha
    return x, seeded.normal(41, 2, shape, 1.0, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", SHAPES)
def test_leakyrelu(gpu, oracle, dtype, shape):
    x, dy = data(dtype, shape)
    op = LeakyReLUOperation(0.01)
    y = op.Forward(Matrix.from_numpy(x)).to_numpy()
    dx = op.Backward(Matrix.from_numpy(dy)).Item1.to_numpy()
    assert np.array_equal(y, oracle.leakyrelu_fwd(x, 0.01))  # one multiply: bit exact
    assert np.array_equal(dx, oracle.leakyrelu_bwd(x, dy, 0.01))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("name", ["sigmoid", "tanh", "gelu"])
def test_transcendental_activations(gpu, oracle, dtype, shape, name):
    x, dy = data(dtype, shape)
    cls, fwd, bwd = {"sigmoid": (SigmoidOperation, oracle.sigmoid_fwd, oracle.sigmoid_bwd),
                     "tanh": (TanhOperation, oracle.tanh_fwd, oracle.tanh_bwd),
                     "gelu": (GELUOperation, oracle.gelu_fwd, oracle.gelu_bwd)}[name]
    op = cls.Instantiate(None)
    y = op.Forward(Matrix.from_numpy(x)).to_numpy()
    assert_parity(y, fwd(x), dtype, name + " forward")
    dx = op.Backward(Matrix.from_numpy(dy)).Item1.to_numpy()
    src = x if name == "gelu" else y  # Sigmoid/Tanh differentiate through their own cached output
    assert_parity(dx, bwd(src, dy), dtype, name + " backward")


@pytest.mark.parametrize("dtype", DTYPES)
def test_gelu_reference_formula_known_values(gpu, dtype):
    op = GELUOperation.Instantiate(None)
    op.Forward(Matrix.from_numpy(np.array([[0.0, 10.0]], dtype)))
    g = op.Backward(Matrix.from_numpy(np.ones((1, 2), dtype))).Item1.to_numpy()
    assert g[0, 0] == dtype(0.5) and g[0, 1] == dtype(6.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", SHAPES)
def test_hadamard(gpu, oracle, dtype, shape):
    a, b = data(dtype, shape)
    dy = seeded.normal(41, 3, shape, 1.0, dtype)
    op = HadamardProductOperation.Instantiate(None)
    y = op.Forward(Matrix.from_numpy(a), Matrix.from_numpy(b)).to_numpy()
    res = op.Backward(Matrix.from_numpy(dy))
    rda, rdb = oracle.hadamard_bwd(a, b, dy)
    assert np.array_equal(y, oracle.hadamard_fwd(a, b))
    assert np.array_equal(res.Item1.to_numpy(), rda) and np.array_equal(res.Item2.to_numpy(), rdb)
    with pytest.raises(ArgumentException):
        op.Forward(Matrix(2, 3, dtype), Matrix(3, 2, dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_broadcast_and_bias_gradient(gpu, oracle, dtype):
    x, dy = data(dtype, (64, 257))
    b = seeded.normal(41, 4, (1, 257), 1.0, dtype)
    op = MatrixAddBroadcastingOperation.Instantiate(None)
    y = op.Forward(Matrix.from_numpy(x), Matrix.from_numpy(b)).to_numpy()
    assert np.array_equal(y, oracle.add_broadcast_fwd(x, b))
    g = Matrix.from_numpy(dy)
    res = op.Backward(g)
    assert res.Item1 is g and not res.HasMultipleInputs  # dOutput is passed through, not copied
    # the column sum is taken by four wavefronts and combined, not row by row: same value within rounding
    assert_parity(res.Item2.to_numpy(), oracle.add_broadcast_bwd_bias(dy), dtype, "bias gradient")


def test_large_vector_tail_and_size(gpu, oracle):
    """A size that is not a multiple of the vector width or the workgroup span."""
    n = 4 * 1024 * 1024 + 3
    x = seeded.normal(42, 1, (1, n), 1.0, np.float32)
    dy = seeded.normal(42, 2, (1, n), 1.0, np.float32)
    op = SigmoidOperation.Instantiate(None)
    y = op.Forward(Matrix.from_numpy(x)).to_numpy()
    dx = op.Backward(Matrix.from_numpy(dy)).Item1.to_numpy()
    assert_parity(y, oracle.sigmoid_fwd(x), np.float32)
    assert_parity(dx, oracle.sigmoid_bwd(y, dy), np.float32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_bias_gradient_of_a_tall_matrix(gpu, oracle, dtype):
    """Enough rows for the chunked column sum (a whole sequence of gate gradients)."""
    dy = seeded.normal(43, 1, (5000, 130), 1.0, dtype)
    res = MatrixAddBroadcastingOperation.Instantiate(None).Backward(Matrix.from_numpy(dy))
    assert_parity(res.Item2.to_numpy(), oracle.add_broadcast_bwd_bias(dy), dtype, "bias gradient")
