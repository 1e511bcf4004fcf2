"""Tall float products with a small right operand (tens of thousands of rows, K a multiple of 96, K x N floats within
one compute unit's LDS) run on the streaming kernel with the resident right operand; every one of its variants against
the products evaluated in double and the same epilogue arithmetic, and against the tiled kernels' results."""
import ctypes
import os

import numpy as np
import pytest

from conftest import rel_err
from parallelreverseautodiff_amd import _lib, seeded
from parallelreverseautodiff_amd.exceptions import check
from parallelreverseautodiff_amd.matrix import DeviceBuffer

pytestmark = pytest.mark.gpu
F32 = np.float32
TOL = 1e-5


def gelu(x):
    s = np.sqrt(2 / np.pi)
    return 0.5 * (1 + np.tanh(s * (x + 0.044715 * x ** 3))) * x


def gelu_derivative_of_the_reference(x):   # src/RMAD/GELUOperation.cs:94-101, as written there
    s = np.sqrt(2 / np.pi)
    b = np.tanh(s * (x + 0.044715 * x ** 3))
    c = (1 - b * b) ** 2
    d = s * (0.044715 * 3 * x * x + 1)
    return 0.5 * x * (c * d + b) + 0.5 * (1 + b)


def dev(a):
    b = DeviceBuffer.alloc(F32, a.shape[0], a.shape[1])
    b.upload(a)
    return b


# (rows, K, N): widths of four, three and two tiles per unit, one and several 96-column chunks, ragged row counts
SHAPES = [(8192, 96, 96), (8200, 96, 288), (12345, 96, 384), (8192, 384, 96), (9001, 288, 96), (8192, 96, 32), (8208, 192, 160)]


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_forward_with_every_epilogue(gpu, M, K, N):
    lib = _lib.load()
    A = seeded.normal(11, 1, (M, K), 1.0, F32); W = seeded.normal(11, 2, (K, N), 0.08, F32); b = seeded.normal(11, 3, (1, N), 0.2, F32)
    dA, dW, db = dev(A), dev(W), dev(b)
    Z, H, C = DeviceBuffer.alloc(F32, M, N), DeviceBuffer.alloc(F32, M, N), DeviceBuffer.alloc(F32, M, N)
    ref = A.astype(np.float64) @ W.astype(np.float64)
    check(lib.prad_matmul_fwd(dA.handle, dW.handle, C.handle))
    assert rel_err(C.download(), ref) <= TOL
    check(lib.prad_matmul_fwd_fused(dA.handle, dW.handle, db.handle, None, H.handle, _lib.ACT_NONE, 0.0))
    assert rel_err(H.download(), ref + b) <= TOL
    check(lib.prad_matmul_fwd_fused(dA.handle, dW.handle, db.handle, Z.handle, H.handle, _lib.ACT_GELU, 0.0))
    z = Z.download()
    assert rel_err(z, ref + b) <= TOL
    assert rel_err(H.download(), gelu(z.astype(np.float64))) <= TOL      # the activation of the stored pre-activation
    check(lib.prad_matmul_fwd_fused(dA.handle, dW.handle, None, None, H.handle, _lib.ACT_LEAKYRELU, 0.01))
    c = C.download()
    assert np.array_equal(H.download(), np.where(c > 0, c, F32(0.01) * c))   # same product bits, exact activation
    # accumulate: C += A . W
    C0 = seeded.normal(11, 4, (M, N), 1.0, F32)
    C.upload(C0)
    check(lib.prad_gemm(0, 0, dA.handle, dW.handle, C.handle, 1))
    assert rel_err(C.download(), C0.astype(np.float64) + ref) <= TOL


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_input_gradient_with_and_without_activation_backward(gpu, M, K, N):
    """dX = dY . W^T (the weight read in its stored orientation) and dX (.) act'(source)."""
    lib = _lib.load()
    dY = seeded.normal(12, 1, (M, K), 1.0, F32); W = seeded.normal(12, 2, (N, K), 0.08, F32); S = seeded.normal(12, 3, (M, N), 1.0, F32)
    X = seeded.normal(12, 4, (M, N), 1.0, F32)
    ddY, dW, dS, dXin, dX = dev(dY), dev(W), dev(S), dev(X), DeviceBuffer.alloc(F32, M, N)
    ref = dY.astype(np.float64) @ W.astype(np.float64).T
    check(lib.prad_matmul_bwd(ddY.handle, dXin.handle, dW.handle, dX.handle, None, 0, 0))
    assert rel_err(dX.download(), ref) <= TOL
    check(lib.prad_matmul_bwd_fused(ddY.handle, dXin.handle, dW.handle, dX.handle, None, 0, _lib.ACT_GELU, dS.handle, 0.0))
    assert rel_err(dX.download(), ref * gelu_derivative_of_the_reference(S.astype(np.float64))) <= TOL
    plain = DeviceBuffer.alloc(F32, M, N)
    check(lib.prad_matmul_bwd(ddY.handle, dXin.handle, dW.handle, plain.handle, None, 0, 0))
    check(lib.prad_matmul_bwd_fused(ddY.handle, dXin.handle, dW.handle, dX.handle, None, 0, _lib.ACT_LEAKYRELU, dS.handle, 0.01))
    assert np.array_equal(dX.download(), plain.download() * np.where(S > 0, F32(1), F32(0.01)))


def test_matches_the_oracle_on_exact_inputs(gpu, oracle):
    """Small integers are exact in float in any summation order: the streaming kernel, the tiled kernels and the
    reference's k-ascending loop must agree bit for bit."""
    lib = _lib.load()
    M, K, N = 8192, 96, 96
    rng = np.random.default_rng(5)
    A = rng.integers(-4, 5, (M, K)).astype(F32); W = rng.integers(-4, 5, (K, N)).astype(F32)
    dA, dW, C = dev(A), dev(W), DeviceBuffer.alloc(F32, M, N)
    check(lib.prad_matmul_fwd(dA.handle, dW.handle, C.handle))
    got = C.download()
    assert np.array_equal(got[:256], oracle.matmul_fwd(np.ascontiguousarray(A[:256]), W, threads=4))
    assert np.array_equal(got, (A.astype(np.float64) @ W.astype(np.float64)).astype(F32))
    head, small = dev(A[:4096]), DeviceBuffer.alloc(F32, 4096, N)  # fewer rows: the tiled kernels
    check(lib.prad_matmul_fwd(head.handle, dW.handle, small.handle))
    assert np.array_equal(small.download(), got[:4096])
