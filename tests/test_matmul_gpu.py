"""Parity of the HIP matrix-multiply path with the CPU oracle, through the operation classes and
the C ABI.  Bar: bit-exact where the arithmetic is exact (small integers), otherwise
max |x - ref| / max(|ref|, rms(ref)) <= 1e-12 (double) / 1e-5 (float) and every entry of a product
within the order-independent rounding bound 8*sqrt(K)*eps*(|A|.|B|)_ij; the reduction order of the
MFMA kernels differs from the reference's k-ascending loop, which is what the tolerance is for."""
import ctypes
import json
import math
import os
import threading

import numpy as np
import pytest

from conftest import assert_parity, dot_bound, rel_err
from parallelreverseautodiff_amd import _lib, seeded
from parallelreverseautodiff_amd.exceptions import ArgumentException, InvalidOperationException
from parallelreverseautodiff_amd.matrix import DeepMatrix, DeviceBuffer, Matrix
from parallelreverseautodiff_amd.operations import (BatchGpuMatrixMultiplyOperation, CudaMatrixMultiplyOperation,
                                                   GpuMatrixMultiplyOperation, MatrixMultiplyOperation, accumulate_gradient)

pytestmark = pytest.mark.gpu
DTYPES = [np.float64, np.float32]
HERE = os.path.dirname(os.path.abspath(__file__))

SHAPES = [  # M, K, N: tile-aligned, ragged in every dimension, degenerate vectors, MLP layers
    (128, 128, 128), (256, 64, 384), (1, 1, 1), (1, 7, 1), (5, 3, 2), (127, 129, 130), (129, 17, 3), (257, 33, 65),
    (64, 784, 256), (64, 256, 128), (64, 128, 10), (100, 100, 1), (1, 100, 100), (384, 512, 256), (130, 260, 390),
    # whole tiles with a ragged reduction: one slab plus a tail, a tail only, an odd number of slabs
    (128, 70, 64), (64, 40, 32), (256, 200, 256), (512, 1000, 512), (2048, 24, 2048),
    # rows that start 16-byte aligned but tiles that hang over the edge (vector loads clamped at the edge), on the
    # 64 and 128 tiles, with a tiny M and with a narrow N
    (1000, 64, 1000), (2052, 36, 2060), (4, 8, 260), (3000, 100, 12),
]


def inputs(dtype, M, K, N, seed=seeded.DEFAULT_SEED):
    return (seeded.uniform(seed, 1, (M, K), -1, 1, dtype), seeded.uniform(seed, 2, (K, N), -1, 1, dtype),
            seeded.normal(seed, 3, (M, N), 1.0, dtype))


def check_against_oracle(oracle, dtype, got, A, B, dC, threads=8, what=""):
    """Compares (C, dA, dB) with the oracle: relative error bar plus the per-entry rounding bound."""
    C, dA, dB = got
    rC = oracle.matmul_fwd(A, B, threads=threads)
    rdA, rdB = oracle.matmul_bwd(dC, A, B, threads=threads)
    assert_parity(C, rC, dtype, "C " + what, bound=dot_bound(A, B, dtype))
    assert_parity(dA, rdA, dtype, "dA " + what, bound=dot_bound(dC, B.T, dtype))
    assert_parity(dB, rdB, dtype, "dB " + what, bound=dot_bound(A.T, dC, dtype))


def run_op(cls, A, B, dC):
    op = cls.Instantiate(None)
    mA, mB = Matrix.from_numpy(A), Matrix.from_numpy(B)
    C = op.Forward(mA, mB)
    assert op.GetOutput() is C and (C.Rows, C.Cols) == (A.shape[0], B.shape[1])
    res = op.Backward(Matrix.from_numpy(dC))
    assert res.HasMultipleInputs and len(res.Results) == 2
    return C.to_numpy(), res.Item1.to_numpy(), res.Item2.to_numpy()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", SHAPES)
def test_forward_backward_matches_oracle(gpu, oracle, dtype, shape):
    M, K, N = shape
    A, B, dC = inputs(dtype, M, K, N)
    check_against_oracle(oracle, dtype, run_op(GpuMatrixMultiplyOperation, A, B, dC), A, B, dC, what=str(shape))


@pytest.mark.parametrize("cls", [MatrixMultiplyOperation, GpuMatrixMultiplyOperation, CudaMatrixMultiplyOperation])
def test_all_operation_names_share_the_path(gpu, oracle, cls):
    A, B, dC = inputs(np.float64, 70, 90, 50)
    C, dA, dB = run_op(cls, A, B, dC)
    assert_parity(C, oracle.matmul_fwd(A, B), np.float64)
    rdA, rdB = oracle.matmul_bwd(dC, A, B)
    assert_parity(dA, rdA, np.float64)
    assert_parity(dB, rdB, np.float64)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [512, 1024])
def test_square_sizes_of_the_benchmark(gpu, oracle, dtype, n):
    A, B, dC = inputs(dtype, n, n, n)
    check_against_oracle(oracle, dtype, run_op(GpuMatrixMultiplyOperation, A, B, dC), A, B, dC, threads=16, what=str(n))


@pytest.mark.parametrize("dtype", DTYPES)
def test_exact_integer_products_are_bit_exact(gpu, oracle, dtype):
    rng = np.random.default_rng(3)
    A = rng.integers(-8, 9, (200, 150)).astype(dtype)
    B = rng.integers(-8, 9, (150, 140)).astype(dtype)
    dC = rng.integers(-8, 9, (200, 140)).astype(dtype)
    C, dA, dB = run_op(GpuMatrixMultiplyOperation, A, B, dC)
    rdA, rdB = oracle.matmul_bwd(dC, A, B)
    assert np.array_equal(C, oracle.matmul_fwd(A, B))
    assert np.array_equal(dA, rdA) and np.array_equal(dB, rdB)


@pytest.mark.parametrize("dtype", DTYPES)
def test_identity_and_ones(gpu, dtype):
    B = seeded.uniform(9, 1, (200, 130), -1, 1, dtype)
    C, _, _ = run_op(GpuMatrixMultiplyOperation, np.eye(200, dtype=dtype), B, np.zeros((200, 130), dtype))
    assert np.array_equal(C, B)
    C, _, _ = run_op(GpuMatrixMultiplyOperation, np.ones((131, 777), dtype), np.ones((777, 5), dtype), np.zeros((131, 5), dtype))
    assert np.array_equal(C, np.full((131, 5), 777, dtype))


def test_reference_gpu_vs_cpu_contract(gpu, oracle):
    """test/ParallelReverseAutoDiff.Test/GpuMatrixMultiplyOperationTest.cs:24-53: A 1000x1000 Xavier, B and the
    upstream gradient 1000x1 Xavier; GPU and CPU results equal after rounding to 10 decimals."""
    A = seeded.xavier(31, 1, 1000, 1000)
    B = seeded.xavier(31, 2, 1000, 1)
    dC = seeded.xavier(31, 3, 1000, 1)
    C, dA, dB = run_op(GpuMatrixMultiplyOperation, A, B, dC)
    rC = oracle.matmul_fwd(A, B, threads=8)
    rdA, rdB = oracle.matmul_bwd(dC, A, B, threads=8)
    for got, ref in ((C, rC), (dA, rdA), (dB, rdB)):
        assert np.max(np.abs(got - ref)) < 5e-11
        assert_parity(got, ref, np.float64)


def test_golden_small_cases(gpu):
    golden = json.load(open(os.path.join(HERE, "golden", "golden.json")))
    for name in ("tiny_f64", "tiny_f32"):
        case = golden["matmul"][name]
        dtype = np.dtype(case["dtype"])
        A, B, dC = inputs(dtype, case["M"], case["K"], case["N"])
        C, dA, dB = run_op(GpuMatrixMultiplyOperation, A, B, dC)
        for got, key in ((C, "C"), (dA, "dA"), (dB, "dB")):
            want = np.array([float.fromhex(h) for h in case[key]["hex"]], dtype).reshape(case[key]["shape"])
            assert_parity(got, want, dtype, "%s %s" % (name, key))  # K = 6: no room for reordering error


@pytest.mark.parametrize("n", [2048, 4096])
def test_full_size_properties_fp64(gpu, n):
    """At sizes the oracle cannot finish in seconds: sampled entries against exactly rounded dot products,
    and the adjoint identity <dA, A> = <dB, B> = <dC, C>."""
    A, B, dC = inputs(np.float64, n, n, n)
    C, dA, dB = run_op(GpuMatrixMultiplyOperation, A, B, dC)
    rng = np.random.default_rng(n)
    scale_c = math.sqrt(n / 3.0)
    for _ in range(48):
        i, j = int(rng.integers(n)), int(rng.integers(n))
        assert abs(C[i, j] - math.fsum(A[i, :] * B[:, j])) <= 1e-12 * scale_c
        assert abs(dA[i, j] - math.fsum(dC[i, :] * B[j, :])) <= 1e-12 * math.sqrt(n)
        assert abs(dB[i, j] - math.fsum(A[:, i] * dC[:, j])) <= 1e-12 * math.sqrt(n)
    lhs = float(np.sum(dC * C))
    assert abs(float(np.sum(dA * A)) - lhs) <= 1e-11 * abs(lhs)
    assert abs(float(np.sum(dB * B)) - lhs) <= 1e-11 * abs(lhs)


@pytest.mark.parametrize("n", [2048, 4096])
def test_full_size_properties_fp32(gpu, n):
    A, B, dC = inputs(np.float32, n, n, n)
    C, dA, dB = run_op(GpuMatrixMultiplyOperation, A, B, dC)
    rng = np.random.default_rng(5)
    A64, B64, G64 = A.astype(np.float64), B.astype(np.float64), dC.astype(np.float64)
    for _ in range(48):
        i, j = int(rng.integers(n)), int(rng.integers(n))
        assert abs(C[i, j] - math.fsum(A64[i, :] * B64[:, j])) <= 1e-5 * math.sqrt(n / 3.0)
        assert abs(dA[i, j] - math.fsum(G64[i, :] * B64[j, :])) <= 1e-5 * math.sqrt(n)
        assert abs(dB[i, j] - math.fsum(A64[:, i] * G64[:, j])) <= 1e-5 * math.sqrt(n)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [2048, 4096])
def test_full_size_whole_matrix_identities(gpu, dtype, n):
    """Every tile of every output is touched for O(N^2) host work: a product applied to the all-ones vector
    equals the chain of matrix-vector products, C.1 = A.(B.1) and 1^T.C = (1^T.A).B, and likewise for
    dA = dC.B^T and dB = A^T.dC.  The right-hand sides are evaluated in double.  The worst-case rounding bound of
    the sums an entry stands for is 8 sqrt(K) eps (|X|.|Y|.1)_i; rounding errors of different entries cancel, and the
    sums measured on the device stay below 1e-4 of it, so the bar is 1e-3 of that bound: one wrong entry of typical
    magnitude in a row (let alone a misplaced, dropped or doubled tile) exceeds it."""
    A, B, dC = inputs(dtype, n, n, n)
    C, dA, dB = run_op(GpuMatrixMultiplyOperation, A, B, dC)
    f = lambda x: x.astype(np.float64)
    A64, B64, G64 = f(A), f(B), f(dC)
    one = np.ones(n)
    eps = float(np.finfo(dtype).eps)
    factor = 8.0 * math.sqrt(n) * eps
    worst = 0.0

    def check_pair(out, X, Y, what):
        # out = X . Y (already oriented): rows against X.(Y.1), columns against (1^T.X).Y
        nonlocal worst
        out64 = f(out)
        for got, ref, bound in ((out64 @ one, X @ (Y @ one), np.abs(X) @ (np.abs(Y) @ one)),
                                (one @ out64, (one @ X) @ Y, (one @ np.abs(X)) @ np.abs(Y))):
            excess = np.abs(got - ref) / (factor * bound)
            worst = max(worst, float(excess.max()))
            assert excess.max() <= 1e-3, "%s: a row or column sum is off by %.2e x its rounding bound" % (what, excess.max())

    check_pair(C, A64, B64, "C")
    check_pair(dA, G64, B64.T, "dA")
    check_pair(dB, A64.T, G64, "dB")
    print("whole-matrix identities %s n=%d: worst sum at %.2e of its bound" % (np.dtype(dtype).name, n, worst))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("trans", [(0, 0), (0, 1), (1, 0)])
def test_shared_tiles_of_a_poorly_filled_last_round(gpu, oracle, dtype, trans):
    """An output of 20 x 26 = 520 tiles of 128 x 128 over 512 workgroup slots: 8 tiles are split along K (several
    workgroups per tile, reduced by the last to arrive) inside the same launch as the 512 unsplit ones.  Every entry is
    held to its order-independent rounding bound against the product in double, rows sampled from every tile row
    (split tiles and tiles that hang over the ragged edge included) to the parity bar against the oracle, and a second
    launch into the same buffer adds onto the first (accumulate)."""
    lib = _lib.load()
    from parallelreverseautodiff_amd.exceptions import check
    tA, tB = trans
    M, K, N = 2500, 1056, 3300
    X = seeded.uniform(17, 1, (K, M) if tA else (M, K), -1, 1, dtype)      # op(X) is M x K
    Y = seeded.uniform(17, 2, (N, K) if tB else (K, N), -1, 1, dtype)      # op(Y) is K x N
    bx, by, bc = DeviceBuffer.alloc(dtype, *X.shape), DeviceBuffer.alloc(dtype, *Y.shape), DeviceBuffer.alloc(dtype, M, N)
    bx.upload(X); by.upload(Y)
    check(lib.prad_gemm(tA, tB, bx.handle, by.handle, bc.handle, 0))
    C = bc.download()
    opX = np.ascontiguousarray(X.T) if tA else X
    opY = np.ascontiguousarray(Y.T) if tB else Y
    exact = opX.astype(np.float64) @ opY.astype(np.float64)
    assert float(np.max(np.abs(C - exact) - dot_bound(opX, opY, dtype))) <= 0.0
    rows = np.unique(np.concatenate([np.arange(3, M, 128), np.arange(M - 40, M, 7)]))
    assert_parity(C[rows], oracle.matmul_fwd(np.ascontiguousarray(opX[rows]), opY, threads=16), dtype, "sampled rows")
    check(lib.prad_gemm(tA, tB, bx.handle, by.handle, bc.handle, 1))
    assert np.array_equal(bc.download(), C + C)
    check(lib.prad_gemm(tA, tB, bx.handle, by.handle, bc.handle, 0))       # same bits on every run
    assert np.array_equal(bc.download(), C)


@pytest.mark.parametrize("dtype", DTYPES)
def test_accumulating_backward(gpu, oracle, dtype):
    """dW += A^T.dC written by the product's own epilogue equals OperationBase.AccumulateGradient after Backward."""
    lib = _lib.load()
    A, B, dC = inputs(dtype, 96, 200, 72)
    dest0 = seeded.normal(4, 9, (200, 72), 1.0, dtype)
    mA, mB, mG, dest = (Matrix.from_numpy(x) for x in (A, B, dC, dest0))
    from parallelreverseautodiff_amd.exceptions import check
    check(lib.prad_matmul_bwd(mG.device().handle, mA.device().handle, mB.device().handle, None, dest.device().handle, 0, 1))
    dest._device_written()
    _, rdB = oracle.matmul_bwd(dC, A, B)
    assert_parity(dest.to_numpy(), oracle.accumulate(dest0, rdB), dtype)
    # the separate accumulate kernel gives the same
    d2 = Matrix.from_numpy(dest0)
    accumulate_gradient(d2, Matrix.from_numpy(rdB))
    assert np.array_equal(d2.to_numpy(), oracle.accumulate(dest0, rdB))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", ["leakyrelu", "sigmoid", "tanh", "gelu"])
def test_fused_epilogues(gpu, oracle, dtype, act):
    lib = _lib.load()
    from parallelreverseautodiff_amd.exceptions import check
    code = {"leakyrelu": _lib.ACT_LEAKYRELU, "sigmoid": _lib.ACT_SIGMOID, "tanh": _lib.ACT_TANH, "gelu": _lib.ACT_GELU}[act]
    alpha = 0.01
    M, K, N = 70, 150, 130
    A, B, _ = inputs(dtype, M, K, N)
    bias = seeded.normal(6, 4, (1, N), 0.5, dtype)
    mA, mB, mb = Matrix.from_numpy(A), Matrix.from_numpy(B), Matrix.from_numpy(bias)
    Z, H = DeviceBuffer.alloc(dtype, M, N), DeviceBuffer.alloc(dtype, M, N)
    check(lib.prad_matmul_fwd_fused(mA.device().handle, mB.device().handle, mb.device().handle, Z.handle, H.handle, code, alpha))
    rZ = oracle.add_broadcast_fwd(oracle.matmul_fwd(A, B), bias)
    fwd = {"leakyrelu": lambda z: oracle.leakyrelu_fwd(z, alpha), "sigmoid": oracle.sigmoid_fwd, "tanh": oracle.tanh_fwd,
           "gelu": oracle.gelu_fwd}[act]
    gZ = Z.download()
    assert_parity(gZ, rZ, dtype, "Z")
    # the activation is checked on the GPU's own pre-activation, so that only the activation is compared
    assert_parity(H.download(), fwd(gZ), dtype, "H")
    # backward: dA = (dC . B^T) (.) act'(src), src shaped like A
    dC = seeded.normal(6, 5, (M, N), 1.0, dtype)
    src = seeded.normal(6, 6, (M, K), 1.0, dtype)
    if act in ("sigmoid", "tanh"):
        src = fwd(src)  # these cache their output
    mG, mS = Matrix.from_numpy(dC), Matrix.from_numpy(src)
    dA, dB = DeviceBuffer.alloc(dtype, M, K), DeviceBuffer.alloc(dtype, K, N)
    check(lib.prad_matmul_bwd_fused(mG.device().handle, mA.device().handle, mB.device().handle, dA.handle, dB.handle, 0, code,
                                    mS.device().handle, alpha))
    rdA, rdB = oracle.matmul_bwd(dC, A, B)
    bwd = {"leakyrelu": lambda s, g: oracle.leakyrelu_bwd(s, g, alpha), "sigmoid": oracle.sigmoid_bwd, "tanh": oracle.tanh_bwd,
           "gelu": oracle.gelu_bwd}[act]
    assert_parity(dA.download(), bwd(src, rdA), dtype, "fused dA")
    assert_parity(dB.download(), rdB, dtype, "dB", bound=dot_bound(A.T, dC, dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_batched_products(gpu, oracle, dtype):
    depth, M, K, N = 5, 40, 70, 30
    A = seeded.uniform(8, 1, (depth, M, K), -1, 1, dtype)
    B = seeded.uniform(8, 2, (depth, K, N), -1, 1, dtype)
    dC = seeded.normal(8, 3, (depth, M, N), 1.0, dtype)
    op = BatchGpuMatrixMultiplyOperation.Instantiate(None)
    out = op.Forward(DeepMatrix.from_numpy(A), DeepMatrix.from_numpy(B))
    res = op.Backward(DeepMatrix.from_numpy(dC))
    assert out.Depth == depth and len(res) == depth
    for i in range(depth):
        assert_parity(out[i].to_numpy(), oracle.matmul_fwd(A[i], B[i]), dtype, bound=dot_bound(A[i], B[i], dtype))
        rdA, rdB = oracle.matmul_bwd(dC[i], A[i], B[i])
        assert_parity(res[i].Item1.to_numpy(), rdA, dtype, bound=dot_bound(dC[i], B[i].T, dtype))
        assert_parity(res[i].Item2.to_numpy(), rdB, dtype, bound=dot_bound(A[i].T, dC[i], dtype))
    # (DeepMatrix, Matrix) overload: the single matrix is shared by every sample
    op2 = BatchGpuMatrixMultiplyOperation.Instantiate(None)
    out2 = op2.Forward(DeepMatrix.from_numpy(A), Matrix.from_numpy(B[0]))
    for i in range(depth):
        assert_parity(out2[i].to_numpy(), oracle.matmul_fwd(A[i], B[0]), dtype, bound=dot_bound(A[i], B[0], dtype))
    op3 = BatchGpuMatrixMultiplyOperation.Instantiate(None)
    out3 = op3.Forward(Matrix.from_numpy(A[1]), DeepMatrix.from_numpy(B))
    for i in range(depth):
        assert_parity(out3[i].to_numpy(), oracle.matmul_fwd(A[1], B[i]), dtype, bound=dot_bound(A[1], B[i], dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_one_shot_host_entry_points(gpu, oracle, dtype):
    """Jagged rows in, jagged rows out, one call per operation (today's GpuMatrixMultiplyOperation behaviour)."""
    lib = _lib.load()
    from parallelreverseautodiff_amd.exceptions import check
    M, K, N = 37, 53, 29
    A, B, dC = inputs(dtype, M, K, N)
    code = _lib.PRAD_F64 if dtype == np.float64 else _lib.PRAD_F32

    def jag(a):
        rows = [np.array(a[i]) for i in range(a.shape[0])]
        return rows, (ctypes.c_void_p * len(rows))(*[r.ctypes.data for r in rows])

    ra, pa = jag(A); rb, pb = jag(B); rg, pg = jag(dC)
    rc, pc = jag(np.zeros((M, N), dtype)); rda, pda = jag(np.zeros((M, K), dtype)); rdb, pdb = jag(np.zeros((K, N), dtype))
    check(lib.prad_matmul_fwd_host(code, pa, pb, pc, M, K, K, N))
    check(lib.prad_matmul_bwd_host(code, pg, pa, pb, pda, pdb, M, K, N))
    assert_parity(np.stack(rc), oracle.matmul_fwd(A, B), dtype, bound=dot_bound(A, B, dtype))
    rdA, rdB = oracle.matmul_bwd(dC, A, B)
    assert_parity(np.stack(rda), rdA, dtype, bound=dot_bound(dC, B.T, dtype))
    assert_parity(np.stack(rdb), rdB, dtype, bound=dot_bound(A.T, dC, dtype))
    assert lib.prad_matmul_fwd_host(code, pa, pb, pc, M, K, K + 1, N) == _lib.PRAD_ERR_SHAPE


def test_error_behaviour(gpu):
    op = GpuMatrixMultiplyOperation.Instantiate(None)
    with pytest.raises(InvalidOperationException, match="Input 1 columns do not match Input 2 rows"):
        op.Forward(Matrix(3, 4), Matrix(5, 2))
    lib = _lib.load()
    a, b, c = DeviceBuffer.alloc(np.float64, 3, 4), DeviceBuffer.alloc(np.float64, 5, 2), DeviceBuffer.alloc(np.float64, 3, 2)
    assert lib.prad_matmul_fwd(a.handle, b.handle, c.handle) == _lib.PRAD_ERR_SHAPE
    assert b"Input 1 columns do not match Input 2 rows" in lib.prad_last_error()
    b2, cbad = DeviceBuffer.alloc(np.float64, 4, 2), DeviceBuffer.alloc(np.float64, 2, 2)
    assert lib.prad_matmul_fwd(a.handle, b2.handle, cbad.handle) == _lib.PRAD_ERR_ARG
    f = DeviceBuffer.alloc(np.float32, 4, 2)
    assert lib.prad_matmul_fwd(a.handle, f.handle, c.handle) == _lib.PRAD_ERR_DTYPE
    assert lib.prad_matmul_fwd(a.handle, None, c.handle) == _lib.PRAD_ERR_BAD_HANDLE
    assert lib.prad_gemm(1, 1, a.handle, b2.handle, c.handle, 0) == _lib.PRAD_ERR_ARG
    # jagged upload with a short row
    m = Matrix([np.zeros(4), np.zeros(3)])
    with pytest.raises(InvalidOperationException, match="not rectangular"):
        m.device()
    rows = [np.zeros(4), np.zeros(4)]
    ptrs = (ctypes.c_void_p * 2)(*[r.ctypes.data for r in rows])
    lens = (ctypes.c_int64 * 2)(4, 3)
    d = DeviceBuffer.alloc(np.float64, 2, 4)
    assert lib.prad_buf_upload_rows(d.handle, ptrs, lens) == _lib.PRAD_ERR_NOT_RECTANGULAR
    h = ctypes.c_void_p()
    assert lib.prad_buf_alloc(7, 2, 2, ctypes.byref(h)) == _lib.PRAD_ERR_DTYPE
    assert lib.prad_buf_alloc(_lib.PRAD_F64, 0, 2, ctypes.byref(h)) == _lib.PRAD_ERR_ARG


def test_residency_protocol(gpu, oracle):
    """Weights are marshalled once; a host-side in-place edit is seen by the next operation; outputs are
    downloaded only when the host reads them."""
    A, B, _ = inputs(np.float64, 20, 30, 10)
    mA, mB = Matrix.from_numpy(A), Matrix.from_numpy(B)
    op = GpuMatrixMultiplyOperation.Instantiate(None)
    C1 = op.Forward(mA, mB)
    assert mB._dev_valid and not C1._host_valid
    assert_parity(C1.to_numpy(), oracle.matmul_fwd(A, B), np.float64)
    assert not C1._host_valid  # to_numpy does not materialise rows
    mB[0][0] += 1.0  # host mutation through the live row, as Adam does in the reference
    assert not mB._dev_valid
    B2 = B.copy(); B2[0, 0] += 1.0
    C2 = op.Forward(mA, mB)
    assert_parity(C2.to_numpy(), oracle.matmul_fwd(A, B2), np.float64)
    row = C2[3]  # jagged host access downloads
    assert C2._host_valid and np.array_equal(row, C2.to_numpy()[3])


def test_store_restore_intermediates(gpu, oracle):
    op = GpuMatrixMultiplyOperation.Instantiate(None)
    A1, B1, dC = inputs(np.float64, 12, 9, 7, seed=1)
    A2, B2, _ = inputs(np.float64, 12, 9, 7, seed=2)
    op.Forward(Matrix.from_numpy(A1), Matrix.from_numpy(B1)); op.Store("s1")
    op.Forward(Matrix.from_numpy(A2), Matrix.from_numpy(B2)); op.Store("s2")
    op.Restore("s1")
    rdA, rdB = oracle.matmul_bwd(dC, A1, B1)
    res = op.Backward(Matrix.from_numpy(dC))
    assert_parity(res.Item1.to_numpy(), rdA, np.float64)
    assert_parity(res.Item2.to_numpy(), rdB, np.float64)


def test_concurrent_backward_from_pool_threads(gpu, oracle):
    """The reference's visitor runs Backward of different operations on pool threads at the same time
    (src/RMAD/OperationNeuralNetworkVisitor.cs:303-306)."""
    cases = []
    for s in range(6):
        A, B, dC = inputs(np.float64, 60 + s, 80, 50 - s, seed=100 + s)
        op = GpuMatrixMultiplyOperation.Instantiate(None)
        op.Forward(Matrix.from_numpy(A), Matrix.from_numpy(B))
        cases.append((op, A, B, dC))
    results = [None] * len(cases)
    errors = []

    def work(i):
        try:
            for _ in range(5):
                results[i] = cases[i][0].Backward(Matrix.from_numpy(cases[i][3]))
        except Exception as exc:  # pragma: no cover
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(cases))]
    [t.start() for t in threads]
    [t.join() for t in threads]
    assert not errors
    for (op, A, B, dC), res in zip(cases, results):
        rdA, rdB = oracle.matmul_bwd(dC, A, B)
        assert_parity(res.Item1.to_numpy(), rdA, np.float64)
        assert_parity(res.Item2.to_numpy(), rdB, np.float64)


def test_raw_pointer_entry_point_with_leading_dimensions(gpu, oracle):
    lib = _lib.load()
    from parallelreverseautodiff_amd.exceptions import check
    M, K, N, lda, ldb, ldc = 50, 40, 30, 47, 33, 36
    A = seeded.uniform(2, 1, (M, lda), -1, 1); B = seeded.uniform(2, 2, (K, ldb), -1, 1)
    dA_, dB_, dC_ = DeviceBuffer.alloc(np.float64, M, lda), DeviceBuffer.alloc(np.float64, K, ldb), DeviceBuffer.alloc(np.float64, M, ldc)
    dA_.upload(A); dB_.upload(B)
    check(lib.prad_gemm_f64(0, 0, M, N, K, dA_.ptr, lda, dB_.ptr, ldb, dC_.ptr, ldc, 0))
    got = dC_.download()
    assert_parity(got[:, :N], oracle.matmul_fwd(np.ascontiguousarray(A[:, :K]), np.ascontiguousarray(B[:, :N])), np.float64)
    assert not got[:, N:].any()  # padding columns untouched
    assert lib.prad_gemm_f64(0, 0, M, N, K, dA_.ptr, K - 1, dB_.ptr, ldb, dC_.ptr, ldc, 0) == _lib.PRAD_ERR_ARG


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("shape", [(64, 784, 256), (64, 128, 10), (1024, 64, 64), (2500, 40, 70), (33, 17, 129)])
def test_bias_gradient_riding_with_the_weight_gradient(gpu, dtype, shape):
    """prad_matmul_bias_bwd = prad_add_broadcast_bwd_bias + prad_matmul_bwd_fused, bit for bit: the column sum
    shares the launch of the dB product (also when that product is split along K: 1024 x 64 x 64) or gets its
    own launches (no dB requested; 2500 rows, which are summed in row chunks)."""
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    M, K, N = shape
    A, B, dC, Z = (seeded.normal(71, i, s, 1.0, dtype) for i, s in enumerate([(M, K), (K, N), (M, N), (M, K)]))
    up = lambda a: (lambda b: (b.upload(a), b)[1])(DeviceBuffer.alloc(dtype, *a.shape))
    bA, bB, bdC, bZ = up(A), up(B), up(dC), up(Z)
    dA1, dA2 = DeviceBuffer.alloc(dtype, M, K), DeviceBuffer.alloc(dtype, M, K)
    dB1, dB2 = DeviceBuffer.alloc(dtype, K, N), DeviceBuffer.alloc(dtype, K, N)
    db1, db2, db3 = (DeviceBuffer.alloc(dtype, 1, N) for _ in range(3))
    check(lib.prad_add_broadcast_bwd_bias(bdC.handle, db1.handle))
    check(lib.prad_matmul_bwd_fused(bdC.handle, bA.handle, bB.handle, dA1.handle, dB1.handle, 0, _lib.ACT_LEAKYRELU, bZ.handle, 0.01))
    check(lib.prad_matmul_bias_bwd(bdC.handle, bA.handle, bB.handle, dA2.handle, dB2.handle, db2.handle, 0, _lib.ACT_LEAKYRELU,
                                   bZ.handle, 0.01))
    check(lib.prad_matmul_bias_bwd(bdC.handle, bA.handle, bB.handle, None, None, db3.handle, 0, _lib.ACT_NONE, None, 0.0))
    assert np.array_equal(dA1.download(), dA2.download())
    assert np.array_equal(dB1.download(), dB2.download())
    assert np.array_equal(db1.download(), db2.download())
    assert np.array_equal(db1.download(), db3.download())
    assert_parity(db2.download(), dC.astype(np.float64).sum(axis=0, keepdims=True).astype(dtype), dtype, "bias gradient")


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("accumulate", [0, 1])
@pytest.mark.parametrize("shape", [(64, 784, 256), (64, 256, 128), (64, 128, 10), (33, 17, 129), (50, 49, 49), (1, 1, 1),
                                   (96, 200, 72), (300, 300, 300), (1024, 1024, 1024), (1000, 1100, 1040), (1000, 1001, 1003),
                                   (2000, 2100, 2050), (2304, 2304, 2304)])
def test_both_gradients_in_one_launch(gpu, dtype, accumulate, shape):
    """A layer gets dA = dC . B^T (with the activation's backward) and dB = A^T . dC (+ bias gradient) from one
    launch where both products run unsplit on tiles of one size (32 x 32, 64 x 64 around a thousand rows and columns,
    128 x 128 around two thousand); asking for one gradient at a time takes the single-product launches.  Same bits
    either way, for aligned and misaligned operands, whole and ragged tiles, with and without accumulation into dB,
    and for a shape too large for the joint launch."""
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    M, K, N = shape
    A, B, dC, Z, dB0 = (seeded.normal(73, i, s, 1.0, dtype) for i, s in enumerate([(M, K), (K, N), (M, N), (M, K), (K, N)]))
    up = lambda a: (lambda b: (b.upload(a), b)[1])(DeviceBuffer.alloc(dtype, *a.shape))
    bA, bB, bdC, bZ = up(A), up(B), up(dC), up(Z)
    dA1, dA2, dB1, dB2 = DeviceBuffer.alloc(dtype, M, K), DeviceBuffer.alloc(dtype, M, K), up(dB0), up(dB0)
    db1, db2 = DeviceBuffer.alloc(dtype, 1, N), DeviceBuffer.alloc(dtype, 1, N)
    args = (accumulate, _lib.ACT_TANH, bZ.handle, 0.0)
    check(lib.prad_matmul_bias_bwd(bdC.handle, bA.handle, bB.handle, dA1.handle, None, None, *args))
    check(lib.prad_matmul_bias_bwd(bdC.handle, bA.handle, bB.handle, None, dB1.handle, db1.handle, *args))
    check(lib.prad_matmul_bias_bwd(bdC.handle, bA.handle, bB.handle, dA2.handle, dB2.handle, db2.handle, *args))
    assert np.array_equal(dA1.download(), dA2.download())
    assert np.array_equal(dB1.download(), dB2.download())
    assert np.array_equal(db1.download(), db2.download())
    # plain upstream gradient (no activation): prad_matmul_bwd against the two single products
    check(lib.prad_gemm(0, 1, bdC.handle, bB.handle, dA1.handle, 0))
    check(lib.prad_gemm(1, 0, bA.handle, bdC.handle, dB1.handle, 0))
    check(lib.prad_matmul_bwd(bdC.handle, bA.handle, bB.handle, dA2.handle, dB2.handle, 0, 0))
    assert np.array_equal(dA1.download(), dA2.download())
    assert np.array_equal(dB1.download(), dB2.download())
    ref_dA = dC.astype(np.float64) @ B.astype(np.float64).T
    assert_parity(dA2.download(), ref_dA.astype(dtype), dtype, "dA", bound=dot_bound(dC, B.T, dtype))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("shape", [(512, 2048, 512), (1024, 1024, 1024), (384, 2100, 500), (512, 4096, 512), (256, 8192, 2048), (500, 6000, 1000)])
def test_products_of_few_tiles_and_long_k(gpu, oracle, dtype, shape):
    """Shapes whose 64 x 64 or 32 x 32 tiles fill between half and one and a half of the chip's workgroup slots and
    whose K holds at least 32 slabs (which of these shapes do depends on the element type), and shapes of few 128 x 128
    tiles and a K of thousands, whose tiles are each shared by several workgroups: parity with the oracle
    for the forward and both backward layouts, fused epilogue included, and the same bits on every run.  With
    PRAD_GEMM_PAIRS=1 in the environment (test_workgroup_pairs_when_switched_on runs this test that way) they run
    with two workgroups per tile, half of K each, the later one adding the other's partial tile: the same bits then
    whichever workgroup of a pair arrives last."""
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    M, K, N = shape
    A = seeded.uniform(91, 1, (M, K), -1.0, 1.0, dtype)
    B = seeded.uniform(91, 2, (K, N), -1.0, 1.0, dtype)
    dC = seeded.normal(91, 3, (M, N), 1.0, dtype)
    bias = seeded.normal(91, 4, (1, N), 1.0, dtype)
    up = lambda a: (lambda b: (b.upload(a), b)[1])(DeviceBuffer.alloc(dtype, *a.shape))
    bA, bB, bdC, bbias = up(A), up(B), up(dC), up(bias)
    C, Z, H = (DeviceBuffer.alloc(dtype, M, N) for _ in range(3))
    dA, dB = DeviceBuffer.alloc(dtype, M, K), DeviceBuffer.alloc(dtype, K, N)
    first = None
    for run in range(4):
        check(lib.prad_matmul_fwd(bA.handle, bB.handle, C.handle))
        check(lib.prad_matmul_fwd_fused(bA.handle, bB.handle, bbias.handle, Z.handle, H.handle, _lib.ACT_LEAKYRELU, 0.01))
        check(lib.prad_matmul_bwd(bdC.handle, bA.handle, bB.handle, dA.handle, dB.handle, 0, 0))
        got = [x.download() for x in (C, Z, H, dA, dB)]
        if first is None:
            first = got
        else:
            for a, b2 in zip(first, got):
                assert np.array_equal(a, b2), "run %d differs from run 0" % run
    # accumulation into the output: the same product added to itself is exactly twice its bits
    check(lib.prad_gemm(0, 0, bA.handle, bB.handle, C.handle, 1))
    assert np.array_equal(C.download(), first[0] + first[0]), "C += A . B"
    if dtype == np.float32 and K >= 4096:
        # The float oracle adds 4096 terms one by one and is itself about 1e-5 off the exact sum, more than the GPU's
        # blocked sums are; both are therefore held against the product taken in double and rounded once.
        wide = lambda x: x.astype(np.float64)
        rC = oracle.matmul_fwd(wide(A), wide(B), threads=8).astype(dtype)
        # (the oracle's own sum: every entry within its rounding bound of the double product - at K = 8192 its normwise
        # error is already 1.3e-5)
        off = np.abs(oracle.matmul_fwd(A, B, threads=8).astype(np.float64) - rC.astype(np.float64))
        assert np.all(off <= dot_bound(A, B, dtype)), "oracle C against the double product"
    else:
        rC = oracle.matmul_fwd(A, B, threads=8)
    rdA, rdB = oracle.matmul_bwd(dC, A, B, threads=8)
    rZ = oracle.add_broadcast_fwd(rC, bias)
    assert_parity(first[0], rC, dtype, "C", bound=dot_bound(A, B, dtype))
    assert_parity(first[1], rZ, dtype, "Z")
    assert_parity(first[2], oracle.leakyrelu_fwd(rZ, dtype(0.01)), dtype, "H")
    assert_parity(first[3], rdA, dtype, "dA", bound=dot_bound(dC, B.T, dtype))
    assert_parity(first[4], rdB, dtype, "dB", bound=dot_bound(A.T, dC, dtype))


def test_operand_larger_than_four_gib(gpu):
    """A 40000 x 30000 float operand (4.8 GB): tile bases lie beyond 2^32 bytes while the per-lane offsets inside a
    slab stay 32-bit.  The operand is 40 copies of one 1000-row block, so every block of 1000 output rows of
    A . B equals the first one, and that one the product taken in double; the same operand read mn-contiguously
    (A^T . dC, dC with the same period) gives 40 times one block's contribution."""
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    lib = _lib.load()
    block_rows, copies, K, N = 1000, 40, 30000, 64
    M = block_rows * copies
    block = seeded.uniform(97, 1, (block_rows, K), -1, 1, np.float32)
    B = seeded.uniform(97, 2, (K, N), -1, 1, np.float32)
    dblock = seeded.uniform(97, 3, (block_rows, N), -1, 1, np.float32)
    A, dC = DeviceBuffer.alloc(np.float32, M, K), DeviceBuffer.alloc(np.float32, M, N)
    for c in range(copies):
        A.view_rows(c * block_rows, block_rows).upload(block)
        dC.view_rows(c * block_rows, block_rows).upload(dblock)
    bB = DeviceBuffer.alloc(np.float32, K, N)
    bB.upload(B)
    C, dB = DeviceBuffer.alloc(np.float32, M, N), DeviceBuffer.alloc(np.float32, K, N)
    check(lib.prad_matmul_fwd(A.handle, bB.handle, C.handle))
    check(lib.prad_gemm(1, 0, A.handle, dC.handle, dB.handle, 0))
    got = C.download()
    first = got[:block_rows]
    ref = block.astype(np.float64) @ B.astype(np.float64)
    assert np.max(np.abs(first - ref)) <= 1e-5 * np.max(np.abs(ref))
    for c in (1, 17, 26, copies - 1):  # 1000 rows are not a multiple of the 128-row tile: compare within tolerance
        assert np.max(np.abs(got[c * block_rows:(c + 1) * block_rows] - ref)) <= 1e-5 * np.max(np.abs(ref))
    ref_dB = copies * (block.astype(np.float64).T @ dblock.astype(np.float64))
    # (40000 float terms per entry that add up coherently, block after block: the rounding of the running sums
    # is what the wider bar is for; a wrong tile base would be off by the size of the entries themselves)
    assert np.max(np.abs(dB.download() - ref_dB)) <= 1e-4 * np.max(np.abs(ref_dB))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(50176, 96, 288), (50001, 100, 96), (49160, 8, 128), (50176, 96, 384)])
def test_tall_products_of_few_slabs(gpu, oracle, dtype, shape):
    """A layer of about a hundred inputs applied to fifty thousand rows: hundreds of 128 x 128 tiles of one to
    six K slabs, the shapes that the half-depth kernel takes (all three layouts, a ragged last row tile, a K that
    ends inside a slab, plain and elementwise epilogues).  Held entry by entry against the product in double."""
    lib = _lib.load()
    from parallelreverseautodiff_amd.exceptions import check
    M, K, N = shape
    A = seeded.uniform(41, 1, (M, K), -1, 1, dtype)
    B = seeded.uniform(41, 2, (K, N), -1, 1, dtype)
    G = seeded.normal(41, 3, (M, N), 1.0, dtype)
    dA_, dB_, dG_ = (DeviceBuffer.alloc(dtype, *x.shape) for x in (A, B, G))
    dA_.upload(A); dB_.upload(B); dG_.upload(G)
    C = DeviceBuffer.alloc(dtype, M, N)
    check(lib.prad_gemm(0, 0, dA_.handle, dB_.handle, C.handle, 0))                      # A . B
    assert_parity(C.download(), A.astype(np.float64) @ B.astype(np.float64), dtype, "A.B", bound=dot_bound(A, B, dtype))
    dX = DeviceBuffer.alloc(dtype, M, K)
    check(lib.prad_gemm(0, 1, dG_.handle, dB_.handle, dX.handle, 0))                     # G . B^T: K of this product is N
    assert_parity(dX.download(), G.astype(np.float64) @ B.T.astype(np.float64), dtype, "G.B^T", bound=dot_bound(G, B.T, dtype))
    # bias, pre-activation copy and GELU in the epilogue; then GELU' of the pre-activation on the way back
    bias = seeded.normal(41, 4, (1, N), 0.5, dtype)
    db = DeviceBuffer.alloc(dtype, 1, N); db.upload(bias)
    Z, H = DeviceBuffer.alloc(dtype, M, N), DeviceBuffer.alloc(dtype, M, N)
    check(lib.prad_matmul_fwd_fused(dA_.handle, dB_.handle, db.handle, Z.handle, H.handle, _lib.ACT_GELU, 0.0))
    gZ = Z.download()
    assert_parity(gZ, A.astype(np.float64) @ B.astype(np.float64) + bias.astype(np.float64), dtype, "Z",
                  bound=dot_bound(A, B, dtype) + 4 * np.finfo(dtype).eps * (np.abs(gZ) + np.abs(bias)))
    rows = slice(M - 300, M)                                                             # the oracle's elementwise part on the last rows
    assert_parity(H.download()[rows], oracle.gelu_fwd(np.ascontiguousarray(gZ[rows])), dtype, "GELU(Z)")
    src = seeded.normal(41, 5, (M, K), 1.0, dtype)
    dS = DeviceBuffer.alloc(dtype, M, K); dS.upload(src)
    dAct = DeviceBuffer.alloc(dtype, M, K)
    check(lib.prad_matmul_bwd_fused(dG_.handle, dA_.handle, dB_.handle, dAct.handle, None, 0, _lib.ACT_GELU, dS.handle, 0.0))
    plain = dX.download()[rows]
    assert_parity(dAct.download()[rows], oracle.gelu_bwd(np.ascontiguousarray(src[rows]), np.ascontiguousarray(plain)), dtype, "GELU' (.) dX")


@pytest.mark.parametrize("shape", [(16384, 96, 288), (9000, 96, 96), (8200, 384, 96), (12001, 288, 96), (8192, 64, 384), (10000, 20, 48)])
def test_rows_of_a_tall_product_do_not_depend_on_how_many_rows_there_are(gpu, oracle, shape):
    """Row i of a product depends on row i of A only, and the tiled kernels all add along K in the same order, whatever
    tile the sizes select (a tall product runs on 128 x 128 tiles, its first 4096 rows alone on smaller ones): the first
    4096 rows of the tall product equal the product of the first 4096 rows bit for bit - for every epilogue (bias,
    pre-activation copy, activation, the upstream activation's derivative, accumulation), both layouts of B, and a
    ragged last tile.  From 8192 rows on, products with K a multiple of 96 run on the streaming kernel, which loads four
    consecutive k per lane and transposes them across the lane groups so that its MFMA steps see k = 4 s + g as well:
    the same bits there too."""
    lib = _lib.load()
    from parallelreverseautodiff_amd.exceptions import check
    dtype = np.float32
    M, K, N = shape
    head = 4096

    def same(x, y):
        return np.array_equal(x, y)
    A = seeded.uniform(43, 1, (M, K), -1, 1, dtype)
    B = seeded.uniform(43, 2, (K, N), -1, 1, dtype)
    Bt = np.ascontiguousarray(B.T)                                  # N x K: the operand of dC . W^T
    bias = seeded.normal(43, 3, (1, N), 0.5, dtype)
    src = seeded.normal(43, 4, (M, N), 1.0, dtype)
    old = seeded.normal(43, 5, (M, N), 1.0, dtype)
    up = lambda a: (lambda b: (b.upload(a), b)[1])(DeviceBuffer.alloc(dtype, *a.shape))
    bA, bB, bBt, bbias, bsrc = up(A), up(B), up(Bt), up(bias), up(src)
    hA, hsrc = bA.view_rows(0, head), bsrc.view_rows(0, head)

    def both(call):
        """Runs `call(A, act_src, out buffers...)` on all rows and on the first `head` rows; returns the downloads."""
        full = [DeviceBuffer.alloc(dtype, M, N) for _ in range(2)]
        part = [DeviceBuffer.alloc(dtype, head, N) for _ in range(2)]
        full[1].upload(old); part[1].upload(old[:head])
        call(bA, bsrc, *full)
        call(hA, hsrc, *part)
        return [f.download() for f in full], [q.download() for q in part]

    # plain store, and accumulation into C
    f, q = both(lambda a, s, c0, c1: (check(lib.prad_gemm(0, 0, a.handle, bB.handle, c0.handle, 0)),
                                      check(lib.prad_gemm(0, 0, a.handle, bB.handle, c1.handle, 1))))
    assert same(f[0][:head], q[0]) and same(f[1][:head], q[1])
    assert_parity(f[0], A.astype(np.float64) @ B.astype(np.float64), dtype, "A.B", bound=dot_bound(A, B, dtype))
    assert_parity(f[1], old + A.astype(np.float64) @ B.astype(np.float64), dtype, "C += A.B")
    # B stored N x K (the layout of dA = dC . W^T)
    f, q = both(lambda a, s, c0, c1: check(lib.prad_gemm(0, 1, a.handle, bBt.handle, c0.handle, 0)))
    assert same(f[0][:head], q[0])
    assert_parity(f[0], A.astype(np.float64) @ B.astype(np.float64), dtype, "A.(B^T)^T", bound=dot_bound(A, B, dtype))
    # bias, pre-activation copy, activation
    f, q = both(lambda a, s, c0, c1: check(lib.prad_matmul_fwd_fused(a.handle, bB.handle, bbias.handle, c1.handle, c0.handle, _lib.ACT_TANH, 0.0)))
    assert same(f[0][:head], q[0]) and same(f[1][:head], q[1])
    assert_parity(f[0][-200:], oracle.tanh_fwd(np.ascontiguousarray(f[1][-200:])), dtype, "tanh(Z), last rows")
    # the upstream activation's derivative on the way out (dA = (dC . W^T) (.) act'(src)): here "dC" = A, "W" = B^T
    f, q = both(lambda a, s, c0, c1: check(lib.prad_matmul_bwd_fused(a.handle, s.handle, bBt.handle, c0.handle, None, 0, _lib.ACT_SIGMOID, s.handle, 0.0)))
    assert same(f[0][:head], q[0])


@pytest.mark.parametrize("forced_tile", [None, "64x64"])
def test_workgroup_pairs_when_switched_on(gpu, forced_tile):
    """Pairs of workgroups per tile are a tuning aid that is off by default (the library reads PRAD_GEMM_PAIRS once):
    the test above runs again in a process of its own with the switch on - and once more with the tile size forced as
    well, where a product can qualify both for pairs and for tiles shared several ways (it is launched on the shared
    tiles, and the workspace has to be sized for those)."""
    import os, subprocess, sys
    env = dict(os.environ, PRAD_GEMM_PAIRS="1")
    if forced_tile:
        env["PRAD_GEMM_TILE"] = forced_tile
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.join(root, "tests", "test_matmul_gpu.py"), "-q", "-x", "-m", "gpu",
                        "-k", "test_products_of_few_tiles_and_long_k", "-p", "no:cacheprovider"],
                       cwd=root, env=env, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "12 passed" in r.stdout, r.stdout[-2000:]


@pytest.mark.parametrize("shape", [(50176, 96, 288), (8192, 96, 96), (16384, 384, 96), (12288, 96, 384), (4096, 64, 320), (20000, 32, 48)])
def test_weight_gradient_of_a_tall_batch_in_one_pass(gpu, oracle, shape):
    """dB = A^T . dC in float for thousands of rows and a small output runs as one pass over A and dC (every workgroup
    multiplies a range of rows into the whole output, a second launch adds the partial outputs in order), and the bias
    gradient - the column sums of dC - is taken in the same pass when prad_matmul_bias_bwd asks for both.  Held against
    the product and the sums in double, with and without accumulation into dB; the same bits on every run; the bias
    gradient equal to the one of the call that asks for it alone."""
    lib = _lib.load()
    from parallelreverseautodiff_amd.exceptions import check
    dtype = np.float32
    K, M, N = shape                                   # K rows of the batch, M inputs, N outputs of the layer
    A = seeded.uniform(47, 1, (K, M), -1, 1, dtype)
    dC = seeded.normal(47, 2, (K, N), 1.0, dtype)
    W = seeded.normal(47, 3, (M, N), 1.0, dtype)
    old = seeded.normal(47, 4, (M, N), 1.0, dtype)
    up = lambda a: (lambda b: (b.upload(a), b)[1])(DeviceBuffer.alloc(dtype, *a.shape))
    bA, bdC, bW = up(A), up(dC), up(W)
    ref = A.astype(np.float64).T @ dC.astype(np.float64)
    ref_db = dC.astype(np.float64).sum(axis=0, keepdims=True)
    first = None
    for run in range(3):
        dB, dBacc, db, db_alone = DeviceBuffer.alloc(dtype, M, N), up(old), DeviceBuffer.alloc(dtype, 1, N), DeviceBuffer.alloc(dtype, 1, N)
        check(lib.prad_matmul_bias_bwd(bdC.handle, bA.handle, bW.handle, None, dB.handle, db.handle, 0, _lib.ACT_NONE, None, 0.0))
        check(lib.prad_matmul_bwd(bdC.handle, bA.handle, bW.handle, None, dBacc.handle, 0, 1))
        check(lib.prad_add_broadcast_bwd_bias(bdC.handle, db_alone.handle))
        got = [x.download() for x in (dB, dBacc, db, db_alone)]
        if first is None:
            first = got
        else:
            for a, b in zip(first, got):
                assert np.array_equal(a, b), "run %d differs from run 0" % run
    # (thousands of float terms per entry: the bar of the long sums, see assert_long_sum_parity)
    scale = np.sqrt(np.mean(ref ** 2))
    assert np.max(np.abs(first[0] - ref)) <= 2e-5 * max(scale, np.max(np.abs(ref)) * 1e-3) + 1e-5 * np.max(np.abs(ref)), "dB"
    assert np.max(np.abs(first[1] - (old + ref))) <= 2e-5 * np.max(np.abs(ref)), "dB accumulated"
    assert_parity(first[2], ref_db.astype(dtype), dtype, "bias gradient")
    assert np.array_equal(first[2], first[3])


@pytest.mark.parametrize("shape", [(16, 40, 16), (33, 128, 10), (7, 5, 3)])
def test_a_product_is_one_chain_of_fused_multiply_adds_along_k(gpu, shape):
    """What fixes a product's bits on this hardware: the matrix instruction adds its terms as fused multiply-adds along
    ascending k (one rounding per term), and every kernel hands it k in ascending order.  In double this is checked
    against exact rational arithmetic rounded once per term; it is what lets kernels of different shapes (and the
    one-workgroup classifier head, which restates the products) give identical results."""
    from fractions import Fraction
    M, K, N = shape
    A = seeded.normal(77, 1, (M, K), 1.0, np.float64)
    B = seeded.normal(77, 2, (K, N), 1.0, np.float64)
    op = MatrixMultiplyOperation.Instantiate(None)
    C = op.Forward(Matrix.from_numpy(A), Matrix.from_numpy(B)).to_numpy()
    ref = np.empty((M, N))
    for i in range(M):
        for j in range(N):
            acc = 0.0
            for k in range(K):
                acc = float(Fraction(A[i, k]) * Fraction(B[k, j]) + Fraction(acc))   # correctly rounded: one fma
            ref[i, j] = acc
    assert np.array_equal(C, ref)
