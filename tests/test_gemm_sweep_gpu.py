"""Seeded sweep of product shapes through the raw-pointer entry points (prad_gemm_f64/f32 and the strided
batched forms): every layout, ragged sizes on either side of each tile and slab edge, padded leading dimensions,
accumulation, batches with shared operands.  Every entry of every result is held against its own rounding bound
around the product taken in double (conftest.dot_bound), which a dropped, duplicated or misplaced term breaks;
the padding of C must come back untouched.  The shapes are drawn so that each kernel family is met: guarded and
vector-load kernels, the three tile sizes, products split along K, workgroup pairs, the single-stage kernel for
batches of one-slab products."""
import numpy as np
import pytest

from conftest import assert_parity, dot_bound
from parallelreverseautodiff_amd import _lib
from parallelreverseautodiff_amd.exceptions import check
from parallelreverseautodiff_amd.matrix import DeviceBuffer

pytestmark = pytest.mark.gpu

LAYOUTS = [(0, 0), (0, 1), (1, 0)]
EDGES = [1, 2, 3, 4, 15, 16, 17, 31, 32, 33, 48, 49, 63, 64, 65, 96, 127, 128, 129, 130, 200, 255, 256, 257, 300]


def _draw_dim(rng, big):
    if rng.random() < 0.6:
        return int(rng.choice(EDGES))
    return int(rng.integers(1, big))


def _operand(rng, rows, cols, ld, dtype):
    full = rng.uniform(-1, 1, (rows, ld)).astype(dtype)
    return full, np.ascontiguousarray(full[:, :cols])


def _single_case(lib, rng, dtype, idx):
    tA, tB = LAYOUTS[idx % 3]
    M, N = _draw_dim(rng, 400), _draw_dim(rng, 400)
    K = _draw_dim(rng, 1500 if idx % 5 == 0 else 400)
    pad = (lambda: int(rng.integers(0, 8))) if idx % 2 else (lambda: 0)   # every other case keeps rows 16-byte aligned when it can
    a_rows, a_cols = (K, M) if tA else (M, K)
    b_rows, b_cols = (N, K) if tB else (K, N)
    lda, ldb, ldc = a_cols + pad(), b_cols + pad(), N + pad()
    Af, A = _operand(rng, a_rows, a_cols, lda, dtype)
    Bf, B = _operand(rng, b_rows, b_cols, ldb, dtype)
    C0 = rng.uniform(-1, 1, (M, ldc)).astype(dtype)
    accumulate = int(rng.random() < 0.3)
    dA_, dB_, dC_ = DeviceBuffer.alloc(dtype, a_rows, lda), DeviceBuffer.alloc(dtype, b_rows, ldb), DeviceBuffer.alloc(dtype, M, ldc)
    dA_.upload(Af); dB_.upload(Bf); dC_.upload(C0)
    fn = lib.prad_gemm_f64 if dtype == np.float64 else lib.prad_gemm_f32
    what = "case %d %s tA=%d tB=%d M=%d N=%d K=%d ld=(%d,%d,%d) acc=%d" % (idx, np.dtype(dtype).name, tA, tB, M, N, K, lda, ldb, ldc, accumulate)
    print(what, flush=True)
    check(fn(tA, tB, M, N, K, dA_.ptr, lda, dB_.ptr, ldb, dC_.ptr, ldc, accumulate))
    got = dC_.download()
    opA, opB = (A.T if tA else A), (B.T if tB else B)
    ref = opA.astype(np.float64) @ opB.astype(np.float64)
    bound = dot_bound(opA, opB, dtype)
    if accumulate:
        ref = ref + C0[:, :N].astype(np.float64)
        bound = bound + 2.0 * float(np.finfo(dtype).eps) * (np.abs(ref) + np.abs(C0[:, :N]))
    assert_parity(got[:, :N], ref, dtype, what, bound=bound + 1e-300)
    assert np.array_equal(got[:, N:], C0[:, N:]), what + ": padding of C written"


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_single_products_over_ragged_shapes(gpu, dtype):
    lib = _lib.load()
    rng = np.random.default_rng(20240611 + (0 if dtype == np.float64 else 1))
    for idx in range(90):
        _single_case(lib, rng, dtype, idx)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_batched_products_over_ragged_shapes(gpu, dtype):
    """Strided batches, some with a shared operand (stride 0), some large enough in count and short enough in K
    for the single-stage kernel (K of a slab or less, 64 products or more)."""
    lib = _lib.load()
    rng = np.random.default_rng(777 + (0 if dtype == np.float64 else 1))
    fn = lib.prad_gemm_strided_batched_f64 if dtype == np.float64 else lib.prad_gemm_strided_batched_f32
    for idx in range(40):
        tA, tB = LAYOUTS[idx % 3]
        batch = int(rng.choice([1, 2, 7, 64, 65, 200]))
        M, N = int(rng.choice([1, 7, 16, 31, 32, 33, 49, 64, 65, 100])), int(rng.choice([1, 8, 17, 32, 49, 64, 66, 96]))
        K = int(rng.choice([1, 3, 16, 31, 32, 33, 49, 64, 65, 128, 129, 200]))
        a_rows, a_cols = (K, M) if tA else (M, K)
        b_rows, b_cols = (N, K) if tB else (K, N)
        share_a, share_b = rng.random() < 0.2, rng.random() < 0.2
        nA, nB = (1 if share_a else batch), (1 if share_b else batch)
        A = rng.uniform(-1, 1, (nA, a_rows, a_cols)).astype(dtype)
        B = rng.uniform(-1, 1, (nB, b_rows, b_cols)).astype(dtype)
        dA_ = DeviceBuffer.alloc(dtype, a_rows, a_cols, depth=nA); dB_ = DeviceBuffer.alloc(dtype, b_rows, b_cols, depth=nB)
        dC_ = DeviceBuffer.alloc(dtype, M, N, depth=batch)
        dA_.upload(A); dB_.upload(B)
        what = "batch case %d %s tA=%d tB=%d batch=%d M=%d N=%d K=%d shared=(%d,%d)" % (
            idx, np.dtype(dtype).name, tA, tB, batch, M, N, K, share_a, share_b)
        print(what, flush=True)
        check(fn(tA, tB, M, N, K, dA_.ptr, a_cols, 0 if share_a else a_rows * a_cols, dB_.ptr, b_cols,
                 0 if share_b else b_rows * b_cols, dC_.ptr, N, M * N, batch, 0))
        got = dC_.download().reshape(batch, M, N)
        for b in range(batch):
            a, bb = A[0 if share_a else b], B[0 if share_b else b]
            opA, opB = (a.T if tA else a), (bb.T if tB else bb)
            ref = opA.astype(np.float64) @ opB.astype(np.float64)
            assert_parity(got[b], ref, dtype, what + " slice %d" % b, bound=dot_bound(opA, opB, dtype) + 1e-300)
