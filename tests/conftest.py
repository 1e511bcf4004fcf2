import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs through libprad_hip.so)")


# Parity contract.  "Max relative error" of a result x against the oracle's ref is measured per element
# against max(|ref|, rms(ref)): entries that cancel towards zero are judged against the typical magnitude
# of the matrix, because the reduction order of the MFMA kernels differs from the reference's k-ascending
# loop and neither order is exact there.  Bars: 1e-12 (double, PRAD), 1e-5 (float, PRADLite).
# A stricter floor (1e-3 * rms) is reported by strict_err() for the record but is not a pass bar: under it
# the reference's own float loop differs from the exactly rounded product by ~4e-4 at K = 64.
TOL = {np.dtype(np.float64): 1e-12, np.dtype(np.float32): 1e-5}


def _floored(x, ref, floor_factor):
    x = np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert x.shape == ref.shape, (x.shape, ref.shape)
    if ref.size == 0:
        return 0.0
    rms = float(np.sqrt(np.mean(ref * ref)))
    floor = max(floor_factor * rms, np.finfo(np.float64).tiny)
    return float(np.max(np.abs(x - ref) / np.maximum(np.abs(ref), floor)))


def rel_err(x, ref):
    """max |x - ref| / max(|ref|, rms(ref))"""
    return _floored(x, ref, 1.0)


def strict_err(x, ref):
    """max |x - ref| / max(|ref|, 1e-3 * rms(ref)) (reported, not a bar)"""
    return _floored(x, ref, 1e-3)


def norm_err(x, ref):
    """Normwise error max|x - ref| / max|ref|."""
    x = np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    scale = float(np.max(np.abs(ref))) if ref.size else 0.0
    diff = float(np.max(np.abs(x - ref))) if ref.size else 0.0
    return diff / scale if scale > 0 else diff


def dot_bound(absA, absB, dtype):
    """Componentwise rounding bound of a length-K dot product evaluated in `dtype` in any order:
    8 * sqrt(K) * eps * (|A| . |B|)_ij.  A dropped or misplaced term is ~1/K of |A|.|B| and breaks it."""
    K = absA.shape[1]
    return 8.0 * np.sqrt(K) * float(np.finfo(dtype).eps) * (np.abs(absA).astype(np.float64) @ np.abs(absB).astype(np.float64))


def assert_parity(x, ref, dtype, what="", bound=None):
    """Fails unless rel_err(x, ref) is within the bar; with `bound` (see dot_bound) also checks every entry
    against its own rounding bound, which is order independent and tighter for small entries."""
    err = rel_err(x, ref)
    tol = TOL[np.dtype(dtype)]
    assert err <= tol, "%s: relative error %.3e exceeds %.1e" % (what, err, tol)
    if bound is not None:
        excess = np.abs(np.asarray(x, np.float64) - np.asarray(ref, np.float64)) - bound
        assert float(np.max(excess)) <= 0.0, "%s: an entry is off by more than its rounding bound" % what
    return err


def assert_long_sum_parity(dev, ref, lhs, rhs, dtype, what=""):
    """Parity of dev = lhs^T . rhs (a weight gradient summed over thousands of rows) with the reference value `ref`.

    In float a sum of several thousand terms carries rounding noise of the size of the 1e-5 bar whatever its order
    (the reference's own k-ascending float loop is 3e-5 from the exact product at K = 50 000), so where the direct
    comparison exceeds the bar the result is held to what reordering can change and no more: every entry within the
    order-independent rounding bound 8 sqrt(K) eps (|lhs|^T.|rhs|)_ij of the product evaluated in double from the
    same operands, no further from that double value (in the relative measure of the other checks) than the bar or
    the distance of the reference's own arithmetic, whichever is larger, and within four times the bar of the
    reference (measured at K = 50 176: device 2e-6 and reference 2.9e-5 from the double product, 3.0e-5 apart).
    Returns the three errors
    (device vs reference, device vs double, reference vs double)."""
    tol = TOL[np.dtype(dtype)]
    direct = rel_err(dev, ref)
    lhs64, rhs64 = np.asarray(lhs, np.float64), np.asarray(rhs, np.float64)
    exact = lhs64.T @ rhs64
    e_dev, e_ref = rel_err(dev, exact), rel_err(ref, exact)
    if direct > tol:
        bound = 8.0 * np.sqrt(lhs64.shape[0]) * float(np.finfo(dtype).eps) * (np.abs(lhs64).T @ np.abs(rhs64))
        worst = float(np.max(np.abs(np.asarray(dev, np.float64) - exact) / bound))
        assert worst <= 1.0, "%s: an entry is off by %.2f x its rounding bound" % (what, worst)
        assert e_dev <= max(tol, e_ref), "%s: %.3e from the double product, the reference's arithmetic %.3e" % (what, e_dev, e_ref)
        assert direct <= 4.0 * tol, "%s: relative error %.3e against the reference" % (what, direct)
    return direct, e_dev, e_ref


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.load()
    return o


@pytest.fixture(scope="session")
def gpu():
    """Initialised library (device 0); GPU tests fail loudly when it cannot start."""
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    CudaBlas.Instance.DeviceId = 0
    CudaBlas.Instance.Initialize()
    assert CudaBlas.Instance.IsInitialized
    yield CudaBlas.Instance
