"""Seeded, counter-based input generator shared by tests, smoke check and benchmark.

The reference seeds its RNG from thread id and clock ticks (src/RMAD/MatrixUtils.cs:23), so it has
no reproducible inputs; every "seeded input" of a benchmark configuration is produced here.
Element i of tensor t under seed s is SplitMix64(SplitMix64(s ^ t*C) + i) mapped to a 53-bit
uniform in [0, 1); values do not depend on how the tensor is later split or ordered.
"""
import numpy as np

DEFAULT_SEED = 20240611
_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(z):
    with np.errstate(over="ignore"):
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def u01(seed, tensor, n, offset=0):
    """n uniforms in [0, 1) for element indices offset .. offset+n-1 of tensor `tensor`."""
    with np.errstate(over="ignore"):
        key = _splitmix64(np.array([np.uint64(seed) ^ (np.uint64(tensor) * np.uint64(0xD1B54A32D192ED03))], dtype=np.uint64))
        idx = np.arange(offset, offset + n, dtype=np.uint64)
        z = _splitmix64(key + idx)
    return (z >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def uniform(seed, tensor, shape, lo=0.0, hi=1.0, dtype=np.float64):
    n = int(np.prod(shape))
    return (lo + (hi - lo) * u01(seed, tensor, n)).reshape(shape).astype(dtype)


def normal(seed, tensor, shape, sigma=1.0, dtype=np.float64):
    """Box-Muller on uniform pairs (2i, 2i+1); generated in double and rounded once."""
    n = int(np.prod(shape))
    u = u01(seed, tensor, 2 * n)
    r = np.sqrt(-2.0 * np.log1p(-u[0::2]))
    return (sigma * r * np.cos(2.0 * np.pi * u[1::2])).reshape(shape).astype(dtype)


def xavier(seed, tensor, rows, cols, dtype=np.float64):
    """(2u - 1) * sqrt(6 / (rows + cols)), the formula of Matrix.InitializeXavier (src/RMAD/Matrix.cs:1037-1046)."""
    u = u01(seed, tensor, rows * cols)
    return ((2.0 * u - 1.0) * np.sqrt(6.0 / (rows + cols))).reshape(rows, cols).astype(dtype)


def one_hot_labels(seed, tensor, rows, classes, dtype=np.float64):
    labels = np.minimum((u01(seed, tensor, rows) * classes).astype(np.int64), classes - 1)
    out = np.zeros((rows, classes), dtype=dtype)
    out[np.arange(rows), labels] = 1
    return out
