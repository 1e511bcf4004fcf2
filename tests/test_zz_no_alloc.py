"""The allocation-free form of the clip + Adam update (prad_clip_adam_multi_noalloc) against the entry point it is a
variant of (prad_clip_adam_multi): bit for bit, on two calls in a row, the second on smaller tensors, so that anything
the first call left in the static scratch would show; then its limits."""
import numpy as np
import pytest

from parallelreverseautodiff_amd import _lib, seeded
from parallelreverseautodiff_amd.exceptions import check
from parallelreverseautodiff_amd.matrix import DeviceBuffer
from parallelreverseautodiff_amd.operations import handle_array

pytestmark = pytest.mark.gpu

CLIP, MIN, LR, B1, B2, EPS = 4.0, 1e-16, 1e-3, 0.9, 0.999, 1e-8


def make_group(dtype, shapes, seed):
    host = []
    for i, shape in enumerate(shapes):
        w = seeded.normal(seed, 10 * i + 1, shape, 0.5, dtype)
        g = seeded.normal(seed, 10 * i + 2, shape, 2.0, dtype)
        g.reshape(-1)[::97] *= 40.0                         # outliers that the clamp catches
        g.reshape(-1)[5::1013] = 1e-20                      # magnitudes below the floor
        m = seeded.normal(seed, 10 * i + 3, shape, 0.1, dtype)
        v = np.abs(seeded.normal(seed, 10 * i + 4, shape, 0.1, dtype))
        host.append((w, m, v, g))
    return host


def upload(dtype, host):
    dev = []
    for arrays in host:
        bufs = []
        for x in arrays:
            b = DeviceBuffer.alloc(dtype, *x.shape)
            b.upload(x)
            bufs.append(b)
        dev.append(bufs)
    return dev


def run(entry, dev, t):
    cols = list(zip(*dev))                                  # (w...), (m...), (v...), (g...)
    w, m, v, g = (handle_array(list(c)) for c in cols)
    check(entry(w, m, v, g, len(dev), CLIP, MIN, LR, B1, B2, EPS, float(t)))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_no_alloc_clip_adam_equals_the_allocating_entry_point(gpu, dtype):
    lib = _lib.load()
    # first call: a model-sized group (one tensor of several hundred chunks, ragged ones, a 1 x 1); second: smaller
    first = [(784, 256), (1, 256), (256, 128), (1, 1), (1237, 911), (3, 5)]
    second = [(64, 10), (1, 10), (129, 33)]
    for shapes, seed, t in ((first, 11, 1.0), (second, 12, 2.0)):
        host = make_group(dtype, shapes, seed)
        ref, got = upload(dtype, host), upload(dtype, host)
        run(lib.prad_clip_adam_multi, ref, t)
        run(lib.prad_clip_adam_multi_noalloc, got, t)
        gpu.Synchronize()
        for i, (r, x) in enumerate(zip(ref, got)):
            for name, rb, xb in zip("wmvg", r, x):
                a, b = rb.download(), xb.download()
                assert np.array_equal(a, b), "%s of tensor %d %s differs" % (name, i, shapes[i])
            assert not np.array_equal(x[0].download(), host[i][0]) or host[i][0].size == 0   # the update did happen


def test_no_alloc_limits(gpu):
    lib = _lib.load()
    dtype = np.float32
    one = upload(dtype, make_group(dtype, [(4, 4)], 1))
    cols = list(zip(*(one * 65)))
    w, m, v, g = (handle_array(list(c)) for c in cols)
    assert lib.prad_clip_adam_multi_noalloc(w, m, v, g, 65, CLIP, MIN, LR, B1, B2, EPS, 1.0) == _lib.PRAD_ERR_ARG
    assert "at most 64 tensors" in lib.prad_last_error().decode()
    # more chunks than the static scratch holds: 45 000 chunks of 4096 floats (uninitialised contents do not matter,
    # nothing is enqueued)
    big = [DeviceBuffer.alloc(dtype, 45000, 4096) for _ in range(2)]
    h = handle_array([big[0]])
    hg = handle_array([big[1]])
    assert lib.prad_clip_adam_multi_noalloc(h, h, h, hg, 1, CLIP, MIN, LR, B1, B2, EPS, 1.0) == _lib.PRAD_ERR_ARG
    assert "static scratch" in lib.prad_last_error().decode()
    assert lib.prad_clip_adam_multi_noalloc(h, h, h, hg, 0, CLIP, MIN, LR, B1, B2, EPS, 1.0) == _lib.PRAD_OK
