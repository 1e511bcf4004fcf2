"""Parity of gradient clipping and Adam with the oracle; multi-tensor launches over a small model."""
import numpy as np
import pytest

from conftest import assert_parity, rel_err
from parallelreverseautodiff_amd import seeded
from parallelreverseautodiff_amd.matrix import DeepMatrix, Matrix
from parallelreverseautodiff_amd.optim import AdamOptimizer, GradientClipper, ModelLayer, NeuralNetworkParameters

pytestmark = pytest.mark.gpu
DTYPES = [np.float64, np.float32]


def layer_of(weights, grads, ms=None, vs=None):
    layer = ModelLayer()
    for i, w in enumerate(weights):
        layer.AddModelElementGroup("W%d" % i, w, grads[i], None if ms is None else ms[i], None if vs is None else vs[i])
    return layer


@pytest.mark.parametrize("dtype", DTYPES)
def test_clip_matches_oracle_on_a_model(gpu, oracle, dtype):
    params = NeuralNetworkParameters(lite=dtype == np.float32)
    shapes = [(784, 256), (1, 256), (256, 128), (1, 128), (128, 10), (1, 10), (1, 1), (3, 5000)]
    grads = []
    for i, s in enumerate(shapes):
        g = seeded.normal(51, i, s, 0.3 * (i + 1), dtype)
        if g.size > 100:
            g.reshape(-1)[7] = 40.0 * (i + 1)  # outlier: clamps to min(4, 1 + |z|)
            g.reshape(-1)[11] = 1e-20         # below the minimum magnitude
            g.reshape(-1)[13] = -1e-20
        grads.append(g)
    mats = [Matrix.from_numpy(g) for g in grads]
    GradientClipper(params).Clip([layer_of(mats, mats)])
    for g, m in zip(grads, mats):
        ref = oracle.clip(g, params.ClipValue, params.MinimumClipValue)
        got = m.to_numpy()
        assert_parity(got, ref, dtype, "clip %s" % (g.shape,))
        if g.size > 100:
            assert got.reshape(-1)[11] == dtype(params.MinimumClipValue) and got.reshape(-1)[13] == dtype(-params.MinimumClipValue)
            assert got.reshape(-1)[7] == dtype(4.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_clip_degenerate_matrices_are_unchanged(gpu, oracle, dtype):
    params = NeuralNetworkParameters(lite=dtype == np.float32)
    const = np.full((5, 6), 2.5, dtype)
    single = np.array([[123.0]], dtype)
    mats = [Matrix.from_numpy(const), Matrix.from_numpy(single)]
    GradientClipper(params).Clip([layer_of(mats, mats)])
    assert np.array_equal(mats[0].to_numpy(), const) and np.array_equal(mats[1].to_numpy(), single)


def test_clip_with_large_mean_small_spread(gpu, oracle):
    """Statistics must survive mean >> sigma: a sum-of-squares shortcut for the variance would be wrong by a
    factor here.  With mean/sigma = 1e9 the reference's own one-by-one sum carries ~1e-8 of rounding noise in
    its mean, so the comparison with the oracle is at 1e-6 and the sharp check is against exactly rounded
    statistics (math.fsum).  A double near 1e6 has a spacing of 1.2e-10 = 1.2e-7 sigma here, and every merge of two
    partial means rounds to it once: a mean a few spacings from the exactly rounded one moves the clamped values
    (1 + |z|) by that many times 1e-7, which is what the bar of 5e-7 allows - a variance from sums of squares would
    be wrong in the first digit."""
    import math
    g = 1.0e6 + seeded.normal(52, 1, (200, 300), 1e-3)
    m = Matrix.from_numpy(g)
    GradientClipper(NeuralNetworkParameters()).Clip([layer_of([m], [m])])
    got = m.to_numpy()
    assert rel_err(got, oracle.clip(g, 4.0, 1e-16)) <= 1e-6
    mean = math.fsum(g.reshape(-1)) / g.size
    std = math.sqrt(math.fsum(((g - mean) ** 2).reshape(-1)) / g.size)
    lim = np.minimum(4.0, 1 + np.abs((g - mean) / std))
    assert rel_err(got, np.clip(g, -lim, lim)) <= 5e-7


@pytest.mark.parametrize("dtype", DTYPES)
def test_clip_deep_matrix_uses_joint_statistics(gpu, oracle, dtype):
    params = NeuralNetworkParameters(lite=dtype == np.float32)
    g = seeded.normal(53, 1, (4, 30, 20), 1.0, dtype)
    g[2, 3, 4] = 60.0
    deep = DeepMatrix.from_numpy(g)
    GradientClipper(params).Clip([layer_of([deep], [deep])])
    ref = oracle.clip(g.reshape(1, -1), params.ClipValue, params.MinimumClipValue).reshape(g.shape)
    assert_parity(deep.to_numpy(), ref, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_adam_matches_oracle_over_steps(gpu, oracle, dtype):
    params = NeuralNetworkParameters(lite=dtype == np.float32)
    shapes = [(784, 256), (1, 256), (256, 128), (128, 10), (1, 1), (7, 4099)]
    ws = [seeded.xavier(61, i, *s).astype(dtype) for i, s in enumerate(shapes)]
    gs = [seeded.normal(62, i, s, 1.0, dtype) for i, s in enumerate(shapes)]
    wm = [Matrix.from_numpy(w) for w in ws]
    gm = [Matrix.from_numpy(g) for g in gs]
    layer = layer_of(wm, gm)
    ref = [(w.copy(), np.zeros_like(w), np.zeros_like(w)) for w in ws]
    for step in (1, 2, 3):
        params.AdamIteration = float(step)
        AdamOptimizer(params).Optimize([layer])
        ref = [oracle.adam(w, m, v, g, params.LearningRate, params.AdamBeta1, params.AdamBeta2, params.AdamEpsilon, float(step))
               for (w, m, v), g in zip(ref, gs)]
    for i, (w, m, v) in enumerate(ref):
        name = "W%d" % i
        if dtype == np.float64:
            # same operations in the same order, unfused: bit exact
            assert np.array_equal(layer[name, "Weight"].to_numpy(), w)
            assert np.array_equal(layer[name, "FirstMoment"].to_numpy(), m)
            assert np.array_equal(layer[name, "SecondMoment"].to_numpy(), v)
        else:
            assert_parity(layer[name, "Weight"].to_numpy(), w, dtype)
            assert_parity(layer[name, "FirstMoment"].to_numpy(), m, dtype)
            assert_parity(layer[name, "SecondMoment"].to_numpy(), v, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_adam_revert_matches_oracle_and_undoes_the_step(gpu, oracle, dtype):
    """AdamOptimizer.Revert (src/RMAD/AdamOptimizer.cs:97-193) on the device: the same numbers as the oracle's
    restatement of ReverseAdamUpdate, and, as its algebra promises, the weights and moments of the step before
    (to rounding: the moments are divided by beta again, which amplifies their last bits by 1/beta)."""
    params = NeuralNetworkParameters(lite=dtype == np.float32)
    shapes = [(784, 256), (1, 256), (128, 10), (1, 1), (7, 4099)]
    ws = [seeded.xavier(63, i, *s).astype(dtype) for i, s in enumerate(shapes)]
    gs = [seeded.normal(64, i, s, 1.0, dtype) for i, s in enumerate(shapes)]
    wm = [Matrix.from_numpy(w) for w in ws]
    gm = [Matrix.from_numpy(g) for g in gs]
    layer = layer_of(wm, gm)
    opt = AdamOptimizer(params)
    ref = [(w.copy(), np.zeros_like(w), np.zeros_like(w)) for w in ws]
    before = None
    for step in (1, 2, 3):
        before = ref
        params.AdamIteration = float(step)
        opt.Optimize([layer])
        ref = [oracle.adam(w, m, v, g, params.LearningRate, params.AdamBeta1, params.AdamBeta2, params.AdamEpsilon, float(step))
               for (w, m, v), g in zip(ref, gs)]
    opt.Revert([layer])  # AdamIteration is still 3: the iteration of the update being undone
    undone = [oracle.adam(w, m, v, g, params.LearningRate, params.AdamBeta1, params.AdamBeta2, params.AdamEpsilon, 3.0, reverse=True)
              for (w, m, v), g in zip(ref, gs)]
    for i, ((w, m, v), (w2, m2, v2)) in enumerate(zip(undone, before)):
        name = "W%d" % i
        got = [layer[name, kind].to_numpy() for kind in ("Weight", "FirstMoment", "SecondMoment")]
        for a, b in zip(got, (w, m, v)):
            if dtype == np.float64:
                assert np.array_equal(a, b)
            else:
                assert_parity(a, b, dtype)
        tol = 1e-9 if dtype == np.float64 else 2e-3
        for a, b in zip(got, (w2, m2, v2)):
            assert rel_err(a, b) <= tol


def test_many_tensors_cross_the_table_limit(gpu, oracle):
    """More tensors than one launch's descriptor table holds."""
    params = NeuralNetworkParameters()
    n = 97
    gs = [seeded.normal(71, i, (3 + i % 5, 50 + i), 1.0) for i in range(n)]
    ws = [seeded.uniform(72, i, g.shape, -1, 1) for i, g in enumerate(gs)]
    gm = [Matrix.from_numpy(g) for g in gs]
    wm = [Matrix.from_numpy(w) for w in ws]
    layer = layer_of(wm, gm)
    GradientClipper(params).Clip([layer])
    AdamOptimizer(params).Optimize([layer])
    for i in range(n):
        cg = oracle.clip(gs[i], 4.0, 1e-16)
        assert_parity(gm[i].to_numpy(), cg, np.float64)
        w, _, _ = oracle.adam(ws[i], np.zeros_like(ws[i]), np.zeros_like(ws[i]), gm[i].to_numpy(), 1e-3, 0.9, 0.999, 1e-8, 1.0)
        assert_parity(wm[i].to_numpy(), w, np.float64)


@pytest.mark.parametrize("dtype", DTYPES)
def test_fused_clip_adam_equals_clip_then_adam(gpu, oracle, dtype):
    """prad_clip_adam_multi must leave exactly what prad_clip_multi followed by prad_adam_multi leaves, for
    tensors whose chunk statistics are merged inside the clamping pass (few chunks) and for a tensor large
    enough to take the separate finalize launch; the small ones are also checked against the oracle."""
    from parallelreverseautodiff_amd import _lib
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    from parallelreverseautodiff_amd.operations import handle_array
    lib = _lib.load()
    for shapes in ([(784, 256), (1, 256), (1, 1), (3, 5000), (128, 10)], [(1100, 1024), (7, 3)]):   # 1100*1024 -> 275 chunks
        host = {k: [] for k in "wmvg"}
        dev = {tag: {k: [] for k in "wmvg"} for tag in ("two", "one")}
        for i, s in enumerate(shapes):
            host["w"].append(seeded.normal(61, 4 * i, s, 1.0, dtype))
            host["m"].append(seeded.normal(61, 4 * i + 1, s, 0.1, dtype))
            host["v"].append(np.abs(seeded.normal(61, 4 * i + 2, s, 0.1, dtype)))
            g = seeded.normal(61, 4 * i + 3, s, 0.5, dtype)
            if g.size > 100:
                g.reshape(-1)[5] = 90.0
                g.reshape(-1)[9] = 1e-20
            host["g"].append(g)
            for tag in dev:
                for k in "wmvg":
                    b = DeviceBuffer.alloc(dtype, *s)
                    b.upload(host[k][i])
                    dev[tag][k].append(b)
        n = len(shapes)
        arr = lambda tag, k: handle_array(dev[tag][k])
        args = (4.0, 1e-16 if dtype == np.float64 else 1e-8, 1e-3, 0.9, 0.999, 1e-8, 3.0)
        check(lib.prad_clip_multi(arr("two", "g"), n, args[0], args[1]))
        check(lib.prad_adam_multi(arr("two", "w"), arr("two", "m"), arr("two", "v"), arr("two", "g"), n, *args[2:]))
        check(lib.prad_clip_adam_multi(arr("one", "w"), arr("one", "m"), arr("one", "v"), arr("one", "g"), n, *args))
        for k in "wmvg":
            for i in range(n):
                assert np.array_equal(dev["two"][k][i].download(), dev["one"][k][i].download()), (k, shapes[i])
        if shapes[0] == (784, 256):
            for i in range(n):
                g = oracle.clip(host["g"][i], args[0], args[1])
                assert_parity(dev["one"]["g"][i].download(), g, dtype, "clamped gradient")
                w, m, v = oracle.adam(host["w"][i], host["m"][i], host["v"][i], dev["one"]["g"][i].download(), *args[2:])
                assert_parity(dev["one"]["w"][i].download(), w, dtype, "weight")
                assert_parity(dev["one"]["m"][i].download(), m, dtype, "first moment")
                assert_parity(dev["one"]["v"][i].download(), v, dtype, "second moment")


@pytest.mark.parametrize("dtype", DTYPES)
def test_device_resident_state_survives_a_checkpoint(gpu, tmp_path, dtype):
    """Weights and moments that live on the device are written in the reference's JSON layout
    (ModelLayer.SaveWeightsAndMoments), loaded into a fresh layer and trained on: both layers stay bit-identical."""
    params = NeuralNetworkParameters(lite=dtype == np.float32)
    shapes = [(33, 17), (1, 17), (5, 4099)]
    grads = [seeded.normal(72, i, s, 1.0, dtype) for i, s in enumerate(shapes)]
    a = layer_of([Matrix.from_numpy(seeded.xavier(71, i, *s).astype(dtype)) for i, s in enumerate(shapes)],
                 [Matrix.from_numpy(g) for g in grads])
    for step in (1, 2):
        params.AdamIteration = float(step)
        AdamOptimizer(params).Optimize([a])                  # state now device-resident
    path = str(tmp_path / "state.json")
    a.SaveWeightsAndMoments(path)
    b = layer_of([Matrix(*s, dtype) for s in shapes], [Matrix.from_numpy(g) for g in grads])
    b.LoadWeightsAndMoments(path)
    params.AdamIteration = 3.0
    AdamOptimizer(params).Optimize([a])
    AdamOptimizer(params).Optimize([b])
    for i in range(len(shapes)):
        for element in ("Weight", "FirstMoment", "SecondMoment"):
            assert np.array_equal(a["W%d" % i, element].to_numpy(), b["W%d" % i, element].to_numpy()), (i, element)


def test_gradient_clearer_zeroes_every_gradient_in_one_call(gpu):
    """GradientClearer.Clear (src/RMAD/GradientClearer.cs:21-86): device-resident gradients of both element types, of odd
    sizes (a 16-byte vector does not divide them), more of them than one launch's table holds, and a host-only one; the
    buffers next to them keep their values."""
    from parallelreverseautodiff_amd.optim import GradientClearer
    shapes = [(1, 1), (3, 5), (1, 10), (7, 9), (128, 10), (255, 33), (64, 4097)] * 7   # 49 tensors: two tables
    mats, guards = [], []
    for i, s in enumerate(shapes):
        dtype = np.float64 if i % 2 else np.float32
        m = Matrix.from_numpy(seeded.normal(61, i, s, 1.0, dtype))
        m.device()                                                       # the gradient lives on the device
        g = Matrix.from_numpy(seeded.normal(62, i, s, 1.0, dtype))
        g.device()
        mats.append(m)
        guards.append((g, g.to_numpy().copy()))
    host_only = Matrix.from_numpy(np.ones((4, 6)))
    GradientClearer().Clear([layer_of(mats + [host_only], mats + [host_only])])
    # a view whose first element is not on a 16-byte boundary (rows 1.. of a 3-column double matrix), straight through the C ABI
    import ctypes
    from parallelreverseautodiff_amd import _lib
    from parallelreverseautodiff_amd.exceptions import check
    from parallelreverseautodiff_amd.matrix import DeviceBuffer
    whole = DeviceBuffer.alloc(np.float64, 5, 3)
    whole.upload(np.arange(15.0).reshape(5, 3) + 1)
    part = whole.view_rows(1, 3)
    check(_lib.load().prad_zero_multi((ctypes.c_void_p * 2)(part.handle.value, mats[0].device().handle.value), 2))
    assert np.array_equal(whole.download(), np.array([[1, 2, 3], [0, 0, 0], [0, 0, 0], [0, 0, 0], [13, 14, 15]], dtype=np.float64))
    for m, s in zip(mats, shapes):
        got = m.to_numpy()
        assert got.shape == s and not got.any()
    assert not host_only.to_numpy().any()
    for g, ref in guards:
        assert np.array_equal(g.to_numpy(), ref)
