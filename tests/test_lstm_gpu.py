"""LSTM layer step (fused 4-gate weight, BPTT, MSE) against the oracle's node-by-node composition of the
reference operations: MatrixMultiply on the concatenated [x_t | h_{t-1}], MatrixAddBroadcasting, Sigmoid, Tanh,
HadamardProduct, MatrixAdd, MeanSquaredError, and their Backward methods in reverse order."""
import os

import numpy as np
import pytest

from conftest import assert_long_sum_parity, assert_parity, norm_err, strict_err
from oracle import compose
from parallelreverseautodiff_amd import _lib
from parallelreverseautodiff_amd.exceptions import ArgumentException, InvalidOperationException
from parallelreverseautodiff_amd.lstm import LSTMLayer

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,cfg", [(np.float64, (16, 32, 8, 5)), (np.float32, (16, 32, 8, 5)), (np.float64, (48, 64, 32, 7)),
                                       (np.float32, (256, 512, 128, 4))])
def test_lstm_step_matches_node_by_node_oracle(gpu, oracle, dtype, cfg):
    I, H, B, T = cfg
    layer = LSTMLayer(I, H, B, T, dtype=dtype)
    layer.step(update=False)
    loss, Hout, dW, db, dX = compose.lstm_forward_backward(layer.host_W, np.zeros((1, 4 * H), dtype), layer.host_X, layer.host_Y, I, H, B, T)
    tol = 1e-12 if dtype == np.float64 else 1e-5
    assert abs(float(layer.loss.download()[0, 0]) - loss) <= tol * abs(loss)
    assert_parity(layer.H_out.download(), Hout, dtype, "hidden states")
    assert_parity(layer.dW.download(), dW, dtype, "dW")
    assert_parity(layer.db.download(), db, dtype, "db")
    assert_parity(layer.dX.download(), dX, dtype, "dX")


def test_lstm_benchmark_configuration_full_size(gpu, oracle):
    """The configuration the benchmark times, at its full size: input 256, hidden 512, batch 128, 64 time steps,
    float.  The node-by-node composition takes some seconds on the host cores.  The weight gradient is a sum over
    64 x 128 = 8192 rows (the reference adds 64 per-step products, the device runs one product): see
    assert_long_sum_parity."""
    I, H, B, T = 256, 512, 128, 64
    layer = LSTMLayer(I, H, B, T, dtype=np.float32)
    layer.step(update=False)
    zero_b = np.zeros((1, 4 * H), np.float32)
    loss, Hout, dW, db, dX = compose.lstm_forward_backward(layer.host_W, zero_b, layer.host_X, layer.host_Y, I, H, B, T, threads=16)
    assert abs(float(layer.loss.download()[0, 0]) - loss) <= 1e-5 * abs(loss)
    for what, got, ref in (("hidden states", layer.H_out, Hout), ("db", layer.db, db), ("dX", layer.dX, dX)):
        g = got.download()
        err = assert_parity(g, ref, np.float32, what)
        print("LSTM 256/512/128/64 float %s: relative %.2e, normwise %.2e, floor 1e-3 rms %.2e" % (what, err, norm_err(g, ref), strict_err(g, ref)))
    XH = np.concatenate([layer.host_X, layer.Hs.download()[:T * B]], axis=1)      # [X | H_prev] over all time steps
    errs = assert_long_sum_parity(layer.dW.download(), dW, XH, layer.dG.download(), np.float32, "dW")
    print("LSTM 256/512/128/64 float dW (K = 8192): against the reference %.2e; against the double product: device %.2e, "
          "reference arithmetic %.2e" % errs)


def test_long_sequence_on_the_sequence_kernels_matches_the_oracle(gpu, oracle):
    """The whole-sequence kernels evaluate the cell's sigmoids and tanhs in float on the hardware exponential (each within
    3e-7 of the rounded double value) and the difference feeds the recurrence: 512 time steps, four times the benchmark's
    count, on a small layer, against the oracle's node-by-node composition at the float bar."""
    I, H, B, T = 32, 64, 16, 512
    layer = LSTMLayer(I, H, B, T, dtype=np.float32, sequence=True)
    layer.step(update=False)
    zero_b = np.zeros((1, 4 * H), np.float32)
    loss, Hout, dW, db, dX = compose.lstm_forward_backward(layer.host_W, zero_b, layer.host_X, layer.host_Y, I, H, B, T)
    assert abs(float(layer.loss.download()[0, 0]) - loss) <= 1e-5 * abs(loss)
    for what, got, ref in (("hidden states", layer.H_out, Hout), ("db", layer.db, db), ("dX", layer.dX, dX)):
        err = assert_parity(got.download(), ref, np.float32, what)
        print("LSTM 32/64/16/512 float %s: relative %.2e" % (what, err))
    XH = np.concatenate([layer.host_X, layer.Hs.download()[:T * B]], axis=1)
    assert_long_sum_parity(layer.dW.download(), dW, XH, layer.dG.download(), np.float32, "dW")


def test_lstm_recorded_step_equals_eager(gpu):
    a, b = LSTMLayer(16, 32, 8, 6, dtype=np.float64), LSTMLayer(16, 32, 8, 6, dtype=np.float64)
    a.step(); b.step()
    b.record()                       # stands for step 2; every replay advances AdamIteration like step() does
    for _ in range(3):
        a.step()
        b.replay()
        gpu.Synchronize()
        for x, y in ((a.W, b.W), (a.b, b.b), (a.dW, b.dW), (a.mW, b.mW), (a.vW, b.vW), (a.loss, b.loss)):
            assert np.array_equal(x.download(), y.download())
    b.release()


@pytest.mark.parametrize("dtype,cfg", [(np.float64, (24, 64, 40, 5)), (np.float64, (16, 128, 32, 4)), (np.float32, (32, 128, 40, 5)),
                                       (np.float32, (256, 512, 128, 3)), (np.float32, (16, 32, 8, 4))])
def test_one_launch_per_time_step_equals_product_plus_cell_kernels(gpu, dtype, cfg):
    """The recurrent product with the cell arithmetic as its epilogue (forward: gate columns gathered per tile;
    backward: on the product split along K) gives the bits of the product followed by the cell kernel; row counts
    that do not fill the tiles and a hidden size that takes the two-launch path (32) included."""
    I, H, B, T = cfg
    a, b = LSTMLayer(I, H, B, T, dtype=dtype, fused=True, sequence=False), LSTMLayer(I, H, B, T, dtype=dtype, fused=False, sequence=False)
    for step in range(2):
        a.step(); b.step()
        for name in ("G", "C", "Hs", "TC", "dG", "dX", "dW", "db", "W", "b", "loss"):
            assert np.array_equal(getattr(a, name).download(), getattr(b, name).download()), (name, step)
        assert np.array_equal(a.dh[1].download(), b.dh[1].download())


@pytest.mark.parametrize("cfg", [(256, 512, 128, 5), (32, 64, 16, 6), (16, 256, 48, 4), (16, 128, 32, 1), (24, 448, 64, 3)])
def test_whole_sequence_in_one_launch_matches_one_launch_per_time_step(gpu, cfg):
    """The time loop inside one kernel each way (recurrent weight in registers, time steps ordered by flags between
    workgroups) against one launch per time step: the same arithmetic per element, another order of the sums along
    hidden (forward) and 4 * hidden (backward), so the float parity bar rather than bits.  One row group and several, a
    single time step, hidden sizes that fill the register slice fully (512) and partly."""
    I, H, B, T = cfg
    a, b = LSTMLayer(I, H, B, T, dtype=np.float32, sequence=True), LSTMLayer(I, H, B, T, dtype=np.float32, sequence=False)
    assert a.sequence and not b.sequence
    # gradients are compared before clipping (which is discontinuous at the minimum clip value)
    a.step(update=False); b.step(update=False)
    for name in ("G", "C", "Hs", "TC", "dG", "dX", "dW", "db"):
        assert_parity(getattr(a, name).download(), getattr(b, name).download(), np.float32, name)
    assert abs(float(a.loss.download()[0, 0]) - float(b.loss.download()[0, 0])) <= 1e-5 * abs(float(b.loss.download()[0, 0]))
    assert_parity(a.dh[1].download(), b.dh[1].download(), np.float32, "dh before the first step")


def test_whole_sequence_kernels_are_deterministic_and_replay(gpu):
    """Partial products are added in producer order, so two runs give the same bits, and so does a recorded step."""
    I, H, B, T = 64, 256, 64, 8
    a, b = LSTMLayer(I, H, B, T, dtype=np.float32, sequence=True), LSTMLayer(I, H, B, T, dtype=np.float32, sequence=True)
    a.step(); b.step()
    b.record()
    for _ in range(3):
        a.step()
        b.replay()
        gpu.Synchronize()
        for x, y in ((a.W, b.W), (a.dW, b.dW), (a.dG, b.dG), (a.Hs, b.Hs), (a.loss, b.loss)):
            assert np.array_equal(x.download(), y.download())
    b.release()


def test_whole_sequence_shapes_it_does_not_take(gpu):
    assert not LSTMLayer(16, 32, 8, 4, dtype=np.float32).sequence       # batch and hidden too small: per-step launches
    assert not LSTMLayer(16, 64, 16, 4, dtype=np.float64).sequence      # double: the weight slice does not fit the registers
    with pytest.raises(ArgumentException):
        LSTMLayer(16, 64, 24, 4, dtype=np.float32, sequence=True)       # batch not a multiple of 16
    layer = LSTMLayer(16, 64, 16, 4, dtype=np.float32, sequence=False)
    assert layer.lib.prad_lstm_sequence_fwd(layer.Wh.handle, layer.G.handle, layer.C.handle, layer.Hs.handle, layer.TC.handle, 3) != 0   # rows % steps


def _error_text(lib):
    return lib.prad_last_error().decode()


def test_whole_sequence_falls_back_when_the_device_does_not_hold_the_grid(gpu):
    """The first sequence call asks the device, with a roll-call kernel of the same grid and footprint, whether it holds
    the whole grid at once.  Forced to fail from the host (a negative poll limit makes the probe report failure without
    waiting for anybody; every kernel ends normally), the sequence kernels go off, the calls run one launch per time step instead and
    succeed, and the results are those of the per-step layer bit for bit."""
    shape = (64, 512, 128, 16)
    code = _lib.PRAD_F32
    lib = _lib.load()
    assert lib.prad_lstm_sequence_enable(1) == 0
    os.environ["PRAD_LSTM_SPIN_LIMIT"] = "-1"
    try:
        layer, ref = LSTMLayer(*shape, dtype=np.float32), LSTMLayer(*shape, dtype=np.float32, sequence=False)
        assert layer.sequence and not ref.sequence
        layer.step(); ref.step()
        gpu.Synchronize()                                               # no error: nothing partial was written
        assert "one launch per time step" in _error_text(lib)
        assert lib.prad_lstm_sequence_supported(code, shape[2], shape[1], shape[3]) == 0
    finally:
        del os.environ["PRAD_LSTM_SPIN_LIMIT"]
    for _ in range(2):
        layer.step(); ref.step()
    gpu.Synchronize()
    for x, y in ((layer.W, ref.W), (layer.dW, ref.dW), (layer.dG, ref.dG), (layer.Hs, ref.Hs), (layer.dX, ref.dX), (layer.loss, ref.loss)):
        assert np.array_equal(x.download(), y.download())
    assert lib.prad_lstm_sequence_enable(1) == 0
    assert lib.prad_lstm_sequence_supported(code, shape[2], shape[1], shape[3]) == 1


def test_whole_sequence_kernel_gives_up_instead_of_waiting_forever(gpu):
    """Every wait on a peer workgroup is bounded.  After a grid has been proven, a limit of one poll makes some workgroup
    give up at once inside the sequence kernels; all the others then leave at their next wait, the kernels end
    normally, the next wait for the stream reports it, and the sequence kernels stay off: the steps after that run
    per time step and are right.  Turning the kernels on again restores the one-launch path."""
    shape = (64, 512, 128, 16)
    lib = _lib.load()
    assert lib.prad_lstm_sequence_enable(1) == 0
    layer, ref = LSTMLayer(*shape, dtype=np.float32), LSTMLayer(*shape, dtype=np.float32, sequence=False)
    seq = LSTMLayer(*shape, dtype=np.float32)
    layer.step(update=False); seq.step(update=False)                   # proves the grid with the default limit
    gpu.Synchronize()
    os.environ["PRAD_LSTM_SPIN_LIMIT"] = "1"
    try:
        layer.step(update=False)
        with pytest.raises(InvalidOperationException, match="gave up waiting"):
            gpu.Synchronize()
    finally:
        del os.environ["PRAD_LSTM_SPIN_LIMIT"]
    assert lib.prad_lstm_sequence_supported(_lib.PRAD_F32, shape[2], shape[1], shape[3]) == 0
    layer.step(update=False); ref.step(update=False)                   # per time step inside the sequence calls
    gpu.Synchronize()
    assert np.array_equal(layer.dW.download(), ref.dW.download())
    assert np.array_equal(layer.Hs.download(), ref.Hs.download())
    assert lib.prad_lstm_sequence_enable(1) == 0
    layer.step(update=False); seq.step(update=False)                   # the one-launch path again, after a fresh probe
    gpu.Synchronize()
    assert np.array_equal(layer.dW.download(), seq.dW.download())


def test_sequence_calls_take_every_shape_and_element_type(gpu, oracle):
    """Shapes and element types the one-launch kernels do not take run per time step inside the same two calls."""
    for dtype, shape in ((np.float64, (16, 64, 16, 4)), (np.float32, (16, 32, 8, 5))):
        a = LSTMLayer(*shape, dtype=dtype, sequence=False)
        b = LSTMLayer(*shape, dtype=dtype, sequence=False)
        b.sequence = True                                              # drive the sequence entry points anyway
        a.step(); b.step()
        gpu.Synchronize()
        for x, y in ((a.W, b.W), (a.dW, b.dW), (a.Hs, b.Hs), (a.dX, b.dX)):
            assert np.array_equal(x.download(), y.download())
