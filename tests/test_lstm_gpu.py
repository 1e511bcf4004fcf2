"""LSTM layer step (fused 4-gate weight, BPTT, MSE) against the oracle's node-by-node composition of the
reference operations: MatrixMultiply on the concatenated [x_t | h_{t-1}], MatrixAddBroadcasting, Sigmoid, Tanh,
HadamardProduct, MatrixAdd, MeanSquaredError, and their Backward methods in reverse order."""
import numpy as np
import pytest

from conftest import assert_parity
from oracle import compose
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


def test_lstm_recorded_step_equals_eager(gpu):
    a, b = LSTMLayer(16, 32, 8, 6, dtype=np.float64), LSTMLayer(16, 32, 8, 6, dtype=np.float64)
    a.step(); b.step()
    b.record(adam_iteration=2.0)
    for _ in range(3):
        a.iteration = 1
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
    a, b = LSTMLayer(I, H, B, T, dtype=dtype, fused=True), LSTMLayer(I, H, B, T, dtype=dtype, fused=False)
    for step in range(2):
        a.step(); b.step()
        for name in ("G", "C", "Hs", "TC", "dG", "dX", "dW", "db", "W", "b", "loss"):
            assert np.array_equal(getattr(a, name).download(), getattr(b, name).download()), (name, step)
        assert np.array_equal(a.dh[1].download(), b.dh[1].download())
