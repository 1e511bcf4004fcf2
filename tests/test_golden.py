"""The oracle must reproduce the committed golden fixtures exactly (tests/golden/golden.json,
written by tests/golden/make_golden.py)."""
import hashlib
import importlib.util
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "golden.json")) as f:
    GOLDEN = json.load(f)

_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
make_golden = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_golden)


def matches(array, entry):
    array = np.ascontiguousarray(array)
    assert list(array.shape) == entry["shape"]
    flat = array.reshape(-1)
    if "hex" in entry:
        assert [float(v).hex() for v in flat] == entry["hex"]
    else:
        for i, h in entry["probe"].items():
            assert float(flat[int(i)]).hex() == h
    assert hashlib.sha256(array.tobytes()).hexdigest() == entry["sha256"]


def decode_values(hexes, dtype):
    return np.array([float.fromhex(h) for h in hexes], dtype=dtype)


@pytest.mark.parametrize("name", sorted(GOLDEN["matmul"]))
def test_matmul_golden(oracle, name):
    case = GOLDEN["matmul"][name]
    dtype = np.dtype(case["dtype"])
    A, B, dC = make_golden.matmul_inputs(dtype, case["M"], case["K"], case["N"])
    matches(oracle.matmul_fwd(A, B, threads=3), case["C"])
    dA, dB = oracle.matmul_bwd(dC, A, B, threads=3)
    matches(dA, case["dA"])
    matches(dB, case["dB"])


@pytest.mark.parametrize("dt", ["float64", "float32"])
def test_elementwise_and_optim_golden(oracle, dt):
    dtype = np.dtype(dt)
    ew = GOLDEN["elementwise"][dt]
    x, dy = make_golden.elementwise_inputs(dtype)
    matches(oracle.leakyrelu_fwd(x, 0.01), ew["leakyrelu_fwd"])
    matches(oracle.leakyrelu_bwd(x, dy, 0.01), ew["leakyrelu_bwd"])
    matches(oracle.hadamard_bwd(x, dy, x)[0], ew["hadamard_bwd_da"])
    matches(oracle.sigmoid_bwd(np.abs(x) / (1 + np.abs(x)), dy), ew["sigmoid_bwd_of_y"])
    ulp = np.finfo(dtype).eps
    for key, fn in (("sigmoid_fwd", lambda: oracle.sigmoid_fwd(x)), ("tanh_fwd", lambda: oracle.tanh_fwd(x)),
                    ("gelu_fwd", lambda: oracle.gelu_fwd(x)), ("gelu_bwd", lambda: oracle.gelu_bwd(x, dy))):
        want = decode_values(ew["values"][key], dtype)
        assert np.allclose(fn()[:32], want, rtol=64 * ulp, atol=4 * ulp)
    g, w, m, v = make_golden.optim_inputs(dtype)
    op = GOLDEN["optim"][dt]
    matches(oracle.clip(g, 4.0, 1e-16 if dt == "float64" else 1e-8), op["clip"])
    w1, m1, v1 = oracle.adam(w, m, v, g, 1e-3, 0.9, 0.999, 1e-8, 3.0)
    matches(w1, op["adam_w"])
    matches(m1, op["adam_m"])
    matches(v1, op["adam_v"])


@pytest.mark.parametrize("dt", ["float64", "float32"])
def test_adjacent_operations_golden(oracle, dt):
    dtype = np.dtype(dt)
    gold = GOLDEN["adjacent"][dt]
    a, b, c = make_golden.adjacent_inputs(dtype)
    matches(oracle.matrix_add(a, b), gold["add"])
    matches(oracle.matrix_add_three(a, b, c), gold["add_three"])
    matches(oracle.matrix_transpose(a), gold["transpose"])
    y, mean, std = oracle.layernorm_fwd(a)
    matches(y, gold["layernorm_y"])
    matches(mean, gold["layernorm_mean"])
    matches(std, gold["layernorm_std"])
    matches(oracle.layernorm_bwd(a, mean, std, b), gold["layernorm_bwd"])
    ulp = np.finfo(dtype).eps
    for key, got in (("amplified_sigmoid_fwd", oracle.amplified_sigmoid_fwd(a)), ("amplified_sigmoid_bwd", oracle.amplified_sigmoid_bwd(a, b))):
        assert np.allclose(got.reshape(-1)[:32], decode_values(gold["values"][key], dtype), rtol=64 * ulp, atol=4 * ulp)
