"""Writes tests/golden/golden.json: expected outputs of the CPU oracle on seeded inputs.

The reference ships no golden vectors for this path and cannot run here (C#, no .NET runtime),
so these fixtures come from the oracle after tests/test_oracle.py has pinned it.  They freeze the
oracle (a later edit that changes any result fails tests/test_golden.py) and give the GPU tests
fixed expected values.  Inputs are not stored: they are regenerated from (seed, tensor id, shape)
by parallelreverseautodiff_amd/seeded.py.  Outputs are stored exactly, as the hex form of every
element for small cases and as a SHA-256 of the raw bytes plus a few probe elements for larger
ones.

Run from the repository root:  python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle  # noqa: E402
from parallelreverseautodiff_amd import seeded  # noqa: E402

SEED = seeded.DEFAULT_SEED

MATMUL_CASES = [  # name, dtype, M, K, N
    ("tiny_f64", "float64", 4, 6, 3),
    ("ragged_f64", "float64", 33, 70, 19),
    ("mlp_layer1_f64", "float64", 64, 784, 256),
    ("mlp_layer3_f64", "float64", 64, 128, 10),
    ("column_vector_f64", "float64", 100, 100, 1),
    ("square256_f64", "float64", 256, 256, 256),
    ("tiny_f32", "float32", 4, 6, 3),
    ("ragged_f32", "float32", 33, 70, 19),
    ("square256_f32", "float32", 256, 256, 256),
]


def matmul_inputs(dtype, M, K, N):
    A = seeded.uniform(SEED, 1, (M, K), -1.0, 1.0, dtype)
    B = seeded.uniform(SEED, 2, (K, N), -1.0, 1.0, dtype)
    dC = seeded.normal(SEED, 3, (M, N), 1.0, dtype)
    return A, B, dC


def elementwise_inputs(dtype, n=96):
    x = seeded.normal(SEED, 11, (n,), 1.5, dtype)
    dy = seeded.normal(SEED, 12, (n,), 1.0, dtype)
    return x, dy


def optim_inputs(dtype, rows=24, cols=17):
    g = seeded.normal(SEED, 21, (rows, cols), 1.0, dtype)
    g[2, 3] = 50.0
    g[5, 5] = 1e-20
    w = seeded.uniform(SEED, 22, (rows, cols), -1.0, 1.0, dtype)
    m = seeded.normal(SEED, 23, (rows, cols), 0.1, dtype)
    v = np.abs(seeded.normal(SEED, 24, (rows, cols), 0.01, dtype))
    return g, w, m, v


def adjacent_inputs(dtype, rows=7, cols=13):
    a = seeded.normal(SEED, 31, (rows, cols), 2.0, dtype)
    b = seeded.normal(SEED, 32, (rows, cols), 1.0, dtype)
    c = seeded.uniform(SEED, 33, (rows, cols), -3.0, 3.0, dtype)
    return a, b, c


def encode(a):
    a = np.ascontiguousarray(a)
    entry = {"shape": list(a.shape), "sha256": hashlib.sha256(a.tobytes()).hexdigest()}
    flat = a.reshape(-1)
    if flat.size <= 64:
        entry["hex"] = [float(v).hex() for v in flat]
    else:
        idx = [0, flat.size // 3, flat.size // 2, flat.size - 1]
        entry["probe"] = {str(i): float(flat[i]).hex() for i in idx}
    return entry


def main():
    out = {"seed": SEED, "matmul": {}, "elementwise": {}, "optim": {}, "adjacent": {}}
    for name, dt, M, K, N in MATMUL_CASES:
        dtype = np.dtype(dt)
        A, B, dC = matmul_inputs(dtype, M, K, N)
        C = oracle.matmul_fwd(A, B)
        dA, dB = oracle.matmul_bwd(dC, A, B)
        out["matmul"][name] = {"dtype": dt, "M": M, "K": K, "N": N, "C": encode(C), "dA": encode(dA), "dB": encode(dB)}
    for dt in ("float64", "float32"):
        dtype = np.dtype(dt)
        x, dy = elementwise_inputs(dtype)
        y_sig, y_tanh = oracle.sigmoid_fwd(x), oracle.tanh_fwd(x)
        # Only operations without exp/tanh/pow(x, 3) are hashed; the others depend on libm's last ulp
        # and are stored as values to compare within 4 ulp.
        out["elementwise"][dt] = {
            "leakyrelu_fwd": encode(oracle.leakyrelu_fwd(x, 0.01)),
            "leakyrelu_bwd": encode(oracle.leakyrelu_bwd(x, dy, 0.01)),
            "hadamard_bwd_da": encode(oracle.hadamard_bwd(x, dy, x)[0]),
            "sigmoid_bwd_of_y": encode(oracle.sigmoid_bwd(np.abs(x) / (1 + np.abs(x)), dy)),
            "values": {
                "sigmoid_fwd": [float(v).hex() for v in y_sig[:32]],
                "tanh_fwd": [float(v).hex() for v in y_tanh[:32]],
                "gelu_fwd": [float(v).hex() for v in oracle.gelu_fwd(x)[:32]],
                "gelu_bwd": [float(v).hex() for v in oracle.gelu_bwd(x, dy)[:32]],
            },
        }
        g, w, m, v = optim_inputs(dtype)
        minv = 1e-16 if dt == "float64" else 1e-8
        w1, m1, v1 = oracle.adam(w, m, v, g, 1e-3, 0.9, 0.999, 1e-8, 3.0)
        out["optim"][dt] = {"clip": encode(oracle.clip(g, 4.0, minv)), "adam_w": encode(w1), "adam_m": encode(m1),
                            "adam_v": encode(v1)}
    for dt in ("float64", "float32"):
        dtype = np.dtype(dt)
        a, b, c = adjacent_inputs(dtype)
        y, mean, std = oracle.layernorm_fwd(a)
        # sums, square roots and divisions only: exact fixtures; pow(b, -x) depends on libm: values within a few ulp
        out["adjacent"][dt] = {
            "add": encode(oracle.matrix_add(a, b)), "add_three": encode(oracle.matrix_add_three(a, b, c)),
            "transpose": encode(oracle.matrix_transpose(a)),
            "layernorm_y": encode(y), "layernorm_mean": encode(mean), "layernorm_std": encode(std),
            "layernorm_bwd": encode(oracle.layernorm_bwd(a, mean, std, b)),
            "values": {"amplified_sigmoid_fwd": [float(v).hex() for v in oracle.amplified_sigmoid_fwd(a).reshape(-1)[:32]],
                       "amplified_sigmoid_bwd": [float(v).hex() for v in oracle.amplified_sigmoid_bwd(a, b).reshape(-1)[:32]]},
        }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote", path)


if __name__ == "__main__":
    main()
