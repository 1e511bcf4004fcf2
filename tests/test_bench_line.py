"""bench.py's last line: the harness that runs the benchmark keeps the tail of stdout, so the line has to stay
compact whatever the other legs return, and carry the roofline and CPU baseline of the headline kernel."""
import argparse
import json

import bench


def _stub_legs():
    errors = {"against_reference_arithmetic": {"normwise": 1.234567e-15, "elementwise_floor_1e-3_rms": 2.345678e-13,
                                               "elementwise_floor_rms": 3.456789e-15}, "sampled_rows_per_output": 48}
    head = {"ms": 108.7654321, "wall_ms": 109.123456, "spot": 1.23456789e-16, "errors": errors,
            "isolated_launch_ms": {"NN C=A.B": 1.8123456, "NT dA=dC.B^T": 1.8234567, "TN dB=A^T.dC": 1.8345678}}
    cpu = {"value": 0.0123456789, "unit": "TFLOP/s", "cores": 16, "kind": "port", "n": 2048, "secs": 4.123456,
           "sample": "x" * 300}
    roof = lambda frac: {"bound": "mfma", "achieved": 100.123456, "peak": 157.3, "unit": "TFLOP/s", "frac": frac, "traffic": 123456789,
                         "kernel": "k" * 120}
    also = {"matmul_fwd_bwd_%s_n%d" % (d, n): {"TFLOPs": 1.0, "roofline": roof(0.5123456), "errors": errors}
            for d in ("f64", "f32") for n in (4096, 2048, 1024, 512)}
    for d in ("f64", "f32"):
        also["mlp_train_steps_per_s_" + d] = {"value": 17000.123456, "roofline": roof(0.0123), "cpu_baseline": {"steps_per_s": 53.21}}
        also["mlp_operation_walk_" + d] = {"value": 2100.123456, "roofline": roof(0.0023)}
        also["gradient_kernels_64Mi_" + d] = {k: {"ms": 0.5, "roofline": dict(roof(0.7123456), bound="hbm")}
                                              for k in ("leakyrelu_bwd", "sigmoid_bwd", "tanh_bwd", "gelu_bwd", "hadamard_bwd", "accumulate", "clip", "adam")}
    also["lstm_train_steps_per_s_f32"] = {"value": 907.123456, "roofline": roof(0.446)}
    also["swin_block_train_steps_per_s_f32"] = {"error": "RuntimeError('" + "y" * 500 + "')"}
    also["matmul_and_sum_f32"] = {"forward": {"ms": 0.1, "roofline": roof(0.757)}, "backward": {"ms": 0.02, "roofline": dict(roof(0.709), bound="hbm")}}
    table = [{"config": "c" * 80, "gpu_ms": 1.0} for _ in range(40)]
    return head, cpu, also, table


def test_last_line_is_compact_and_complete():
    args = argparse.Namespace(n=4096, steps=20, warmup=5, dtype="f64")
    head, cpu, also, table = _stub_legs()
    line, detail = bench.headline_lines(args, head, cpu, also, table)
    text = json.dumps(line, separators=(",", ":"))
    assert len(text) < bench.MAX_LINE_CHARS <= 1800, len(text)
    back = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in back, key
    assert back["metric"] == bench.METRIC and back["config"]["workload"].startswith("configs[1]")
    roof = back["roofline"]
    assert roof["bound"] == "mfma" and roof["peak"] == 78.6 and roof["unit"] == "TFLOP/s"
    # three launches of 2 N^3 flop per step: achieved follows from the step time, frac from achieved
    assert abs(roof["achieved"] - 2 * 4096.0 ** 3 / (head["ms"] / 60 * 1e-3) / 1e12) < 1e-2
    assert abs(roof["frac"] - roof["achieved"] / 78.6) < 1e-3
    assert abs(back["value"] - 3 * roof["achieved"] / 3) < 1e-2
    assert roof["launch_ms_isolated"] > 0 and 0 < roof["frac_isolated"] < 1
    assert roof["traffic"] is None or roof["traffic"] > 0
    assert back["cpu_baseline"]["value"] > 0 and back["cpu_baseline"]["cores"] == 16 and back["cpu_baseline"]["kind"] == "port"
    assert back["also"]["failed_legs"] == 1 or "failed_legs" not in back["also"]
    # nothing is lost: the detail object keeps the legs in full
    assert detail["also"] is also and detail["table"] is table and detail["headline"]["errors"] is head["errors"]


def test_last_line_without_the_other_legs():
    args = argparse.Namespace(n=1024, steps=3, warmup=1, dtype="f32")
    head, _, _, table = _stub_legs()
    head["errors"] = None
    line, detail = bench.headline_lines(args, head, None, None, table[:1])
    text = json.dumps(line, separators=(",", ":"))
    assert len(text) < bench.MAX_LINE_CHARS
    assert "cpu_baseline" not in line and "also" not in line and line["roofline"]["peak"] == 157.3
