"""The contract's JSON line of bench.py stays short enough for a log tail to hold it whole."""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402


def _records():
    head = {
        "n": 128,
        "workload": "c4_k3_f16_128_28: quaternion conv 3x3 stride 1, N=128 (4N=512 rows), 128->128 q-channels, 28x28, "
                    "fwd+input-grad+filter-grad",
        "product_mode": 16, "fp16_policy": "backward32", "padding": "VALID", "dtype": "f16",
        "value": 1174.23487234, "unit": "TFLOP/s", "ms_per_step": 1.2103498734,
        "kernel_ms": {"fwd": 0.1, "bwd_data": 0.2, "bwd_weights": 0.3}, "hip_graph": {"used": True, "note": "x" * 300},
        "roofline": {"bound": "mfma", "pass": "bwd_weights",
                     "kernel": "qconv_wgrad_f16mfma_p16_f16_ch64x64_taps3_sw1_flat_z21_and_more",
                     "kernel_ms": 0.39923487, "achieved": 1187.2348, "peak": 2500.0, "unit": "TFLOP/s", "frac": 0.4748234,
                     "executed_frac": 0.474234, "algorithmic_bytes": 206045184, "traffic": 407312345.0,
                     "regime": "issue/latency", "arithmetic_intensity": 2291.123, "ridge": 312.5},
        "cpu_baseline": {"value": 4.9623487, "unit": "TFLOP/s", "cores": 16,
                         "cpu_model": "Some Vendor Model 9575F 64-Core Processor with a long marketing name",
                         "kind": "port", "ms_per_step_sample": 572.2348,
                         "sample": "16/128 images, fwd+bwd, factorized path, torch 2.10.0+rocm7.0 CPU (oneDNN) convs, "
                                   "fp32, median of 50"},
    }
    short = {}
    for name in list(bench.CONVS) + list(bench.DENSE):
        for pol in (("fp32",) if name.endswith("f32") else ("full16", "backward32")):
            for m in (8, 16):
                short.setdefault(name, {}).setdefault(pol, {})[str(m)] = bench.sig(
                    [0.012345678, 0.0026623456] if name in bench.DENSE else [1.2345678, 1174.56], 3)
    extra = {"c5": {"images_per_s": 7287.2348, "ms_per_step": 8.782348, "images_per_s_other_mode": 7246.234},
             "per_config": short, "stale_profiles": 12}
    return head, extra


def test_contract_line_is_short_and_complete():
    head, extra = _records()
    text = bench.line(head, argparse.Namespace(steps=20, warmup=5), extra)
    assert "\n" not in text and len(text) <= bench.LINE_LIMIT
    out = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "c5", "per_config"):
        assert key in out
    assert out["config"]["workload"].startswith("c4_k3_f16_128_28")
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in out["roofline"]
    for key in ("value", "unit", "cores", "kind", "sample", "cpu_model"):
        assert key in out["cpu_baseline"]
    assert isinstance(out["per_config"], dict) and len(out["per_config"]) == len(bench.CONVS) + len(bench.DENSE)
    assert out["per_config"]["c4_pw_f16_128_28"]["backward32"]["16"] == [1.23, 1170]
    assert out["per_config"]["c1_dense_f32"]["fp32"]["8"] == [0.0123, 0.00266]


def test_an_oversized_table_is_dropped_rather_than_the_headline():
    head, extra = _records()
    extra["per_config"] = {("w%d" % i): {"p": {"8": [1.0, 2.0]}} for i in range(400)}
    text = bench.line(head, argparse.Namespace(steps=20, warmup=5), extra)
    assert len(text) <= bench.LINE_LIMIT and isinstance(json.loads(text)["per_config"], str)


def test_significant_digits():
    assert bench.sig(1174.2348) == 1174 and bench.sig(0.39923487) == 0.3992 and bench.sig(206045184) == 206045184
    assert bench.sig(float("nan")) is None and bench.sig({"a": [1.23456, "s"]}) == {"a": [1.235, "s"]}


def test_more_than_one_gpu_is_refused(capsys, monkeypatch):
    monkeypatch.setattr(sys, "argv", ["bench.py", "--gpus", "2"])
    assert bench.main() == 2
    assert "one GPU" in capsys.readouterr().err


def test_channels_last_needs_one_convolution_workload(capsys, monkeypatch):
    monkeypatch.setattr(sys, "argv", ["bench.py", "--channels-last"])
    assert bench.main() == 2
    assert "--workload" in capsys.readouterr().err
