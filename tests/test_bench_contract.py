"""bench.py without a GPU: what it says for more than one GPU, and its counts of bytes and operations at the
headline sizes against figures worked out by hand."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_more_than_one_gpu_is_one_line_and_exit_code_2():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1 and "--gpus 2" in r.stdout


def test_bytes_of_a_decode_step_at_the_headline_sizes():
    c = bench.SIZES["a27b"][0]
    # a layer without experts: q, k, v (with bias) and o 16.78 M, router and shared gate 0.12 M, shared expert 34.60 M,
    # two norms; an expert 8.65 M; embedding rows are not read, the vocabulary's matrix is: 311.2 M
    no_experts = bench.layer_weight_elems(c, 0.0)
    assert abs(no_experts - (16.78e6 + 0.125e6 + 34.60e6)) < 0.02e6
    assert abs(bench.layer_weight_elems(c, 1.0) - no_experts - 8.65e6) < 0.01e6
    # one token with 4 experts a layer and no context: 2 bytes * (24 layers + vocabulary) = 4.76 GB
    assert abs(bench.decode_bytes(c, 24, 1, 0, used=4.0) - 4.76e9) < 0.01e9
    # keys and values: 196,608 bytes per token and sequence
    per_token = bench.decode_bytes(c, 24, 1, 1, used=4.0) - bench.decode_bytes(c, 24, 1, 0, used=4.0)
    assert per_token == 196608
    # without a count, a batch reaches E (1 - (1 - k/E)^B) experts in expectation: 25.4 of 60 for 8 tokens
    exp8 = (bench.decode_bytes(c, 1, 8, 0) - bench.decode_bytes(c, 1, 8, 0, used=0.0)) / (2 * 8.65e6)
    assert abs(exp8 - 25.4) < 0.1


def test_operations_of_a_prompt_step_at_the_headline_sizes():
    c = bench.SIZES["a27b"][0]
    # 2,048 tokens through 24 layers: 8.47 TFLOP of products and 0.41 of attention, and one row of logits
    total = bench.prefill_flops(c, 24, 2048)
    assert abs(total - 8.87e12) < 0.03e12
    one_more_row = bench.prefill_flops(c, 24, 2048, rows_out=2) - total
    assert one_more_row == 2 * 2048 * 151936


import json  # noqa: E402

import pytest  # noqa: E402


@pytest.mark.gpu
def test_the_line_of_a_short_run_on_the_gpu():
    """One layer, a few steps: the line has the contract's keys, a flat configuration of at most 20 keys, and figures
    that fit each other (tokens a second and milliseconds a step; bytes a step, time and rate; a context that the
    timed steps really ended at, which bench.py checks against the cache and refuses to print otherwise)."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "1", "--steps", "6", "--warmup", "2",
                        "--batch", "3", "--context", "330", "--points-context", "330", "--no-points"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 6 and line["warmup"] == 2 and line["dtype"] == "bf16"
    cfg = line["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 1 and cfg["layers_of_full_model"] == 24 and cfg["global_batch"] == 3 and cfg["seq_len"] == 330
    assert abs(line["value"] - 3 / (line["ms_per_step"] * 1e-3)) < 0.01 * line["value"]
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    detail = line["points_detail"]["decode_b3_ctx330"]
    # the bytes of a step at the mean context of the timed steps: they find 324 .. 329 positions and read one more
    want = bench.decode_bytes(bench.SIZES["a27b"][0], 1, 3, (324 + 1 + 330) / 2.0, 2, cfg["experts_read_per_layer"]) / 1e9
    assert abs(detail["gb_per_step"] - want) < 0.01 * want
    assert abs(roof["achieved"] - detail["gb_per_step"] / (line["ms_per_step"] * 1e-3)) < 0.01 * roof["achieved"]
    pre = line["prefill"]
    assert pre["tokens"] == 2048 and abs(pre["value"] - 2048 / (pre["ms"] * 1e-3)) < 0.01 * pre["value"] and 0 < pre["frac"] < 1


@pytest.mark.gpu
def test_a_prompt_of_another_length_for_profiles():
    """--prefill-only --prefill-tokens N times a prompt step of N tokens alone and says how long the host was busy
    launching it (the default, and the contract's line, is 2,048 tokens)."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "1", "--prefill-only", "--prefill-tokens", "300"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert "300 tokens" in line["metric"] and line["layers"] == 1 and line["dtype"] == "bf16"
    assert abs(line["value"] - 300 / (line["ms"] * 1e-3)) < 0.01 * line["value"]
    assert 0 < line["host_ms"] <= line["ms"] * 1.01 and 0 < line["frac"] < 1


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_a_workload_of_unequal_prompts_on_the_gpu(dtype):
    """The record that the default run adds under "workloads" for each of the two other stated workloads, here with one
    layer, three prompts and four decode steps: the line's keys, a flat configuration, figures that fit each other."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "unequal", "--dtype", dtype, "--layers", "1",
                        "--batch", "3", "--prompt-min", "5", "--prompt-max", "300", "--decode-steps", "4"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "ms_per_step", "dtype", "config", "prefill", "roofline"):
        assert key in line, key
    cfg = line["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 1 and cfg["layers_of_full_model"] == 24 and cfg["global_batch"] == 3
    assert 15 <= cfg["prompt_tokens"] <= 900 and 5 <= cfg["shortest_prompt"] <= cfg["longest_prompt"] <= 300
    assert line["dtype"] == ("bf16" if dtype == "bfloat16" else "fp32") and line["steps"] == 4
    assert abs(line["value"] - 3 / (line["ms_per_step"] * 1e-3)) < 0.01 * line["value"]
    assert line["prefill"]["tokens"] == cfg["prompt_tokens"] and 0 < line["prefill"]["frac"] < 1
    assert 0 < line["roofline"]["frac"] < 1


def test_the_stated_workloads_of_unequal_prompts():
    assert bench.unequal_defaults("a14b") == {"batch": 8, "lo": 512, "hi": 4096, "steps": 256, "seed": 3}
    assert bench.unequal_defaults("a27b") == {"batch": 64, "lo": 1, "hi": 2048, "steps": 64, "seed": 4}
