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
