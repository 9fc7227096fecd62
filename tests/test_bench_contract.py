"""bench.py's command-line contract, checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2")
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and "--gpus 2" in r.stderr
    assert r.stdout.strip() == ""  # no JSON line for a run that did not happen


def test_help_names_the_workloads():
    r = run("--help")
    assert r.returncode == 0
    for word in ("--steps", "--warmup", "--gpus", "decode", "gemv", "prefill", "--max-seq", "--model", "qwen3-0.6b",
                 "llama2-7b-bf16"):
        assert word in r.stdout


def test_prompt_pass_report_counts_the_flops_of_the_shape():
    sys.path.insert(0, ROOT)
    import bench
    cfg = dict(hidden_size=8, intermediate_size=16, vocab_size=32, num_hidden_layers=2, num_attention_heads=2,
               num_key_value_heads=1)
    rep = bench.prefill_report(cfg, 10, 1.0)
    per_layer = 2 * 4 * 8 + 2 * 1 * 4 * 8 + 8 * 2 * 4 + 3 * 8 * 16  # q, k|v, o, gate|up|down
    assert rep["gemm_flops"] == 2.0 * 10 * 2 * per_layer + 2.0 * 32 * 8  # + lm_head on the last row
    assert rep["attention_flops"] == 4.0 * 2 * 2 * 4 * 10 * 10 / 2.0
    assert rep["tokens_per_s"] == 10000.0
