"""bench.py's command-line contract, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                         text=True, timeout=120)
    assert res.returncode == 2
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


def test_help_lists_the_workloads():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True,
                         timeout=120)
    assert res.returncode == 0
    for name in ("llama2_7b_layer_batch1", "llama3_8b_layer_batches", "llama2_7b_dequant_full_model",
                 "llama2_7b_decode", "llama2_7b_prefill", "--steps", "--warmup"):
        assert name in res.stdout
