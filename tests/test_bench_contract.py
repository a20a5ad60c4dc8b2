"""bench.py's command-line contract, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, cwd=ROOT,
                          timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_help_lists_the_workloads_of_every_benchmark_configuration():
    r = run("--help")
    assert r.returncode == 0
    for w in ("c1", "c2", "c2-ragged", "c2-paged", "c3", "c4", "c5-decode", "c5-prefill"):
        assert w in r.stdout


def test_without_a_gpu_nothing_is_measured_and_no_line_is_printed():
    import torch
    if torch.cuda.is_available():
        return  # this check is for machines without a GPU
    r = run("--steps", "1", "--warmup", "0")
    assert r.returncode != 0 and "GPU" in r.stderr and not r.stdout.strip().startswith("{")
