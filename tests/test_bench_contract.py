"""CPU-only: the parts of bench.py's command-line contract that need no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    p = run_bench("--gpus", "2")
    assert p.returncode == 2
    assert "one GPU only" in p.stderr + p.stdout
    assert p.stdout.strip() == "" or not p.stdout.strip().startswith("{")  # no result line


def test_help_names_the_contract_flags():
    p = run_bench("--help")
    assert p.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--config", "--shape", "--no-cpu"):
        assert flag in p.stdout
