"""bench.py on a machine without a GPU: what can be checked of its command-line contract."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode != 0
    assert "one GPU" in run.stderr
    assert run.stdout.strip() == ""          # no JSON line for a run that did not happen


def test_help_lists_the_contract_flags():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in run.stdout
