"""bench.py on a machine without a GPU: the parts of its contract that need none."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode != 0
    assert "single-GPU" in r.stderr and r.stdout.strip() == ""


def test_help_lists_the_contract_flags():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--config", "--no-e2e", "--pipeline-switches"):
        assert flag in r.stdout
