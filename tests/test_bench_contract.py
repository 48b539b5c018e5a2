"""bench.py's contract: the parts that need no GPU, and its JSON line on a small batch."""
import os
import subprocess
import sys

import pytest

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
    for flag in ("--gpus", "--steps", "--warmup", "--config", "--no-e2e", "--no-extra-legs",
                 "--pipeline-switches"):
        assert flag in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [["--config", "4", "--pool-slices", "2"], ["--config", "2"],
                                   ["--config", "3"], ["--config", "2", "--place-tries", "2"],
                                   ["--config", "2", "--pipeline-switches", "scripts"]])
def test_bench_line_on_a_small_batch(extra):
    """One JSON line with the contract's keys, on a batch small enough for a test."""
    import json
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--batch", "4", "--steps", "2",
                        "--warmup", "1", "--no-e2e", "--cpu-sample", "2", *extra],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline",
                "cpu_baseline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 2 and out["value"] > 0
    roof = out["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert out["cpu_baseline"]["kind"] == "port" and out["cpu_baseline"]["value"] > 0
    assert "traffic" in roof and "traffic_source" in roof
    if "--place-tries" in extra:   # separate pools picked by the probe: an extra report
        assert out["placement"]["slabs"] == 2 and "separate allocations" in roof["pools"]
        first = roof["first_two_allocations"]
        assert abs(first["frac"] - first["achieved"] / roof["peak"]) < 1e-3
    else:                          # the default: one cache allocation, as the engine makes it
        assert "placement" not in out and "one cache allocation" in roof["pools"]
    if extra[:2] == ["--config", "4"]:
        assert out["config"]["layers"] == 36 and "36 layers" in out["unit"]
        assert len(roof["avg_launch_us_by_layer_slice"]) == 2
    assert "workload" in out["config"] and "model" not in out["config"]
