"""bench.py's command line, where no GPU is needed: more than one GPU is refused with a message, and the
GPU run's JSON line carries what the measurement contract names."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode != 0
    assert "one GPU" in done.stderr + done.stdout
    assert not [line for line in done.stdout.splitlines() if line.startswith("{")]


@pytest.mark.gpu
def test_small_workload_prints_one_contract_line():
    """The plumbing configuration (2 layers) through the whole bench path: one JSON line with the metric, the
    roofline of the dominant kernel measured live, and the CPU baseline beside it."""
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "c1", "--steps", "3", "--warmup", "1"],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [line for line in done.stdout.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    result = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in result, key
    assert result["n_gpus"] == 1 and result["steps"] == 3 and result["vs_baseline"] is None and result["higher_is_better"] is False
    assert "workload" in result["config"] and "model" not in result["config"]
    roof = result["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and roof["achieved"] > 0
    cpu = result["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
