"""The bench.py command-line contract: one JSON line with the agreed keys; more than one GPU is refused."""

import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
	r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
	assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [[], ["--graph"]])
def test_one_json_line_with_roofline_and_baseline(extra):
	cmd = [sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "tiny", "--steps", "2", "--warmup", "1"] + extra
	r = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=ROOT)
	assert r.returncode == 0, r.stderr[-2000:]
	lines = [l for l in r.stdout.splitlines() if l.strip()]
	assert len(lines) == 1
	out = json.loads(lines[0])
	for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
		assert key in out, key
	assert out["n_gpus"] == 1 and out["steps"] == 2 and out["warmup"] == 1 and out["unit"] == "tokens/s" and out["vs_baseline"] is None
	assert out["value"] > 0 and out["ms_per_step"] > 0 and out["config"]["workload"] == "tiny" and out["config"]["hip_graph"] == bool(extra)
	roof = out["roofline"]
	assert roof["bound"] == "mfma" and roof["unit"] == "TFLOP/s" and roof["peak"] == 2500.0
	assert roof["achieved"] > 0 and roof["frac"] == pytest.approx(roof["achieved"] / roof["peak"]) and roof["launches"] > 0
	cpu = out["cpu_baseline"]
	assert cpu["kind"] == "port" and cpu["value"] > 0 and cpu["cores"] >= 1 and cpu["sample"]
