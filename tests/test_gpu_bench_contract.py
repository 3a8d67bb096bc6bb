"""bench.py's output line: the fields the driver reads, on the small functional workload."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + list(args), capture_output=True, text=True,
                       timeout=280)
    return r.returncode, r.stdout, r.stderr


def test_bench_line_on_the_small_workload():
    rc, out, err = _run("--workload", "tiny-q4ks", "--steps", "16", "--warmup", "4", "--repeats", "1", "--cpu-seconds", "1")
    assert rc == 0, err[-2000:]
    lines = [l for l in out.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 16 and d["warmup"] == 4 and d["higher_is_better"] is True
    assert d["unit"] == "tok/s" and d["value"] > 0 and d["vs_baseline"] is None and d["data"] == "synthetic"
    assert abs(d["value"] * d["ms_per_step"] - 1000.0) < 1.0  # tokens per second and milliseconds per token agree
    assert d["config"]["workload"] == "tiny-q4ks" and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["value"] > 0 and c["cores"] >= 1 and c["sample"]


def test_bench_refuses_more_than_one_gpu():
    rc, out, err = _run("--gpus", "2")
    assert rc != 0 and "gpu" in (out + err).lower()
