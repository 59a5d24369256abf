"""The benchmark's command line and the one JSON line it prints."""
import json
import os
import subprocess
import sys

import pytest

from conftest import ROOT

BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 2
    assert "ONE GPU" in out.stderr and not out.stdout.strip()


def test_a_multi_rank_launch_is_refused_too():
    env = dict(os.environ, WORLD_SIZE="2", RANK="0", LOCAL_RANK="0")
    out = subprocess.run([sys.executable, BENCH], capture_output=True, text=True, timeout=120, env=env)
    assert out.returncode == 2 and "ONE GPU" in out.stderr


def test_defaults_are_one_gpu_and_a_run_of_minutes_at_most():
    out = subprocess.run([sys.executable, BENCH, "--help"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in out.stdout


@pytest.mark.gpu
def test_json_line_on_the_gpu():
    out = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "2", "--no-extra"],
                         capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    r = json.loads(lines[0])
    assert r["n_gpus"] == 1 and r["steps"] == 5 and r["warmup"] == 2
    assert r["unit"] == "GB/s" and r["higher_is_better"] is True and r["vs_baseline"] is None
    assert r["data"] == "synthetic" and r["dtype"] == "i32" and "workload" in r["config"]
    assert abs(r["value"] - r["config"]["bytes_in"] / (r["ms_per_step"] * 1e-3) / 1e9) < 0.01 * r["value"]
    rf = r["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3
    assert abs(rf["achieved"] - rf["algorithmic_bytes_per_launch"] / (rf["avg_launch_ms"] * 1e-3) / 1e9) < 0.01 * rf["achieved"]
    assert 0.9 < rf["traffic"] / rf["algorithmic_bytes_per_launch"] < 1.1
    cb = r["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] == 1 and cb["unit"] == "GB/s" and cb["value"] > 0 and cb["sample"]
