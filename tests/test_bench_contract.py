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


def test_the_line_is_cut_to_its_limit_by_dropping_the_least_important_figures():
    sys.path.insert(0, ROOT)
    try:
        import bench
    finally:
        sys.path.remove(ROOT)
    contract = {"metric": "m" * 70, "value": 1.0, "config": {"workload": "w" * 150}, "roofline": {"frac": 0.5},
                "cpu_baseline": {"value": 0.2}}
    also = {f"figure_{i}": [0.123, 0.456] for i in range(60)}
    full = dict(contract, also=also, extra_file="../" * 20 + "extra.json")
    line = bench.fit_line(full)
    assert len(line) <= bench.LINE_LIMIT < 1500
    r = json.loads(line)
    assert all(r[k] == v for k, v in contract.items())          # the contract's keys are untouched
    kept = list(r["also"])
    assert kept and kept == list(also)[:len(kept)]               # dropped from the end only
    assert r["extra_file"] == "extra.json"
    short = dict(contract, also={"a": 1}, extra_file="gpurun_out/bench_extra.json")
    assert json.loads(bench.fit_line(short)) == short            # a line that fits is left alone


def _check_line(r, steps, warmup):
    assert r["n_gpus"] == 1 and r["steps"] == steps and r["warmup"] == warmup
    assert r["unit"] == "GB/s" and r["higher_is_better"] is True and r["vs_baseline"] is None
    assert r["data"] == "synthetic" and r["dtype"] == "fp32" and "workload" in r["config"]
    assert abs(r["value"] - r["config"]["bytes_in"] / (r["ms_per_step"] * 1e-3) / 1e9) < 0.01 * r["value"]
    rf = r["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3
    assert abs(rf["achieved"] - rf["algorithmic_bytes_per_launch"] / (rf["avg_launch_ms"] * 1e-3) / 1e9) < 0.01 * rf["achieved"]
    assert 0.9 < rf["traffic"] / rf["algorithmic_bytes_per_launch"] < 1.1
    # one kernel cannot take longer than the step that contains it
    assert rf["avg_launch_ms"] < r["ms_per_step"]
    cb = r["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] == 1 and cb["unit"] == "GB/s" and cb["value"] > 0 and cb["sample"]


@pytest.mark.gpu
def test_json_line_on_the_gpu(tmp_path):
    out = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "2", "--no-extra",
                          "--extra-file", str(tmp_path / "extra.json")],
                         capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and len(lines[0]) < 1500
    _check_line(json.loads(lines[0]), 5, 2)


@pytest.mark.gpu
def test_the_drivers_command_prints_a_short_last_line(tmp_path):
    """`python bench.py --gpus 1 --steps 20 --warmup 5`, everything switched on: the
    last line of stdout is one JSON object short enough for a 2000-character tail,
    and the rest of the figures are in the file it names."""
    extra = tmp_path / "extra.json"
    out = subprocess.run([sys.executable, BENCH, "--gpus", "1", "--steps", "20", "--warmup", "5",
                          "--extra-file", str(extra)], capture_output=True, text=True, timeout=900)
    assert out.returncode == 0, out.stderr[-2000:]
    last = [l for l in out.stdout.splitlines() if l.strip()][-1]
    assert len(last) < 1500, len(last)
    r = json.loads(last)
    _check_line(r, 20, 5)
    assert "extra" not in r and r["also"]
    def numbers(v):
        if isinstance(v, dict):
            v = list(v.values())
        return [x for item in v for x in numbers(item)] if isinstance(v, list) else [v]

    assert all(x > 0 for x in numbers(r["also"]))
    # the small-field, cold-cache and swap figures are the first to be kept when the line is cut
    assert {"zfp_r8_c1_16MB", "cold", "swap_c4_ms"} <= set(r["also"])
    assert len(r["also"]["cold"]["attn402MB"]) == 2 and r["also"]["swap_c4_ms"]["worst_vs_raw"] > 0
    full = json.loads(extra.read_text())
    assert full["also"]["box_copy_GBs"] > 1000               # what a plain device copy reaches on this box
    assert len(full["also"]["zvc_256MiB_cpu_GBs"]) == 2      # the CPU sparse path beside the ZVC figures
    assert set(r["also"]) <= set(full["also"])               # what the line dropped is still in the file
    assert full["value"] == r["value"] and "zvc_relu_512MiB" in full["extra"] and "swap" in full["extra"]
    assert full["extra"]["zvc_relu_256MiB"]["cpu_baseline"]["all_cores"]["cores"] >= 1
