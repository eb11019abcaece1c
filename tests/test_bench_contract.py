"""bench.py's contract: more than one GPU is refused with a message before anything is imported; a run prints exactly
one JSON line with the agreed keys, a `roofline` object whose fraction is achieved / peak, and (unless switched off) a
`cpu_baseline` object."""

import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KEYS = {"metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype",
        "data", "config", "roofline"}


def _bench(*flags, timeout=600):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True, timeout=timeout, cwd=ROOT)


def test_more_than_one_gpu_is_refused():
    run = _bench("--gpus", "2", timeout=60)
    assert run.returncode != 0 and run.stdout.strip() == ""
    assert "ONE GPU" in run.stderr


def _one_line(run):
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [l for l in run.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, lines
    return json.loads(lines[0])


@pytest.mark.gpu
def test_headline_line_has_the_agreed_shape():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    print("[case] bench contract, headline", flush=True)
    line = _one_line(_bench("--steps", "3", "--warmup", "1", "--no-jagged", "--no-bwd"))
    assert KEYS <= set(line) and "cpu_baseline" in line
    assert line["n_gpus"] == 1 and line["steps"] == 3 and line["warmup"] == 1 and line["higher_is_better"] is True
    assert line["vs_baseline"] is None and line["data"] == "synthetic" and line["dtype"] == "bf16" and line["unit"] == "TFLOP/s"
    assert line["config"]["workload"] == "headline" and "model" not in line["config"]
    roof = line["roofline"]
    assert roof["bound"] == "mfma" and roof["peak"] == 2500.0 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert abs(roof["achieved"] - line["value"]) < 0.1
    # per-step HIP events: mean (what the line is computed from), median and spread, and how many steps
    assert roof["timed_steps"] == 3 and roof["kernel_ms_p10"] <= roof["kernel_ms_median"] <= roof["kernel_ms_p90"]
    assert roof["kernel_ms_p10"] <= roof["kernel_ms"] <= roof["kernel_ms_p90"] * 1.0001
    # the measured HBM traffic comes from the tracked table next to the profile summaries, never from a literal here
    table = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    assert roof["traffic"] == table["headline"]["bytes"] and roof["traffic_source"] == table["headline"]["profile"]
    assert os.path.exists(os.path.join(ROOT, roof["traffic_source"]))
    cpu = line["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["unit"] == "TFLOP/s" and cpu["sample"]


@pytest.mark.gpu
@pytest.mark.parametrize("workload,bound", [("cfg2", "hbm"), ("kvcat", "hbm"), ("normmul", "hbm"), ("bwd_cfg3", "mfma"), ("layer", "mfma")])
def test_other_workloads_print_one_line(workload, bound):
    import torch

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    print(f"[case] bench contract, {workload}", flush=True)
    line = _one_line(_bench("--workload", workload, "--steps", "3", "--warmup", "1", "--no-cpu"))
    assert KEYS <= set(line) and line["config"]["workload"] == workload and line["roofline"]["bound"] == bound
    assert 0.0 < line["roofline"]["frac"] < 1.0 and line["value"] > 0
    assert {"kernel_ms", "kernel_ms_median", "kernel_ms_p10", "kernel_ms_p90", "timed_steps", "traffic", "traffic_source"} <= set(line["roofline"])


def test_no_traffic_literal_in_bench_and_table_points_at_summaries():
    """`roofline.traffic` is read from profiles/traffic.json, which the command that writes a summary also writes."""
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert "MEASURED_TRAFFIC" not in src and "traffic.json" in src
    table = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    assert "headline" in table
    for key, entry in table.items():
        assert entry["bytes"] > 0 and os.path.exists(os.path.join(ROOT, entry["profile"])), key
