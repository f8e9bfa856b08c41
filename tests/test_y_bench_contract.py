"""bench.py's contract with its driver: one GPU only (a larger --gpus, or a WORLD_SIZE above one, exits with a
message and no JSON line), a clear refusal without a GPU, and on a GPU one JSON line that carries the metric, the
workload, the roofline of the dominant kernel and (for the headline) the CPU baseline."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def run(args, env=None):
    e = dict(os.environ)
    e.update(env or {})
    return subprocess.run([sys.executable, BENCH] + args, capture_output=True, text=True, env=e, timeout=600)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run(["--gpus", "2"])
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
    r = run([], env={"WORLD_SIZE": "2"})
    assert r.returncode == 2 and "ONE GPU" in r.stderr


def test_without_a_gpu_the_bench_refuses_to_run():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    r = run(["--steps", "1", "--warmup", "0", "--cpu-seconds", "0"])
    assert r.returncode == 3 and "no CPU fallback" in r.stderr and r.stdout.strip() == ""


@pytest.mark.gpu
def test_headline_line_has_every_field_the_driver_reads():
    r = run(["--steps", "3", "--warmup", "1", "--cpu-seconds", "1"])
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [x for x in r.stdout.splitlines() if x.strip()]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 3 and rec["warmup"] == 1 and rec["unit"] == "TFLOP/s"
    assert rec["vs_baseline"] is None and rec["dtype"] == "bf16" and rec["data"] == "synthetic"
    assert "workload" in rec["config"] and "model" not in rec["config"]
    roof = rec["roofline"]
    assert roof["bound"] == "mfma" and roof["peak"] == 2500.0 and roof["unit"] == "TFLOP/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and 0.2 < roof["frac"] < 1.0
    # whole-call value and the kernel's own rate agree (one launch per step)
    assert abs(rec["value"] - roof["achieved"]) / roof["achieved"] < 0.1
    assert roof["traffic"] > roof["min_hbm_bytes"] and roof["traffic_source"].startswith("profiles/")
    # the rows the CPU baseline computed were compared with the timed launches' output
    par = rec["parity"]
    assert par["ok"] and par["rows"] >= 16 and par["heads"] == 12 and par["max_abs"] <= 1e-2 and par["cosine"] >= 0.9999
    cpu = rec["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "TFLOP/s" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]


@pytest.mark.gpu
@pytest.mark.parametrize("workload", ["tiny", "cross", "softmax", "kvcache1"])
def test_other_workloads_emit_one_json_line(workload):
    r = run(["--workload", workload, "--steps", "2", "--warmup", "1", "--cpu-seconds", "0"])
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [x for x in r.stdout.splitlines() if x.strip()]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    assert rec["n_gpus"] == 1 and rec["value"] > 0 and "workload" in rec["config"] and "roofline" in rec
    assert rec["roofline"]["bound"] in ("mfma", "hbm") and 0 < rec["roofline"]["frac"] < 1.0


@pytest.mark.gpu
def test_folded_scale_run_is_labelled_and_checks_its_own_output():
    r = run(["--workload", "tiny", "--fold-scale", "1", "--steps", "2", "--warmup", "1", "--cpu-seconds", "1"])
    assert r.returncode == 0, r.stderr[-2000:]
    rec = json.loads([x for x in r.stdout.splitlines() if x.strip()][-1])
    assert "folded" in rec["metric"] and "ln 2" in rec["data"] and rec["roofline"]["kernel"].endswith("true>")
    assert rec["parity"]["ok"]
