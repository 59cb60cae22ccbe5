"""bench.py's command line, as far as it can be checked without a GPU: one GPU only, and no silent CPU run."""
import os
import subprocess
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    done = _bench("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert done.returncode == 2 and done.stdout.strip() == ""              # no JSON line that could be mistaken for a result
    assert "one GPU" in done.stderr and "--gpus 1" in done.stderr


def test_without_a_gpu_the_bench_fails_instead_of_measuring_something_else():
    if torch.cuda.is_available():
        return                                                             # the GPU suite covers the real run
    done = _bench("--steps", "1", "--warmup", "0")
    assert done.returncode != 0 and done.stdout.strip() == ""
    assert "needs a GPU" in done.stderr


import json

import pytest


@pytest.mark.gpu
def test_bench_prints_one_json_line_with_the_contract_fields():
    done = _bench("--steps", "5", "--warmup", "2", "--no-extras")
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [l for l in done.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 5 and out["warmup"] == 2 and out["vs_baseline"] is None
    assert out["unit"] == "TFLOP/s" and out["dtype"] == "fp16" and "workload" in out["config"] and "model" not in out["config"]
    roof = out["roofline"]
    assert roof["bound"] == "mfma" and roof["peak"] == 2500.0 and roof["unit"] == "TFLOP/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and 0.2 < roof["frac"] < 0.7
    # the algorithmic count: 2 * B * H * S_q * S_kv * (d_qk + d_v) at B4 H32 S2048 D128
    assert roof["algorithmic_flops_per_launch"] == 2 * 4 * 32 * 2048 * 2048 * 256
    assert abs(out["value"] - roof["algorithmic_flops_per_launch"] / (out["ms_per_step"] * 1e-3) / 1e12) < 0.01 * out["value"]
    cpu = out["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "TFLOP/s" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
