"""The benchmark's command-line contract, as far as it can be checked without a GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args, env=None):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          env={**os.environ, **(env or {})}, timeout=300)


def test_more_than_one_gpu_is_refused():
    r = run_bench("--gpus", "2")
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)
    r = run_bench(env={"WORLD_SIZE": "2"})
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)


def test_no_gpu_means_no_number():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    r = run_bench()
    assert r.returncode != 0 and "no CPU fallback" in (r.stderr + r.stdout)
    assert not r.stdout.strip().startswith("{")


@pytest.mark.gpu
def test_json_line_has_the_contract_fields():
    r = run_bench("--steps", "3", "--warmup", "1", "--no-cpu-baseline")
    assert r.returncode == 0, r.stderr[-2000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(line) == 1
    d = json.loads(line[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["vs_baseline"] is None and "workload" in d["config"]
    rf = d["roofline"]
    assert rf["bound"] == "mfma" and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3 and rf["traffic"] > 0
