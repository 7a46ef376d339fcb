"""bench.py end to end at its smallest configuration, once per mode, as the driver starts it (a child process):
every mode must print one JSON line with the contract's keys."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
COMMON = ["--config", "c1", "--steps", "16", "--warmup", "4", "--repeats", "3", "--no-read-probe"]


@pytest.mark.parametrize("mode", [
    [],                                                       # device-resident store, the headline path
    ["--no-graph", "--no-kmeans"],                            # eager launches
    ["--residency", "host", "--layers", "2"],                 # host store, block cache managed on the device
    ["--residency", "host", "--layers", "2", "--overlap"],    # ... cached rows attended beside the miss staging
    ["--residency", "host", "--layers", "2", "--block-cache", "host"],   # ... managed by the worker threads
    ["--dtype", "fp16", "--no-other-configs"],                # IEEE half elements, device-resident store
    ["--dtype", "fp16", "--residency", "host", "--layers", "2"],   # ... host store
])
def test_bench_mode_prints_the_contract_line(dev, mode):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + COMMON + mode, capture_output=True, text=True,
                       timeout=110, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 16 and line["value"] > 0
    assert "workload" in line["config"]
    assert line["roofline"] is not None and line["roofline"]["bound"] == "hbm" and 0 < line["roofline"]["frac"] < 1
    assert line["cpu_baseline"] is not None and line["cpu_baseline"]["kind"] in ("port", "reference")
    assert line["dtype"] == ("f16" if "fp16" in mode else "bf16")
    assert line["cpu_baseline"]["max_abs_vs_gpu"] <= 2e-2     # the oracle's output of the same step


@pytest.mark.parametrize("mode", [
    ["--estimate-next", "--layers", "4"],     # zones of the next layer chosen from a predicted query on a side stream
    ["--end-to-end"],                         # the random-weight model around the path, whole tokens per graph
])
def test_bench_side_modes_run(dev, mode):
    """The two modes that measure something other than the contract's metric still run and print one JSON line."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + COMMON + mode, capture_output=True, text=True,
                       timeout=110, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert line["value"] > 0 and line["n_gpus"] == 1 and "workload" in line["config"]


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=110, cwd=ROOT)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)
