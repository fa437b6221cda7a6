"""bench.py's command line and the one JSON line it prints.

Without a GPU: more than one GPU is turned away with a message, and so is a machine without a GPU (no CPU fallback
is ever timed as the product).  With a GPU: a short run on a small memory map prints one JSON line that carries
every field of the contract, a roofline whose figures are consistent with each other and a CPU baseline."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def run(*args, timeout=600):
    return subprocess.run([sys.executable, BENCH, *args], capture_output=True, text=True, cwd=ROOT, timeout=timeout)


def test_more_than_one_gpu_is_turned_away():
    proc = run("--gpus", "2")
    assert proc.returncode != 0 and "ONE GPU" in proc.stderr and proc.stdout.strip() == ""


def test_without_a_gpu_nothing_is_measured():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    proc = run("--steps", "2", "--warmup", "1")
    assert proc.returncode != 0 and "no GPU" in proc.stderr and proc.stdout.strip() == ""


@pytest.mark.gpu
def test_the_json_line_carries_the_contract():
    import torch
    torch.cuda.empty_cache()   # this process may hold pools of earlier tests; the benchmark builds its own map
    proc = run("--steps", "6", "--warmup", "2", "--no-extras", "--weight-gib", "4", "--pool-blocks", "8192")
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, proc.stdout[-2000:]
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 6 and d["warmup"] == 2 and d["higher_is_better"] is True
    assert d["unit"] == "GB/s" and d["vs_baseline"] is None and d["data"].startswith("synthetic")
    assert "workload" in d["config"] and "model" not in d["config"]
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert 0.3 < roof["frac"] < 1.0 and 0.3 < roof["frac_compact"] < 1.0
    nbytes = d["config"]["valid_tokens"] * d["config"]["layers"] * 6144     # 6n bytes per valid token and layer
    assert abs(roof["achieved"] - nbytes / roof["kernel_us_mean"] / 1e3) < 0.01 * roof["achieved"]
    assert roof["traffic"] is None or roof["traffic"] >= nbytes
    # whole-job throughput can not beat the kernel's own rate
    assert d["value"] <= roof["achieved"] * 1.02 and abs(d["value"] - nbytes / d["ms_per_step"] / 1e6) < 0.01 * d["value"]
    cpu = d["cpu_baseline"]
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    # the same write as PyTorch CPU operations, beside the port
    torch_cpu = d["cpu_baseline_pytorch"]
    assert torch_cpu["kind"] == "pytorch" and torch_cpu["cores"] >= 1 and torch_cpu["value"] > 0 and torch_cpu["sample"]
    # where the traffic figure comes from: a day and a commit, not just a file
    assert "measured on 20" in roof["traffic_source"] and "commit" in roof["traffic_source"]
    assert d["extras"]["box_reference"]["torch_copy_1GiB_GBps"] > 0
