"""bench.py's command line and the shape of its one JSON line (the driver parses it)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*flags, timeout=600):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True,
                          timeout=timeout, cwd=ROOT)


def test_bench_measures_one_gpu_only():
    res = run_bench("--gpus", "2", timeout=60)
    assert res.returncode != 0
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


def _check_roofline(obj, bound, unit):
    r = obj["roofline"]
    assert r["bound"] == bound and r["unit"] == unit
    assert r["peak"] > 0 and r["achieved"] > 0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9
    assert "traffic" in r and "kernel" in r


@pytest.mark.gpu
def test_bench_line_has_the_fields_the_driver_reads():
    """A short run of the headline leg (configs[3] decode) and of the prefill leg: one JSON line on stdout with the
    contract's fields, `value` consistent with `ms_per_step`, rooflines that carry their own arithmetic."""
    print("case: bench.py --only decode / --only prefill, 3 steps", flush=True)
    res = run_bench("--only", "decode", "--steps", "3", "--warmup", "1", "--no-cpu")
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [ln for ln in res.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["unit"] == "GB/s" and d["vs_baseline"] is None and "workload" in d["config"]
    assert abs(d["value"] - d["config"]["algorithmic_bytes"] / d["ms_per_step"] / 1e6) < 1e-6 * d["value"]
    _check_roofline(d, "hbm", "GB/s")

    res = run_bench("--only", "prefill", "--steps", "3", "--warmup", "1", "--no-cpu")
    assert res.returncode == 0, res.stderr[-2000:]
    d = json.loads([ln for ln in res.stdout.splitlines() if ln.strip()][-1])
    assert d["unit"] == "TFLOP/s" and d["dtype"] == "bf16" and "configs[2]" in d["config"]["workload"]
    _check_roofline(d, "mfma", "TFLOP/s")
    _check_roofline(d["prefill"], "mfma", "TFLOP/s")
