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
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-4 * r["frac"]
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
    assert len(lines[0]) <= 7000
    _check_roofline(d, "hbm", "GB/s")

    res = run_bench("--only", "prefill", "--steps", "3", "--warmup", "1", "--no-cpu")
    assert res.returncode == 0, res.stderr[-2000:]
    d = json.loads([ln for ln in res.stdout.splitlines() if ln.strip()][-1])
    assert d["unit"] == "TFLOP/s" and d["dtype"] == "bf16" and "configs[2]" in d["config"]["workload"]
    _check_roofline(d, "mfma", "TFLOP/s")
    _check_roofline(d["prefill"], "mfma", "TFLOP/s")
    assert list(d)[-1] == "prefill"


def _fake_leg(bound, unit, workload, with_cpu=False):
    """A leg object of the shape bench.py builds, with floats as long as real ones."""
    o = {"value": 1234.5678901234567, "unit": unit, "ms_per_step": 0.9052512345678901, "dtype": "bf16",
         "algorithmic_flops": 1099511627776, "kv_splits": 8, "config": {"workload": workload, "algorithmic_bytes": 4582589688},
         "roofline": {"bound": bound, "kernel": "some_kernel_name<with, template, arguments> + another_kernel",
                      "achieved": 1216.8123456789012, "peak": 2500.0, "unit": unit, "frac": 0.48672493827156048,
                      "device_ms": 0.90362123456789012, "traffic": 683572122}}
    if with_cpu:
        o["cpu_baseline"] = {"value": 0.14660123456789012, "unit": unit, "cores": 16, "kind": "port",
                             "seconds_per_pass": 0.46873123456789012, "passes": 20, "sample": "s" * 160}
        o["parity"] = {"checked_heads": 8, "max_abs_err": 0.0039115123456789012, "within_2e-2_abs_1e-2_rel": True}
    return o


def test_printed_line_ends_with_the_prefill_object_and_stays_short():
    """The driver keeps the last 8 KB of stdout and quotes the last 2 KB: the printed line must stay well below the
    first and carry the configs[2] prefill object (roofline, cpu_baseline, parity) whole inside the second."""
    sys.path.insert(0, ROOT)
    import bench

    long = "w" * 170
    full = {"metric": bench.METRIC, "n_gpus": 1, "steps": 20, "warmup": 5, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "data": "synthetic (seeded)", "burn_in_ms_before_every_leg_but_decode": 40.0,
            "value": 6358.454536586412, "unit": "GB/s", "ms_per_step": 0.720708100000067, "dtype": "bf16",
            "config": {"workload": long, "tokens": 1118216, "algorithmic_bytes": 4582589688},
            "roofline": _fake_leg("hbm", "GB/s", long)["roofline"]}
    full["prefill_few_sequences"] = {n: _fake_leg("mfma", "TFLOP/s", long) for n in
                                     ("prompt_8192", "prompt_16384", "prompt_2048", "chunk_256_over_16384", "ragged_batch_16")}
    full["prefill_small_shapes"] = {n: _fake_leg("mfma", "TFLOP/s", long, True) for n in ("prefill_cfg1", "prefill_sample_model")}
    full["prefill_backward"] = _fake_leg("mfma", "TFLOP/s", long)
    full["decode_fp8"] = _fake_leg("hbm", "GB/s", long, True)
    full["decode_fp8"]["parity_vs_bf16_kv"] = {"reference": "r" * 60, "checked_sequences": 128, "max_abs_err": 0.050432123456,
                                               "rms_err_over_rms_ref": 0.0379791234567, "bound": "b" * 50, "within_bound": True}
    full["cache_producers"] = {n: _fake_leg("hbm", "GB/s", long) for n in ("rope_and_cache", "rope_and_cache_fp8", "quantize_kv_fp8")}
    full["layer_ops"] = {n: _fake_leg("hbm", "GB/s", long) for n in ("rms_norm_residual", "silu_mul")}
    full["decode_few_sequences"] = {n: _fake_leg("hbm", "GB/s", long) for n in
                                    ("one_sequence_8192", "one_sequence_32768", "four_sequences_8192")}
    full["decode_loop"] = {"config": {"workload": long}, "eager": {"ms_per_step": 0.97977123456, "tokens_per_s": 8165.1},
                           "hip_graph": {"ms_per_step": 0.28304123456, "tokens_per_s": 28264.9}, "speedup": 3.46}
    full["cpu_baseline"] = _fake_leg("hbm", "GB/s", long, True)["cpu_baseline"]
    full["parity"] = {"checked_sequences": 128, "max_abs_err": 0.00081845123456, "within_2e-2_abs_1e-2_rel": True}
    full["config0"] = {"config": {"workload": long}, "cpu_baseline": full["cpu_baseline"],
                       "gpu": {"ms_per_step": 0.0163, "device_ms": 0.0126123456789, "dtype": "bf16", "note": "n" * 50},
                       "parity": {"max_abs_err": 0.0015764, "within_2e-2_abs_1e-2_rel": True}}
    full["prefill"] = _fake_leg("mfma", "TFLOP/s", long, True)

    line = json.dumps(bench.compact_line(full))
    assert len(line) <= bench.LINE_BUDGET, len(line)
    d = json.loads(line)
    assert list(d)[-1] == "prefill"
    tail = line[-bench.PREFILL_TAIL:]
    start = tail.find('"prefill": {')
    assert start >= 0, "the prefill object does not fit the quoted tail"
    obj = json.loads(tail[start + len('"prefill": '):-1])
    for key in ("value", "unit", "ms_per_step", "roofline", "cpu_baseline", "parity"):
        assert key in obj, key
    assert {"frac", "achieved", "peak", "bound", "traffic"} <= set(obj["roofline"])
    assert {"value", "unit", "cores", "kind", "sample"} <= set(obj["cpu_baseline"])
    # headline fields pass through untouched
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data"):
        assert d[key] == full[key], key
    assert d["config"]["workload"] == long and "frac" in d["roofline"] and d["cpu_baseline"]["cores"] == 16
    assert set(d["legs"]) >= {"prefill_cfg1", "prefill_sample_model", "prefill_backward_cfg2", "ragged_batch_16", "config0"}
