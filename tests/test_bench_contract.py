"""bench.py's command-line contract, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)


def test_workload_table_covers_the_baseline_configs():
    sys.path.insert(0, ROOT)
    import bench
    # one workload per BASELINE configuration plus the north-star dense layer; the default run times all of
    # them and puts the largest single-GPU configuration on the top level of the line
    assert set(bench.WORKLOADS) == {"cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "dense"}
    assert set(bench.ALL_ORDER) == set(bench.WORKLOADS) and bench.HEADLINE == "cfg5"
    assert bench.ALIASES == {"mlp": "cfg2", "conv": "cfg3", "cifar": "cfg4", "imagenet": "cfg5", "dense128": "cfg1"}


def test_carried_counters_name_their_source():
    sys.path.insert(0, ROOT)
    import bench
    c = bench.carried_counters("cfg3", "scan")
    assert c["hbm_bytes_per_launch"] > 0 and 0 < c["valu_busy"] <= 1.0 and "commit" in c["source"]
    assert bench.carried_counters("cfg3", "no_such_kernel") == {}


def test_roofline_picks_the_binding_side():
    sys.path.insert(0, ROOT)
    import bench
    # 1 GFLOP and 1 MB in 1 ms: compute side binds (6.4 us against 0.125 us)
    r = bench.roofline_for("k", 1e9, 1e6, 1.0, 1)
    assert r["bound"] == "mfma" and r["unit"] == "TFLOP/s" and r["peak"] == bench.VALU_PEAK_TFLOPS
    assert r["achieved"] == pytest.approx(1.0) and r["frac"] == pytest.approx(1.0 / bench.VALU_PEAK_TFLOPS)
    # 1 MFLOP and 1 GB in 1 ms: memory side binds
    r = bench.roofline_for("k", 1e6, 1e9, 0.5, 2)
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == bench.HBM_PEAK_GBS
    assert r["achieved"] == pytest.approx(1000.0) and r["frac"] == pytest.approx(0.125)


def test_weight_init_law():
    sys.path.insert(0, ROOT)
    import bench
    w = bench._w_init(np.random.default_rng(0), 784, 800)
    assert w.shape == (785, 800) and w.dtype == np.float32
    assert abs(w.mean() - 4.0 / 784) < 2e-4 and abs(w.var() - 1.0 / 784) < 2e-5


def _canned(key, batch):
    """What bench.measure() returns for one workload, with awkward (long, many-digit) values."""
    kernels = {f"kernel_{i}": {"launches_per_step": 10.0, "avg_us": 409.12345678901234, "us_per_step": 4091.2345678,
                               "gflop_per_step": 96.2712345678, "mbyte_per_step": 2423.123456789, "bound": "mfma",
                               "frac": 0.14961234567} for i in range(14)}
    return {
        "value": 3192.123456789012, "unit": "samples/s", "ms_per_step": 10.025123456789,
        "config": {"workload": "imagenet-shaped conv net B=32 fwd+bwd", "batch": batch, "launch": "hip graph replay",
                   "graph_note": None},
        "eager_ms_per_step": 10.0251234567, "graph_ms_per_step": 10.04012345678,
        "roofline": {"bound": "mfma", "achieved": 23.531234567890123, "peak": 157.3, "unit": "TFLOP/s",
                     "frac": 0.14961234567890123, "traffic": 540612345.6789, "valu_busy": 0.95212345678,
                     "note": "x" * 200, "kernel": "scan", "avg_launch_us": 409.12345678901234,
                     "launches_per_step": 10.0, "algorithmic_flops_per_step": 96271234567.0,
                     "algorithmic_bytes_per_step": 2423123456.0,
                     "counters_source": "profiles/counters.json at commit 0123456"},
        "kernels": kernels, "library_kernel_us_per_step": 9876.54321,
        "cpu_baseline": {"value": 0.11451234567, "unit": "samples/s", "cores": 1, "kind": "port",
                         "sample": "B=1, the same conv/dense layers (pooling and loss left out), fwd+bwd; reference "
                                   "host functors restated in C, gcc -O3, 1 thread",
                         "seconds": 8.7312345678, "host_cpus": 16},
        "gpu_over_cpu": 27876.123456,
    }


def test_record_line_is_short_and_parses_on_its_own():
    """The record line (last line of stdout) must stay under the driver's size limit with all six workloads in
    it, parse by itself, and carry the roofline and the CPU baseline of the headline workload."""
    import json
    sys.path.insert(0, ROOT)
    import bench
    per_config = {k: _canned(k, 32) for k in bench.ALL_ORDER}
    rec = bench.headline(per_config[bench.HEADLINE], per_config, 100, 10, "AMD Instinct MI355X")
    line = json.dumps(rec, separators=(",", ":"))
    assert len(line) < bench.LINE_BUDGET, len(line)
    back = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "per_config"):
        assert key in back, key
    assert back["config"]["workload"] and "model" not in back["config"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in back["roofline"], key
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in back["cpu_baseline"], key
    assert set(back["per_config"]) == set(bench.ALL_ORDER)
    assert all(len(row) == len(back["per_config_fields"]) for row in back["per_config"].values())
    assert back["value"] == pytest.approx(3192.1, rel=1e-4)        # rounded to 5 significant digits
    assert "kernels" not in back
    # a single workload: no per_config table
    one = bench.headline(per_config["cfg3"], None, 20, 5, "AMD Instinct MI355X")
    assert "per_config" not in one and len(json.dumps(one, separators=(",", ":"))) < bench.LINE_BUDGET
