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
    assert c["hbm_bytes_per_launch"] > 0 and 0 < c["valu_busy"] <= 1.1 and "commit" in c["source"]
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
