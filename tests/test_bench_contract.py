"""bench.py host-side contract that needs no GPU."""
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout == ""


def test_algorithmic_bytes_formula_matches_the_stated_c2_figure():
    sys.path.insert(0, ROOT)
    from fusedmm_amd import synth
    # nnz (4K + I) + m (4K [X] + 4K [Z] + 2I):  2^24 * 516 + 2^20 * 1032
    assert synth.algorithmic_bytes("s", 1 << 20, 128, 1 << 24, 4) == 9739173888
    assert synth.algorithmic_bytes("m", 10, 256, 100, 4) == 100 * (1024 + 4 + 4) + 10 * (1024 + 8)
    assert synth.algorithmic_flops("s", 128, 1 << 24) == 4 * 128 * (1 << 24)


def test_scaled_workloads_have_the_advertised_shape():
    sys.path.insert(0, ROOT)
    import bench
    g, X, Y = bench.make_workload("c2", 8)
    assert g["rows"] == 4096 and g["nnz"] == 65536 and X.shape == (4096, 128) and X is not Y
    deg = np.diff(g["rowptr"])
    rid = np.repeat(np.arange(4096), deg)
    assert (g["indx"] != rid).all()                                   # no self loops
    assert all(np.all(np.diff(g["indx"][a:b]) > 0) for a, b in zip(g["rowptr"][:50], g["rowptr"][1:51]))  # sorted, distinct
    g, X, Y = bench.make_workload("c1", 4)
    assert X is Y and np.abs(X).max() <= 1.0                          # A = B, U[-1, 1]
    g, _, _ = bench.make_workload("c5", 6)
    assert np.diff(g["rowptr"]).max() == min(1000000, (1 << 15) // 2)  # hubs at the cap


def test_traffic_figures_come_from_the_committed_profiles():
    """roofline.traffic is read from the rocprofv3 summary of the workload (no table
    in bench.py to go stale): every profiled workload has a parsable figure that sits
    next to the algorithmic bytes the same file states."""
    import re
    sys.path.insert(0, ROOT)
    import bench
    for w, fname in bench.PROFILE_OF.items():
        path = os.path.join(ROOT, "profiles", fname)
        assert os.path.exists(path), fname
        got, src = bench.measured_traffic_bytes(w)
        assert src == "profiles/" + fname and got and got > 0
        text = open(path).read()
        m = re.search(r"traffic per call: ([0-9.]+) GB against ([0-9.]+) GB algorithmic", text)
        assert m, fname
        assert abs(got / 1e9 - float(m.group(1))) < 1e-3
        assert 0.8 < got / 1e9 / float(m.group(2)) < 1.1, (w, got)
        assert "rocprofv3 --kernel-trace --stats" in text and "python3 bench.py --workload " + w in text
    assert bench.measured_traffic_bytes("c1") == (None, None)      # cache-resident case: no roofline claim


def test_uniform_degree_workloads_and_the_bytes_of_the_general_rule():
    sys.path.insert(0, ROOT)
    import bench
    from fusedmm_amd import synth
    g, X, Y = bench.make_workload("u512d16", 8)
    assert g["rows"] == 8192 and g["cols"] == 8192 and g["nnz"] == 8192 * 16 and X.shape == (8192, 512) and Y.shape == (8192, 512)
    assert (np.diff(g["rowptr"]) == 16).all() and g["indx"].min() >= 0 and g["indx"].max() < 8192
    g, X, Y = bench.make_workload("u512d512", 8)
    assert g["rows"] == (1 << 17) // 512 and X.shape[0] == g["rows"] and Y.shape[0] == 8192      # fewer rows than columns
    # the general rule reads Z before it writes it: one more row of K values per row; int64 indices: 8 bytes each
    base = synth.algorithmic_bytes("s", 1000, 128, 16000, 4)
    assert synth.algorithmic_bytes("s", 1000, 128, 16000, 4, beta_nonzero=True) == base + 1000 * 128 * 4
    assert synth.algorithmic_bytes("s", 1000, 128, 16000, 8) == base + 16000 * 4 + 1000 * 2 * 4
    assert synth.algorithmic_bytes("s", 1000, 128, 16000, 4, value_bytes=8) == 16000 * (1024 + 4) + 1000 * (2048 + 8)


def test_the_default_run_also_times_the_other_bandwidth_target_and_the_skewed_graphs():
    """The one JSON line of the default run carries, under "also", the gcn K=256 configuration (the second one
    with a bandwidth target) first, then the skewed graphs; each entry has its own roofline figures and spot check."""
    sys.path.insert(0, ROOT)
    import bench
    assert bench.ALSO_DEFAULT[0] == "c3g" and set(bench.ALSO_DEFAULT) == {"c3g", "c4", "c5", "c3", "k128er"}
    assert all(w in bench.WORKLOADS and w in bench.PROFILE_OF for w in bench.ALSO_DEFAULT)
    full = {"value": 1.0, "unit": "GFLOP/s", "steps": 10, "warmup": 2, "ms_per_step": 2.0, "edges_per_s": 3.0,
            "config": {"workload": "c3g: x", "op": "g", "K": 256, "rows": 4, "nnz": 5, "graph_gen_s": 1.0, "store_tick": "auto",
                       "y_bytes": 4096},
            "split": {"heavy_rows": 1, "segments": 2, "overflow": 0}, "row_order": {"scattered": True},
            "spot_check_vs_oracle": True,
            "roofline": {"bound": "hbm", "achieved": 6400.0, "peak": 8000.0, "unit": "GB/s", "frac": 0.8, "traffic": 7,
                         "traffic_from": "profiles/x.md", "kernel": "fused_kernel", "kernel_ms": 1.9,
                         "algorithmic_bytes": 11, "frac_of_gather_probe": 1.1, "gather_probe": {"plain_loads_GBps": 5800.0}}}
    c = bench.compact("c3g", full)
    for key in ("workload", "ms_per_step", "kernel_ms", "algorithmic_bytes", "roofline", "split", "spot_check_vs_oracle"):
        assert key in c, key
    assert c["roofline"]["frac"] == 0.8 and c["roofline"]["traffic"] == 7 and c["roofline"]["frac_of_gather_probe"] == 1.1
    assert c["roofline"]["gather_probe_GBps"] == 5800.0 and c["kernel_ms"] == 1.9 and c["row_order_scattered"] is True
    assert c["store_tick"] == "auto" and c["y_bytes"] == 4096
    assert (4, 8) in bench.GATHER_PROBE_SHAPES and len(bench.GATHER_PROBE_SHAPES) >= 2     # the kernel's own launch shape and the probe's best
    # the narrow-row workloads: 2^23 rows of 128 and 256 bytes, 2^27 edges
    g, X, Y = bench.make_workload("k32er", 10)
    assert g["rows"] == 8192 and g["nnz"] == 16 * 8192 and X.shape == (8192, 32) and X is not Y
    assert bench.WORKLOADS["k64er"][2] == 64 and "L2-miss" in bench.TRAFFIC_IS


def test_also_rejects_unknown_workloads_before_touching_the_gpu():
    a = bench_args("--also", "c3g,c4")
    assert a.also == "c3g,c4" and a.also_steps == 10
    assert bench_args().also == "auto"


def bench_args(*argv):
    sys.path.insert(0, ROOT)
    import bench
    return bench.parse_args(list(argv))
