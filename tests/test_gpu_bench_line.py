"""bench.py end to end on the smallest workload: the JSON line's contract, and the
variants of the measurement (general pipeline, int64 indices, double precision)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*flags):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "c1", "--steps", "3", "--warmup", "1",
                        "--no-cpu"] + list(flags), stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=170)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1                                    # ONE JSON line
    return json.loads(lines[0])


@pytest.mark.parametrize("flags,pipeline,bits,dtype", [
    ((), "optimised", 32, "f32"),
    (("--general",), "general", 32, "f32"),
    (("--index-bits", "64"), "optimised", 64, "f32"),
    (("--general", "--index-bits", "64"), "general", 64, "f32"),
    (("--dtype", "f64"), "optimised", 32, "f64"),
])
def test_bench_line(flags, pipeline, bits, dtype):
    out = _bench(*flags)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 3 and out["warmup"] == 1 and out["vs_baseline"] is None
    assert out["dtype"] == dtype and out["config"]["pipeline"] == pipeline and out["config"]["index_bits"] == bits
    assert out["spot_check_vs_oracle"] is True and out["value"] > 0
    rl = out["roofline"]
    assert rl["bound"] == "hbm" and rl["peak"] == 8000.0 and abs(rl["frac"] - rl["achieved"] / rl["peak"]) < 1e-12
    # c1 is 262 144 edges of 32 columns: 132 bytes per edge and 264 per row with int32 indices and float values
    vb, ib = (8 if dtype == "f64" else 4), bits // 8
    want = 262144 * (32 * vb + ib) + 16384 * ((3 if pipeline == "general" else 2) * 32 * vb + 2 * ib)
    assert rl["algorithmic_bytes"] == want
    assert rl["traffic"] is None                              # c1 is cache-resident: no counter traffic is quoted for it


def test_forced_row_order_and_wide_z_rows_keep_the_bits():
    """A uniform graph taken in scattered order (FUSEDMM_ROW_ORDER=scattered; the library would
    not choose it here) with the rows of Z four times their length apart: the spot check
    against the oracle still holds bit for bit, and the line says which order ran."""
    env = dict(os.environ, FUSEDMM_ROW_ORDER="scattered")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "u512d64", "--steps", "2", "--warmup", "1",
                        "--no-cpu", "--ldz", "2048"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=170,
                       env=env)
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["spot_check_vs_oracle"] is True and out["row_order"]["scattered"] is True and out["config"]["ldz"] == 2048
    lo, hi = out["row_order"]["sampled_edges_lower_half"], out["row_order"]["sampled_edges_upper_half"]
    assert lo > 0 and abs(lo - hi) <= 0.05 * lo              # the sample itself says: evenly spread


def test_extra_workloads_ride_in_the_same_line():
    """--also: the extra workloads are measured after the headline one and reported compactly in the same
    single JSON line, each with its own roofline figures, gather probe and spot check."""
    out = _bench("--also", "c1,u512d64", "--also-steps", "2")
    assert out["config"]["workload"].startswith("c1:") and "gather_probe" not in out["roofline"]
    also = out["also"]
    assert [a["workload"].split(":")[0] for a in also] == ["c1", "u512d64"]
    for a in also:
        assert a["spot_check_vs_oracle"] is True and a["steps"] == 2 and a["ms_per_step"] > 0 and a["kernel_ms"] > 0
        rl = a["roofline"]
        assert rl["bound"] == "hbm" and abs(rl["frac"] - rl["achieved"] / 8000.0) < 1e-12
        assert rl["gather_probe_GBps"] > 0 and abs(rl["frac_of_gather_probe"] - rl["achieved"] / rl["gather_probe_GBps"]) < 1e-9
        assert a["algorithmic_bytes"] > 0 and set(a["split"]) == {"heavy_rows", "segments", "overflow"}
    assert also[0]["algorithmic_bytes"] == 262144 * 132 + 16384 * 264
