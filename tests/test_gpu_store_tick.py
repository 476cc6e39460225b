"""When finished rows of Z are written (fusedMM_amd_set_store_tick): rows wait in LDS and leave on a common clock
tick, or when a wavefront's share of LDS is full.  Whatever the period -- every few microseconds, never within the
call (so that only full shares trigger a write), or the default -- Z must come out with the bits of the call that
writes every row as it finishes.  The graphs are large enough for every wavefront to take many rows: shares fill
up and several ticks pass inside one call."""
import numpy as np
import pytest

import bench
import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES, Oracle

pytestmark = pytest.mark.gpu


def _run_with_tick(lib, shift, imsg, g, X, Y, Z0, beta, bits=32, vbits=32):
    prev = lib.fusedMM_amd_set_store_tick(shift)
    try:
        rc, Z = gpu_api.run(imsg, g, X, Y, Z0, beta=beta, bits=bits, vbits=vbits)
    finally:
        lib.fusedMM_amd_set_store_tick(prev)
    assert rc == 0
    return Z


# name, scale-down: K=64 R-MAT (packed groups, half the rows empty), K=256 R-MAT (whole-wave rows), K=128 ER
# (two sub-waves per row), K=512 Zipf (two registers per lane: few rows fit a share), K=32 ER
@pytest.mark.parametrize("name,sd", [("c4", 6), ("c3", 5), ("c2", 3), ("c5", 3), ("k32er", 5)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_every_period_gives_the_bits_of_immediate_stores(name, sd, beta):
    desc, tkern, k, kind = bench.WORKLOADS[name]
    g, X, Y = bench.make_workload(name, sd)
    sk = SOP_NAMES[kind] if kind else 0
    gpu_api.set_kind(sk, 32)
    lib = fa.load(32)
    Z0 = graphs.features(g["rows"], k, 5, -1.0, 1.0, stream=3) if beta else np.zeros((g["rows"], k), np.float32)
    print("case", name, sd, beta, "rows", g["rows"], "nnz", g["nnz"], flush=True)
    Zoff = _run_with_tick(lib, 0, MSG[tkern], g, X, Y, Z0, beta)
    assert np.isfinite(Zoff).all() and float(np.abs(Zoff).max()) > 0
    for shift in (8, 24, -1):
        print("  shift", shift, flush=True)
        Z = _run_with_tick(lib, shift, MSG[tkern], g, X, Y, Z0, beta)
        np.testing.assert_array_equal(Z.view(np.uint32), Zoff.view(np.uint32), err_msg="shift %d" % shift)


@pytest.mark.parametrize("bits,vbits", [(64, 32), (32, 64), (64, 64)])
def test_other_libraries(bits, vbits):
    """int64 indices and double precision (a double row takes twice the LDS: half as many rows wait)."""
    np_v = np.float32 if vbits == 32 else np.float64
    it = np.int32 if bits == 32 else np.int64
    g, X, Y = bench.make_workload("c4", 7)
    g = dict(g)
    for key in ("indx", "pntrb", "pntre", "rowptr"):
        g[key] = g[key].astype(it)
    X, Y = X.astype(np_v), Y.astype(np_v)
    Z0 = np.zeros((g["rows"], 64), np_v)
    sk = SOP_NAMES["tdist"]
    gpu_api.set_kind(sk, bits, vbits)
    lib = fa.load(bits, vbits)
    Zoff = _run_with_tick(lib, 0, MSG["t"], g, X, Y, Z0, 0.0, bits, vbits)
    bits_of = np.uint32 if vbits == 32 else np.uint64
    for shift in (8, 24, -1):
        print("lib", bits, vbits, "shift", shift, flush=True)
        Z = _run_with_tick(lib, shift, MSG["t"], g, X, Y, Z0, 0.0, bits, vbits)
        np.testing.assert_array_equal(Z.view(bits_of), Zoff.view(bits_of), err_msg="shift %d" % shift)


def test_general_pipeline_and_the_mirror():
    """The general pipeline (Z is read before it is written) under every period, and the default period against
    the CPU mirror of the kernels' summation order."""
    oracle = Oracle()
    g, X, Y = bench.make_workload("c2", 4)
    k = 128
    sk = SOP_NAMES["sigmoid"]
    gpu_api.set_kind(sk, 32)
    lib = fa.load(32)
    Z0 = graphs.features(g["rows"], k, 6, -1.0, 1.0, stream=3)
    want = gpu_api.oracle_mirror(oracle, "s", g, X, Y, np.zeros_like(Z0), 0.0, sk, k, *gpu_api.default_split(k))
    Z = _run_with_tick(lib, -1, MSG["s"], g, X, Y, np.zeros_like(Z0), 0.0)
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))
    prev_opt = lib.fusedMM_amd_set_opt(0)
    try:
        Zoff = _run_with_tick(lib, 0, MSG["s"], g, X, Y, Z0, 1.0)
        for shift in (8, 24, -1):
            Zg = _run_with_tick(lib, shift, MSG["s"], g, X, Y, Z0, 1.0)
            np.testing.assert_array_equal(Zg.view(np.uint32), Zoff.view(np.uint32), err_msg="general, shift %d" % shift)
    finally:
        lib.fusedMM_amd_set_opt(prev_opt)


@pytest.mark.parametrize("seed", range(8))
def test_random_mixtures_of_row_lengths(seed):
    """Tens of thousands of rows per call, so that every wavefront takes many of them: stretches of empty, short, medium
    and long rows in random order (packed groups, whole-wavefront rows, rows to clear and rows cut into segments all
    meet in one wavefront's share of LDS), random widths with and without idle lanes, strides wider than K, m < rows."""
    from fusedmm_amd import synth
    from test_gpu_random_cases import _random_degrees
    rng = np.random.default_rng(4100 + seed)
    rows, cols = int(rng.integers(60000, 150000)), int(rng.integers(2000, 50000))
    k = [20, 32, 64, 100, 128, 160, 260, 512][seed]
    tkern, kind = [("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist"), ("f", "fr")][seed % 5]
    beta = float(seed % 2)
    deg = _random_degrees(rng, rows)
    deg[rng.integers(0, rows // 2, 3)] = [500, 2000, 7000]   # long rows among the first half (m covers them): cut into segments
    rowptr = np.concatenate([[0], np.cumsum(deg)])
    nnz = int(rowptr[-1])
    g = synth.graph_from_rowptr(rows, cols, rowptr, rng.integers(0, cols, nnz, dtype=np.int64), None, 32)
    g["val"] = synth.edge_values(nnz, seed)
    ld = k + 4 * int(rng.integers(0, 3))
    lo, hi = (-0.5, 0.5) if tkern in ("s", "g", "m") else (-1.0, 1.0)
    X = graphs.features(rows, ld, seed, lo, hi, 1)
    Y = graphs.features(cols, ld, seed, lo, hi, 2)
    if tkern == "f":
        Y = (Y + np.float32(3.0)).astype(np.float32)
    Z0 = graphs.features(rows, ld, seed, -1, 1, 3)
    m = rows if seed % 3 else int(rng.integers(rows // 2, rows))
    sk = SOP_NAMES[kind] if kind else 0
    lib = fa.load(32)
    gpu_api.set_kind(sk, 32)
    gpu_api.set_split(int(rng.integers(40, 400)), int(rng.integers(16, 128)), 32)
    print("case", seed, dict(rows=rows, cols=cols, k=k, op=tkern, beta=beta, ld=ld, m=m, nnz=nnz), flush=True)
    try:
        out = {}
        for shift in (0, 8, 24, 13):
            prev = lib.fusedMM_amd_set_store_tick(shift)
            try:
                rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, m=m, k=k, ldx=ld, ldy=ld, ldz=ld)
            finally:
                lib.fusedMM_amd_set_store_tick(prev)
            assert rc == 0
            out[shift] = Z
    finally:
        gpu_api.set_split(0, 0, 32)
    assert gpu_api.last_split()[1] > 0                      # some rows were cut into segments
    for shift in (8, 24, 13):
        np.testing.assert_array_equal(out[shift].view(np.uint32), out[0].view(np.uint32), err_msg="shift %d" % shift)
    np.testing.assert_array_equal(out[0][m:], Z0[m:])
    np.testing.assert_array_equal(out[0][:, k:], Z0[:, k:])
    assert np.isfinite(out[0]).all()


def test_setter_returns_the_previous_value_and_clamps():
    lib = fa.load(32)
    first = lib.fusedMM_amd_set_store_tick(12)
    try:
        assert lib.fusedMM_amd_set_store_tick(0) == 12
        assert lib.fusedMM_amd_set_store_tick(99) == 0        # out of range: the default
        assert lib.fusedMM_amd_set_store_tick(-1) == -1
    finally:
        lib.fusedMM_amd_set_store_tick(first)
