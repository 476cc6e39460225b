"""Seeded random sweep over shapes, strides, index widths, precisions, tuples and
split thresholds, each checked against the CPU oracle."""
import os

import numpy as np
import pytest

import checks
import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES, Oracle

pytestmark = pytest.mark.gpu
_ORC = {}
# FUSEDMM_TEST_SEEDS=<n> widens both sweeps (default: 48 pattern cases, 32 general tuples)
_N = int(os.environ.get("FUSEDMM_TEST_SEEDS", "0"))


def orc(vbits):
    if vbits not in _ORC:
        _ORC[vbits] = Oracle(vbits=vbits)
    return _ORC[vbits]


@pytest.mark.parametrize("seed", range(_N or 48))
def test_random_pattern_case(seed):
    rng = np.random.default_rng(1000 + seed)
    bits = int(rng.choice([32, 64]))
    vbits = int(rng.choice([32, 64]))
    np_v = np.float32 if vbits == 32 else np.float64
    rows, cols = int(rng.integers(1, 90)), int(rng.integers(1, 120))
    k = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 31, 32, 33, 64, 100, 128, 200, 256, 300, 512, 640]))
    hub = int(rng.choice([0, 5, 70, 900]))
    tkern, kind = [("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist"), ("f", "fr"), ("s", "ll"), ("t", "fa")][seed % 7]
    beta = float(rng.choice([0.0, 1.0]))
    # a ragged graph with arbitrary (possibly repeated, unsorted) columns
    lists = [rng.integers(0, cols, int(rng.integers(0, 9))) for _ in range(rows)]
    if hub and rows > 2:
        lists[int(rng.integers(0, rows))] = rng.integers(0, cols, hub)
    deg = np.array([len(x) for x in lists], np.int64)
    rowptr = np.concatenate([[0], np.cumsum(deg)])
    from fusedmm_amd import synth
    g = synth.graph_from_rowptr(rows, cols, rowptr, np.concatenate(lists) if deg.sum() else np.zeros(0, np.int64), None, bits)
    g["val"] = synth.edge_values(max(1, g["nnz"]), seed)[:g["nnz"]] if g["nnz"] else np.zeros(1, np.float32)
    if g["nnz"] == 0:
        g["indx"] = np.zeros(1, g["indx"].dtype)
    if rng.random() < 0.4 and g["nnz"] > 0:
        g = graphs.split_pointers(g, seed)
    pad = lambda: int(rng.choice([0, 0, 1, 3, 4]))
    ldx, ldy, ldz = k + pad(), k + pad(), k + pad()
    lo, hi = (0.1, 1.0) if kind in ("fr", "fa", "ll") else (-0.5, 0.5) if tkern == "s" else (-1.0, 1.0)
    X = graphs.features(rows, ldx, seed, lo, hi, 1).astype(np_v)
    # distance tuples with 1/s or sqrt bodies: keep X and Y apart (s > 0); the dot tuple with log2(1+sqrt): s > 0
    far = kind in ("fr", "fa", "ll") and tkern != "s"
    Y = graphs.features(cols, ldy, seed, -hi if far else lo, -lo if far else hi, 2).astype(np_v)
    Z0 = graphs.features(rows, ldz, seed, -1, 1, 3).astype(np_v)
    m = rows if rng.random() < 0.7 else int(rng.integers(0, rows + 1))
    sk = SOP_NAMES[kind] if kind else 0
    where = "device" if rng.random() < 0.7 else "host"
    split = None if rng.random() < 0.5 else (int(rng.integers(1, 40)), int(rng.integers(1, 20)))
    print("case", seed, dict(bits=bits, vbits=vbits, rows=rows, cols=cols, k=k, hub=hub, op=tkern, kind=kind, beta=beta,
                             ld=(ldx, ldy, ldz), m=m, where=where, split=split), flush=True)
    gpu_api.set_kind(sk, bits, vbits)
    if split:
        gpu_api.set_split(split[0], split[1], bits, vbits)
    try:
        rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=bits, where=where, m=m, k=k, ldx=ldx, ldy=ldy,
                            ldz=ldz, vbits=vbits)
    finally:
        gpu_api.set_split(0, 0, bits, vbits)
    assert rc == 0
    o = orc(vbits)
    want = Z0.copy()
    assert 0 == o.opt("t" if tkern == "f" else tkern, g, X, Y, want, beta=beta, sop_kind=sk, mode=1, m=m, k=k, ldx=ldx, ldy=ldy, ldz=ldz)
    # rows >= m and padding columns untouched
    np.testing.assert_array_equal(Z[m:], Z0[m:])
    np.testing.assert_array_equal(Z[:, k:], Z0[:, k:])
    eps = float(np.finfo(np_v).eps)
    scale = float(np.abs(want[:m, :k]).max()) + 1.0 if m else 1.0
    tol = 64 * eps * max(1, hub, 9) * scale
    extra = None
    if kind == "sigmoid":
        gg = dict(g)
        extra_full, _ = checks.sigmoid_flip_slack(o.table().astype(np.float32), gg, X[:, :k].astype(np.float64), Y[:, :k].astype(np.float64), m)
        extra = np.zeros((rows, k))
        extra[:m] = extra_full
    err = np.abs(Z[:, :k].astype(np.float64) - want[:, :k].astype(np.float64))
    bound = tol + (extra if extra is not None else 0.0)
    assert np.all(err <= bound), (float(err.max()), tol)


@pytest.mark.parametrize("seed", range(_N or 32))
def test_random_general_tuple(seed):
    """Any non-UDEF stage combination (plus SOP_UDEF with a device body), through
    the run-time switched kernel, against the oracle's restatement of the
    reference's general pipeline."""
    rng = np.random.default_rng(5000 + seed)
    bits = int(rng.choice([32, 64]))
    vbits = int(rng.choice([32, 64]))
    np_v = np.float32 if vbits == 32 else np.float64
    k = int(rng.choice([3, 8, 20, 64, 96, 130, 256]))
    g = graphs.ragged(bits, seed=seed + 1, rows=int(rng.integers(5, 60)), cols=int(rng.integers(30, 90)),
                      hub_deg=int(rng.choice([10, 200])), hub_rows=(3,))
    vop = int(rng.integers(1, 8))
    rop = int(rng.choice([0x00, 0x10, 0x20, 0x30, 0x40, 0x50]))
    sop, vsc = [(0x100, 0x1000), (0x100, 0x2000), (0xF00, 0x1000), (0x000, 0x0000), (0xF00, 0x2000)][int(rng.integers(0, 5))]
    aop = int(rng.choice([0x10000, 0x20000, 0x30000, 0x00000]))
    imsg = vop | rop | sop | vsc | aop
    X = graphs.features(g["rows"], k, seed, -1, 1, 1).astype(np_v)
    Y = graphs.features(g["cols"], k, seed, -1, 1, 2).astype(np_v)
    Z0 = graphs.features(g["rows"], k, seed, -1, 1, 3).astype(np_v)
    split = None if rng.random() < 0.5 else (6, 5)
    print("case", seed, hex(imsg), dict(bits=bits, vbits=vbits, k=k, split=split), flush=True)
    lib = fa.load(bits, vbits)
    gpu_api.set_kind(SOP_NAMES["tdist"], bits, vbits)
    prev = lib.fusedMM_amd_set_opt(0)
    if split:
        gpu_api.set_split(split[0], split[1], bits, vbits)
    try:
        rc, Z = gpu_api.run(imsg, g, X, Y, Z0, bits=bits, vbits=vbits)
    finally:
        lib.fusedMM_amd_set_opt(prev)
        gpu_api.set_split(0, 0, bits, vbits)
    assert rc == 0
    want = Z0.copy()
    assert orc(vbits).generic(imsg, g, X, Y, want, sop_kind=SOP_NAMES["tdist"]) == 0
    eps = float(np.finfo(np_v).eps)
    tol = 256 * eps * 200 * (float(np.abs(want).max()) + 1.0)
    assert float(np.abs(Z.astype(np.float64) - want.astype(np.float64)).max()) <= tol


def _random_degrees(rng, rows):
    """Row lengths of several characters in one matrix: stretches of Poisson lengths, stretches of empty rows,
    power-law lengths, a few long rows."""
    deg = np.zeros(rows, np.int64)
    i = 0
    while i < rows:
        n = int(rng.integers(1, 40))
        kind = int(rng.integers(0, 5))
        if kind == 0:
            d = rng.poisson(float(rng.choice([2, 8, 16, 30])), n)
        elif kind == 1:
            d = np.zeros(n, np.int64)
        elif kind == 2:
            d = np.minimum(rng.zipf(1.7, n), 300)
        elif kind == 3:
            d = rng.integers(0, 70, n)
        else:
            d = np.full(n, int(rng.choice([1, 8, 9, 16, 32, 33, 64, 65])))
        deg[i:i + n] = d[:rows - i]
        i += n
    for _ in range(int(rng.integers(0, 3))):
        deg[int(rng.integers(0, rows))] = int(rng.choice([150, 700, 3000]))
    return deg


@pytest.mark.parametrize("seed", range(_N or 40))
def test_random_structure_matches_the_mirror_bit_for_bit(seed):
    """Random mixtures of row lengths (which decide what is walked one row per sub-wave, what by the whole wavefront
    and what in segments), widths, strides, thresholds and tuples: the library against the CPU mirror of its
    order of operations, bit for bit."""
    from fusedmm_amd import synth
    rng = np.random.default_rng(9000 + seed)
    bits = int(rng.choice([32, 64]))
    vbits = int(rng.choice([32, 32, 64]))
    np_v, u = (np.float32, np.uint32) if vbits == 32 else (np.float64, np.uint64)
    rows, cols = int(rng.integers(1, 700)), int(rng.integers(1, 400))
    k = int(rng.choice([4, 8, 20, 32, 36, 48, 64, 100, 128, 256, 260, 512]))
    tkern, kind = [("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist"), ("f", "fr")][seed % 5]
    beta = float(rng.choice([0.0, 1.0]))
    deg = _random_degrees(rng, rows)
    rowptr = np.concatenate([[0], np.cumsum(deg)])
    nnz = int(rowptr[-1])
    g = synth.graph_from_rowptr(rows, cols, rowptr, rng.integers(0, cols, max(nnz, 1), dtype=np.int64)[:nnz] if nnz else np.zeros(0, np.int64), None, bits)
    if nnz == 0:
        g["indx"] = np.zeros(1, g["indx"].dtype)
        g["val"] = np.zeros(1, np.float32)
    else:
        g["val"] = synth.edge_values(nnz, seed)
        if rng.random() < 0.3:
            g = graphs.split_pointers(g, seed)
    pad = lambda: 4 * int(rng.choice([0, 0, 1, 2]))              # strides that keep the 16-byte layout
    ldx, ldy, ldz = k + pad(), k + pad(), k + pad()
    lo, hi = (-0.5, 0.5) if tkern in ("s", "g", "m") else (-1.0, 1.0)
    X = graphs.features(rows, ldx, seed, lo, hi, 1).astype(np_v)
    Y = graphs.features(cols, ldy, seed, lo, hi, 2).astype(np_v)
    if tkern == "f":
        Y = (Y + np_v(3.0)).astype(np_v)                          # FR: keep X and Y apart (1/s)
    Z0 = graphs.features(rows, ldz, seed, -1, 1, 3).astype(np_v)
    m = rows if rng.random() < 0.6 else int(rng.integers(0, rows + 1))
    sk = SOP_NAMES[kind] if kind else 0
    split = gpu_api.default_split(k, vbits) if rng.random() < 0.4 else (int(rng.integers(20, 200)), int(rng.integers(8, 64)))
    pack = bool(rng.random() < 0.8)
    # when finished rows are written: as they finish, on a 2.6 us or 82 us clock tick, or only when a wavefront's LDS is full
    tick = int(rng.choice([0, 8, 13, 24]))
    print("case", seed, dict(bits=bits, vbits=vbits, rows=rows, cols=cols, k=k, op=tkern, beta=beta, ld=(ldx, ldy, ldz), m=m,
                             split=split, pack=pack, tick=tick, nnz=nnz), flush=True)
    lib = fa.load(bits, vbits)
    gpu_api.set_kind(sk, bits, vbits)
    gpu_api.set_split(split[0], split[1], bits, vbits)
    prev = lib.fusedMM_amd_set_pack_rows(1 if pack else 0)
    prev_tick = lib.fusedMM_amd_set_store_tick(tick)
    try:
        rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=bits, m=m, k=k, ldx=ldx, ldy=ldy, ldz=ldz, vbits=vbits)
    finally:
        gpu_api.set_split(0, 0, bits, vbits)
        lib.fusedMM_amd_set_pack_rows(prev)
        lib.fusedMM_amd_set_store_tick(prev_tick)
    assert rc == 0
    want = gpu_api.oracle_mirror(orc(vbits), tkern, g, X, Y, Z0, beta, sk, k, split[0], split[1], m=m, pack=pack)
    np.testing.assert_array_equal(Z.view(u), want.view(u))
    np.testing.assert_array_equal(Z[m:], Z0[m:])
    np.testing.assert_array_equal(Z[:, k:], Z0[:, k:])
