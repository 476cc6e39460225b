"""Double precision (VALUETYPE double, the reference's -DDREAL build):
libfusedmm_amd_d_i{32,64}.so against the double instance of the oracle."""
import os

import numpy as np
import pytest

import checks
import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES, Oracle

pytestmark = pytest.mark.gpu
KINDS = [("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist"), ("f", "fr")]
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def od():
    return Oracle(vbits=64)


@pytest.fixture(autouse=True)
def restore_split():
    yield
    for bits in (32, 64):
        gpu_api.set_split(0, 0, bits, 64)


def feats(n, k, seed, lo, hi, stream):
    return graphs.features(n, k, seed, lo, hi, stream).astype(np.float64)


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("k", [32, 128, 256, 512, 48, 20, 130])
@pytest.mark.parametrize("tkern,kind", KINDS)
def test_double_pattern_ops_match_oracle(od, tkern, kind, k, bits):
    g = graphs.ragged(bits, hub_deg=60)
    lo, hi = (-0.5, 0.5) if tkern in ("s", "g", "m") else (-1.0, 1.0)
    X, Y = feats(g["rows"], k, 1, lo, hi, 1), feats(g["cols"], k, 1, lo, hi, 2)
    Z0 = feats(g["rows"], k, 1, -1, 1, 3)
    sk = SOP_NAMES[kind] if kind else 0
    print("case", tkern, k, bits, flush=True)
    gpu_api.set_kind(sk, bits, 64)
    for beta in (0.0, 1.0):
        rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=bits, vbits=64)
        assert rc == 0
        Zw = gpu_api.oracle_mirror(od, tkern, g, X, Y, Z0, beta, sk, k, *gpu_api.default_split(k, 64), vec_ok=(k % 4 == 0))
        np.testing.assert_array_equal(Z.view(np.uint64), Zw.view(np.uint64))
    # and against the wide (long double) evaluation: double rounding only, no table flips at this size
    Zq = Z0.copy()
    od.opt("t" if tkern == "f" else tkern, g, X, Y, Zq, beta=1.0, sop_kind=sk, mode=1)
    np.testing.assert_allclose(Z, Zq, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("k", [32, 128, 512, 130])
@pytest.mark.parametrize("tkern,kind", [("m", None), ("s", "sigmoid"), ("t", "tdist")])
def test_double_split_rows_match_mirror(od, tkern, kind, k, bits):
    g = graphs.ragged(bits, hub_deg=3000)
    lo, hi = (-0.5, 0.5) if tkern in ("s", "g", "m") else (-1.0, 1.0)
    X, Y = feats(g["rows"], k, 1, lo, hi, 1), feats(g["cols"], k, 1, lo, hi, 2)
    Z0 = feats(g["rows"], k, 1, -1, 1, 3)
    sk = SOP_NAMES[kind] if kind else 0
    gpu_api.set_kind(sk, bits, 64)
    gpu_api.set_split(10, 7, bits, 64)
    rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=1.0, bits=bits, vbits=64)
    assert rc == 0
    assert gpu_api.last_split(bits, 64)[1] > 400
    want = gpu_api.oracle_mirror(od, tkern, g, X, Y, Z0, 1.0, sk, k, 10, 7, vec_ok=(k % 4 == 0))
    np.testing.assert_array_equal(Z.view(np.uint64), want.view(np.uint64))


def test_double_default_split_and_host_operands(od):
    g = graphs.ragged(32, rows=64, cols=5000, hub_deg=20000)
    k = 128
    X, Y = feats(g["rows"], k, 2, -0.5, 0.5, 1), feats(g["cols"], k, 2, -0.5, 0.5, 2)
    Z0 = np.zeros((g["rows"], k))
    gpu_api.set_kind(1, 32, 64)
    heavy_deg, seg_len = gpu_api.default_split(k, 64)
    want = gpu_api.oracle_mirror(od, "s", g, X, Y, Z0, 0.0, 1, k, heavy_deg, seg_len)
    for where in ("device", "host"):
        rc, Z = gpu_api.run(MSG["s"], g, X, Y, Z0, bits=32, vbits=64, where=where)
        assert rc == 0
        assert gpu_api.last_split(32, 64)[:2] == (1, -(-20000 // seg_len))
        np.testing.assert_array_equal(Z.view(np.uint64), want.view(np.uint64))


def test_double_golden_ops_on_gpu(od):
    """The reference's own double-precision outputs (golden fixtures)."""
    d = np.load(os.path.join(GOLD, "ops_d_i32.npz"))
    rows, cols = (int(v) for v in d["ragged_shape"])
    g = {"rows": rows, "cols": cols, "nnz": int(d["ragged_indx"].size), "pntrb": d["ragged_pntrb"],
         "pntre": d["ragged_pntre"], "indx": d["ragged_indx"], "val": d["ragged_val"]}
    k = 24
    X, Y = d["ragged_X%d" % k], d["ragged_Y%d" % k]
    for t, kind in (("s", "sigmoid"), ("t", "tdist"), ("f", "fr"), ("m", None), ("g", None)):
        sk = SOP_NAMES[kind] if kind else 0
        gpu_api.set_kind(sk, 32, 64)
        rc, Z = gpu_api.run(MSG[t], g, X, Y, np.zeros((rows, k)), bits=32, vbits=64)
        assert rc == 0
        want = d["ragged_%s_k%d_fusedmm" % (t, k)]
        extra = checks.sigmoid_flip_slack(od.table(), g, X, Y)[0] if t == "s" else None
        checks.assert_close(Z, want, 1e-11, 1e-12, extra, t)


def test_double_generic_tuples(od):
    g = graphs.ragged(32, rows=23, cols=31, hub_deg=40)
    k = 8
    X, Y = feats(g["rows"], k, 1, -1, 1, 1), feats(g["cols"], k, 1, -1, 1, 2)
    Z0 = feats(g["rows"], k, 1, -1, 1, 3)
    gpu_api.set_kind(SOP_NAMES["tdist"], 32, 64)
    lib = fa.load(32, 64)
    prev = lib.fusedMM_amd_set_opt(0)
    try:
        for imsg in (0x11155, 0x21F32, 0x30044, 0x12121, 0x11F57, 0x21103):
            rc, Z = gpu_api.run(imsg, g, X, Y, Z0, bits=32, vbits=64)
            assert rc == 0, hex(imsg)
            want = Z0.copy()
            assert od.generic(imsg, g, X, Y, want, sop_kind=SOP_NAMES["tdist"]) == 0
            np.testing.assert_allclose(Z, want, rtol=1e-12, atol=1e-12, err_msg=hex(imsg))
    finally:
        lib.fusedMM_amd_set_opt(prev)
