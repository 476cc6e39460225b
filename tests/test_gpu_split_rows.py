"""Heavy rows: split into edge segments, partials merged in a fixed order."""
import numpy as np
import pytest

import checks
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES

pytestmark = pytest.mark.gpu
KINDS = [("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist"), ("f", "fr")]


@pytest.fixture(autouse=True)
def restore_split():
    yield
    for bits in (32, 64):
        gpu_api.set_split(0, 0, bits)


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("k", [32, 128, 512, 48, 130])
@pytest.mark.parametrize("tkern,kind", KINDS)
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_split_rows_match_mirror(oracle, tkern, kind, k, bits, beta):
    """Forced low thresholds: most rows of the ragged graph become heavy, the hub
    has hundreds of segments.  Result equals the oracle's mirror of the split
    evaluation bit for bit, twice in a row."""
    g = graphs.ragged(bits, hub_deg=3000)
    lo, hi = (-0.5, 0.5) if tkern in ("s", "g", "m") else (-1.0, 1.0)
    X = graphs.features(g["rows"], k, 1, lo, hi, 1)
    Y = graphs.features(g["cols"], k, 1, lo, hi, 2)
    Z0 = graphs.features(g["rows"], k, 1, -1, 1, 3)
    sk = SOP_NAMES[kind] if kind else 0
    heavy_deg, seg_len = 10, 7
    print("case", tkern, k, bits, beta, flush=True)
    gpu_api.set_kind(sk, bits)
    gpu_api.set_split(heavy_deg, seg_len, bits)
    rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=bits)
    assert rc == 0
    h, s, o = gpu_api.last_split(bits)
    deg = g["pntre"] - g["pntrb"]
    assert h == int((deg > heavy_deg).sum()) and o == 0
    assert s == int(np.ceil(deg[deg > heavy_deg] / seg_len).sum())       # no row here exceeds 512 segments
    want = gpu_api.oracle_mirror(oracle, tkern, g, X, Y, Z0, beta, sk, k, heavy_deg, seg_len, vec_ok=(k % 4 == 0))
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))
    rc, Z2 = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=bits)
    np.testing.assert_array_equal(Z.view(np.uint32), Z2.view(np.uint32))      # same bits on every run
    # and within tolerance of the fp64 evaluation (degree-scaled: a 3000-edge fp32 sum)
    Z64 = Z0.copy()
    ot = "t" if tkern == "f" else tkern
    es = np.zeros(int(g["pntre"].max()), np.float32)
    oracle.opt(ot, g, X, Y, Z64, beta=beta, sop_kind=sk, mode=1, edge_s=es if kind else None)
    rows, slots = checks.edge_rows(g)
    d_abs = np.ones(slots.size) if tkern == "g" else (np.abs(g["val"][slots]) if tkern == "m" else
                                                      np.abs(oracle.sop(sk, es[slots])).astype(np.float64))
    extra = 4 * checks.EPS32 * np.sqrt(np.maximum(deg, 1))[:, None] * checks.abs_term_sum(tkern, g, X, Y, d_abs)
    if tkern == "s":
        extra = extra + checks.sigmoid_flip_slack(oracle.table(), g, X, Y)[0]
    rtol, atol = (1e-5, 1e-6) if tkern in ("g", "m") else (1e-4, 1e-6)
    checks.assert_close(Z, Z64, rtol, atol, extra, "%s k=%d" % (tkern, k))


@pytest.mark.parametrize("tkern,kind", [("m", None), ("s", "sigmoid")])
def test_default_thresholds_hub_row(oracle, tkern, kind):
    """Library defaults: one 40 000-edge hub among short rows."""
    bits, k = 32, 128
    g = graphs.ragged(bits, rows=64, cols=5000, hub_deg=40000)
    X = graphs.features(g["rows"], k, 2, -0.5, 0.5, 1)
    Y = graphs.features(g["cols"], k, 2, -0.5, 0.5, 2)
    Z0 = np.zeros((g["rows"], k), np.float32)
    sk = SOP_NAMES[kind] if kind else 0
    gpu_api.set_kind(sk, bits)
    rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, bits=bits)
    assert rc == 0
    heavy_deg, seg_len = gpu_api.default_split(k)
    h, s, o = gpu_api.last_split(bits)
    assert (h, s, o) == (1, -(-40000 // seg_len), 0)                   # 79 segments of 512 edges
    want = gpu_api.oracle_mirror(oracle, tkern, g, X, Y, Z0, 0.0, sk, k, heavy_deg, seg_len)
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))


def test_queue_overflow_is_handled_inline(oracle):
    """A caller-supplied nnz that is far too small undersizes the segment queue:
    rows that do not fit are processed whole in the row phase; the answer stays right."""
    bits, k = 32, 64
    g = graphs.ragged(bits, rows=40, cols=3000, hub_deg=2000, hub_rows=(11, 13, 17))
    Y = graphs.features(g["cols"], k, 3, -0.5, 0.5, 2)
    Z0 = np.zeros((g["rows"], k), np.float32)
    gpu_api.set_split(8, 4, bits)              # 3 hubs x 500 segments + the short rows > 1024
    rc, Z = gpu_api.run(MSG["m"], g, None, Y, Z0, bits=bits, nnz=1)   # queue capacity falls to its floor (1024)
    assert rc == 0
    h, s, o = gpu_api.last_split(bits)
    assert o >= 1
    Z64 = Z0.copy()
    oracle.opt("m", g, None, Y, Z64, mode=1)
    deg = (g["pntre"] - g["pntrb"])
    rows, slots = checks.edge_rows(g)
    extra = 4 * checks.EPS32 * np.sqrt(np.maximum(deg, 1))[:, None] * \
        checks.abs_term_sum("m", g, None, Y, np.abs(g["val"][slots]).astype(np.float64))
    checks.assert_close(Z, Z64, 1e-5, 1e-6, extra, "overflow")


def test_very_long_row_gets_longer_segments(oracle):
    """A row that would need more than 512 segments is cut into 512-at-most longer ones."""
    bits, k = 32, 64
    g = graphs.ragged(bits, rows=30, cols=4000, hub_deg=40000)
    Y = graphs.features(g["cols"], k, 2, -0.5, 0.5, 2)
    Z0 = graphs.features(g["rows"], k, 2, -1, 1, 3)
    gpu_api.set_split(16, 8, bits)
    rc, Z = gpu_api.run(MSG["m"], g, None, Y, Z0, beta=1.0, bits=bits)
    assert rc == 0
    deg = (g["pntre"] - g["pntrb"]).astype(np.int64)
    others = deg[(deg > 16) & (deg < 40000)]
    h, s, o = gpu_api.last_split(bits)
    assert o == 0 and s == int(np.ceil(others / 8).sum()) + -(-40000 // -(-40000 // 512))
    want = gpu_api.oracle_mirror(oracle, "m", g, None, Y, Z0, 1.0, 0, k, 16, 8)
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))
