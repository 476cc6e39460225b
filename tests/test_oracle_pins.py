"""Pins the CPU oracle against what the mathematics fixes: closed forms,
library routines (scipy CSR @ dense), dense brute force in fp64, invariants.
A dropped term, a wrong sign or a transposed operand fails one of these."""
import numpy as np
import pytest
import scipy.sparse as sp

import graphs
from oracle_api import MSG, SOP_FR, SOP_SIGMOID, SOP_TDIST, SOP_LL, SOP_FA, SOP_TDIST_PLAIN


def _csr_matrix(g, pattern=False):
    rows, cols = g["rows"], g["cols"]
    deg = (g["pntre"] - g["pntrb"]).astype(np.int64)
    rid = np.repeat(np.arange(rows), deg)
    slots = np.concatenate([np.arange(b, e) for b, e in zip(g["pntrb"], g["pntre"])]) if rows else np.empty(0, int)
    v = np.ones(slots.size) if pattern else g["val"][slots].astype(np.float64)
    return sp.csr_matrix((v, (rid, g["indx"][slots])), shape=(rows, cols))  # duplicates are summed


def test_table_closed_forms(oracle):
    t = oracle.table()
    assert t.dtype == np.float32 and t.shape == (2048,)
    assert t[1024] == np.float32(0.5)                       # sigma(0)
    x = (np.arange(2048) * 10.0 / 2048 - 5.0)
    np.testing.assert_allclose(t, 1.0 / (1.0 + np.exp(-x)), rtol=3e-7)
    assert np.all(np.diff(t) > 0)                            # strictly increasing
    np.testing.assert_allclose(t[1:] + t[1:][::-1], 1.0, atol=2e-7)  # sigma(x) + sigma(-x) = 1


def test_sigmoid_bin_rule(oracle):
    assert oracle.bin(0.0) == 1024
    assert oracle.bin(-5.0) == 0
    assert oracle.bin(5.0) == 2047                           # clamped (reference reads one past the end)
    assert oracle.bin(5.0000005) == 2048 and oracle.bin(-5.0000005) == -1
    # floor indexing: just below a bin edge stays in the lower bin
    edge = np.float32(10.0 * 1100 / 2048 - 5.0)
    assert oracle.bin(float(edge)) in (1099, 1100)
    assert oracle.bin(float(np.nextafter(edge, np.float32(9)))) == 1100
    assert oracle.bin(float(np.nextafter(np.nextafter(edge, np.float32(-9)), np.float32(-9)))) == 1099


def test_sop_bodies_closed_forms(oracle):
    s = np.array([0.25, 1.0, 3.0, 100.0], np.float32)
    np.testing.assert_allclose(oracle.sop(SOP_FR, s), 1.0 + 1.0 / s.astype(np.float64), rtol=1e-7)
    np.testing.assert_allclose(oracle.sop(SOP_TDIST, s), -2.0 / (1.0 + s.astype(np.float64)), rtol=1e-7)
    np.testing.assert_allclose(oracle.sop(SOP_LL, s), np.log2(1 + np.sqrt(s.astype(np.float64))), rtol=3e-7)
    np.testing.assert_allclose(oracle.sop(SOP_FA, s), np.sqrt(s.astype(np.float64)) + 1.0 / s, rtol=3e-7)
    v = np.array([-7.0, -5.5, 0.0, 5.5, 7.0], np.float32)
    np.testing.assert_array_equal(oracle.sop(SOP_SIGMOID, v), np.array([1, 1, 0.5, 0, 0], np.float32))
    assert np.isinf(oracle.sop(SOP_FR, np.zeros(1, np.float32))[0])      # s == 0: 1 + 1/0


@pytest.mark.parametrize("bits", [32, 64])
def test_spmm_gcn_equal_scipy(oracle, bits):
    g = graphs.ragged(bits)
    k = 24
    Y = graphs.features(g["cols"], k, 2)
    A = _csr_matrix(g)
    for mode in (0, 1, 2):
        Z = np.zeros((g["rows"], k), np.float32)
        oracle.opt("m", g, None, Y, Z, mode=mode, V=4, L=8, S=8)
        np.testing.assert_allclose(Z, A @ Y.astype(np.float64), rtol=2e-5, atol=2e-5)
        Z = np.zeros((g["rows"], k), np.float32)
        oracle.opt("g", g, None, Y, Z, mode=mode, V=4, L=8, S=8)
        np.testing.assert_allclose(Z, _csr_matrix(g, True) @ Y.astype(np.float64), rtol=2e-5, atol=2e-5)
    # Y = 1  =>  Z[i,:] = degree (gcn) / sum of edge values (spmm)
    ones = np.ones((g["cols"], k), np.float32)
    Z = np.zeros((g["rows"], k), np.float32)
    oracle.opt("g", g, None, ones, Z)
    np.testing.assert_array_equal(Z[:, 0], (g["pntre"] - g["pntrb"]).astype(np.float32))
    # generic pipeline with the same tuples agrees with the pattern kernels
    Zg = np.zeros((g["rows"], k), np.float32)
    assert oracle.generic(MSG["m"], g, None, Y, Zg) == 0
    Zo = np.zeros((g["rows"], k), np.float32)
    oracle.opt("m", g, None, Y, Zo, beta=1.0)
    np.testing.assert_array_equal(Zg, Zo)


def _dense_brute(tkern, kind, table, g, X, Y):
    """fp64 evaluation from the definition, edge by edge in Python."""
    Z = np.zeros((g["rows"], Y.shape[1]))
    X64, Y64 = X.astype(np.float64), Y.astype(np.float64)
    for i in range(g["rows"]):
        for j in range(g["pntrb"][i], g["pntre"][i]):
            c = g["indx"][j]
            if tkern == "s":
                s = np.float32(X64[i] @ Y64[c])
                if s > 5:
                    sig = 1.0
                elif s < -5:
                    sig = 0.0
                else:
                    sig = float(table[min(2047, int((float(s) + 5.0) * 2048 / 10.0))])
                Z[i] += (1.0 - sig) * Y64[c]
            else:
                d = X64[i] - Y64[c]
                s = float(np.float32(d @ d))
                w = {"tdist": max(-5.0, min(5.0, -2.0 / (1.0 + s))), "fr": 1.0 + 1.0 / s, "tdist_plain": 1.0 / (1.0 + s)}[kind]
                Z[i] += w * d
    return Z


@pytest.mark.parametrize("tkern,kind,sk", [("s", "sigmoid", SOP_SIGMOID), ("t", "tdist", SOP_TDIST), ("t", "fr", SOP_FR),
                                           ("t", "tdist_plain", SOP_TDIST_PLAIN)])
def test_embedding_ops_equal_dense_brute_force(oracle, tkern, kind, sk):
    g = graphs.tiny_er(60, 200, seed=5)
    k = 16
    X = graphs.features(g["rows"], k, 1, -1, 1)
    Y = graphs.features(g["cols"], k, 2, -1, 1, stream=2)
    want = _dense_brute(tkern, kind, oracle.table(), g, X, Y)
    for mode, tol in ((1, 2e-6), (0, 3e-5), (2, 3e-5)):
        Z = np.zeros((g["rows"], k), np.float32)
        assert oracle.opt(tkern, g, X, Y, Z, sop_kind=sk, mode=mode, V=4, L=8, S=8) == 0
        # a table-bin flip between summation orders would show as ~1e-3: none at this size/seed
        np.testing.assert_allclose(Z, want, rtol=tol, atol=tol)


def test_sigmoid_special_cases(oracle):
    g = graphs.tiny_er(80, 300, seed=6)
    k = 8
    Y = graphs.features(g["cols"], k, 2)
    # X = 0 => every dot is 0 => table[1024] = 0.5 => Z = 0.5 * A_pattern * Y
    Z = np.zeros((g["rows"], k), np.float32)
    oracle.opt("s", g, np.zeros((g["rows"], k), np.float32), Y, Z, sop_kind=SOP_SIGMOID)
    np.testing.assert_allclose(Z, 0.5 * (_csr_matrix(g, True) @ Y.astype(np.float64)), rtol=1e-5, atol=1e-6)
    # dots far above +5 contribute nothing; far below -5 contribute Y[c] exactly
    Ybig = np.abs(Y) + 1.0
    Xpos = np.full((g["rows"], k), 10.0, np.float32)
    Z = np.zeros((g["rows"], k), np.float32)
    oracle.opt("s", g, Xpos, Ybig, Z, sop_kind=SOP_SIGMOID)
    assert not Z.any()
    Z = np.zeros((g["rows"], k), np.float32)
    oracle.opt("s", g, -Xpos, Ybig, Z, sop_kind=SOP_SIGMOID)
    np.testing.assert_allclose(Z, _csr_matrix(g, True) @ Ybig.astype(np.float64), rtol=1e-5)


@pytest.mark.parametrize("vbits", [32, 64])
def test_plain_tdist_weight_is_pinned_by_its_closed_form_and_by_the_harness_body(vbits):
    """1/(1+s), the t-distribution weight as written in the benchmark list; no body of the reference's tester
    computes it.  Exact values on arguments where 1/(1+s) is a power of two; the exact relation -2 * plain ==
    the tester's t-dist body (bit for bit: scaling by a power of two commutes with the one rounding, and the
    body's clamp to [-5, 5] never binds for s >= 0); monotone, in (0, 1]; a plausible slip (1/s, 1/(1+s)^2,
    a missing 1, float instead of double arithmetic) fails one of these."""
    from oracle_api import Oracle
    o = Oracle(vbits=vbits)
    npv = np.float32 if vbits == 32 else np.float64
    s = np.array([0.0, 1.0, 3.0, 7.0, 1023.0, 0.5, 0.25], npv)
    np.testing.assert_array_equal(o.sop(SOP_TDIST_PLAIN, s), np.array([1, 0.5, 0.25, 0.125, 1.0 / 1024, 1 / 1.5, 0.8], npv))
    rng = np.random.Generator(np.random.Philox(key=[4, 4]))
    v = np.concatenate([rng.uniform(0, 40, 5000), rng.uniform(0, 1e-3, 500), 10.0 ** rng.uniform(2, 30, 500)]).astype(npv)
    plain, body = o.sop(SOP_TDIST_PLAIN, v), o.sop(SOP_TDIST, v)
    np.testing.assert_array_equal((npv(-2) * plain).view(np.uint32 if vbits == 32 else np.uint64),
                                  body.view(np.uint32 if vbits == 32 else np.uint64))
    assert (plain > 0).all() and (plain <= 1).all()
    order = np.argsort(v, kind="stable")
    assert (np.diff(plain[order]) <= 0).all()
    # one rounding of the double-precision quotient (what the tester's conventions give), not float arithmetic
    want = (1.0 / (1.0 + v.astype(np.float64))).astype(npv)
    np.testing.assert_array_equal(plain, want)


def test_plain_tdist_identical_rows_contribute_nothing(oracle):
    g = graphs.tiny_er(40, 100, seed=7)
    k = 8
    Y = np.tile(graphs.features(1, k, 3), (g["cols"], 1))
    Z = np.zeros((g["rows"], k), np.float32)
    oracle.opt("t", g, Y.copy(), Y, Z, sop_kind=SOP_TDIST_PLAIN)
    assert not Z.any()                                         # weight 1, difference 0
    # and the whole op is -1/2 of the tester's t-dist op, term by term (mode 0: multiply and add rounded
    # separately, so the factor -2 stays exact through every step)
    X = graphs.features(g["rows"], k, 5, -1, 1)
    Yr = graphs.features(g["cols"], k, 6, -1, 1, stream=2)
    Za, Zb = np.zeros((g["rows"], k), np.float32), np.zeros((g["rows"], k), np.float32)
    oracle.opt("t", g, X, Yr, Za, sop_kind=SOP_TDIST_PLAIN)
    oracle.opt("t", g, X, Yr, Zb, sop_kind=SOP_TDIST)
    np.testing.assert_array_equal((np.float32(-2) * Za).view(np.uint32), Zb.view(np.uint32))


def test_tdist_identical_rows_and_fr_nan(oracle):
    g = graphs.tiny_er(40, 100, seed=7)
    k = 8
    Y = np.tile(graphs.features(1, k, 3), (g["cols"], 1))      # all embeddings equal
    Z = np.zeros((g["rows"], k), np.float32)
    oracle.opt("t", g, Y.copy(), Y, Z, sop_kind=SOP_TDIST)
    assert not Z.any()                                         # X[i] == Y[c] => zero contribution
    Z = np.zeros((g["rows"], k), np.float32)
    oracle.opt("t", g, Y.copy(), Y, Z, sop_kind=SOP_FR)
    deg = g["pntre"] - g["pntrb"]
    assert np.isnan(Z[deg > 0]).all() and not np.isnan(Z[deg == 0]).any()   # inf * 0


@pytest.mark.parametrize("bits", [32, 64])
def test_invariants(oracle, bits):
    g = graphs.ragged(bits)
    k = 12
    X = graphs.features(g["rows"], k, 1)
    Y = graphs.features(g["cols"], k, 2)
    Z0 = graphs.features(g["rows"], k, 3)
    # beta == 0 on a pre-filled Z  ==  beta != 0 on a zeroed Z   (optimised write-back rule)
    A = Z0.copy()
    oracle.opt("s", g, X, Y, A, beta=0.0, sop_kind=SOP_SIGMOID)
    B = np.zeros_like(Z0)
    oracle.opt("s", g, X, Y, B, beta=1.0, sop_kind=SOP_SIGMOID)
    np.testing.assert_array_equal(A, B)
    assert not A[0].any() and not A[5].any()                  # empty rows are overwritten with zeros
    # beta != 0 accumulates; the general pipeline always accumulates
    Cc = Z0.copy()
    oracle.opt("m", g, X, Y, Cc, beta=0.5)
    D = Z0.copy()
    oracle.generic(MSG["m"], g, X, Y, D, beta=0.0)
    np.testing.assert_array_equal(Cc, D)
    # m < rows touches only the first m rows
    E = Z0.copy()
    oracle.opt("g", g, X, Y, E, beta=0.0, m=10)
    np.testing.assert_array_equal(E[10:], Z0[10:])
    # split pointers (pntre[i] != pntrb[i+1]) give the same answer
    gs = graphs.split_pointers(g)
    F = np.zeros_like(Z0)
    oracle.opt("m", gs, X, Y, F)
    G = np.zeros_like(Z0)
    oracle.opt("m", g, X, Y, G)
    np.testing.assert_array_equal(F, G)
    # int32 and int64 builds agree bit for bit
    g2 = graphs.ragged(96 - bits)
    H = np.zeros_like(Z0)
    oracle.opt("m", g2, X, Y, H)
    np.testing.assert_array_equal(G, H)
    # linearity in Y for spmm
    Y2 = graphs.features(g["cols"], k, 8)
    P = np.zeros_like(Z0); Q = np.zeros_like(Z0); R = np.zeros_like(Z0)
    oracle.opt("m", g, X, Y, P, mode=1); oracle.opt("m", g, X, Y2, Q, mode=1)
    oracle.opt("m", g, X, (Y + Y2).astype(np.float32), R, mode=1)
    np.testing.assert_allclose(R, P + Q, rtol=1e-5, atol=1e-5)


def test_wavefront_order_dot(oracle):
    rng = np.random.default_rng(4)
    # small integers: every product and partial sum is exact, so any order gives the same bits,
    # and a wrong lane map (an element used twice or skipped) changes the value
    for k, V, L in [(128, 4, 32), (512, 4, 64), (32, 4, 8), (48, 4, 16), (130, 1, 64), (20, 1, 64), (2048, 4, 64)]:
        x = rng.integers(-8, 9, k).astype(np.float32)
        y = rng.integers(-8, 9, k).astype(np.float32)
        assert oracle.gpu_dot(x, y, V, L) == float(np.dot(x.astype(np.float64), y.astype(np.float64)))
        assert oracle.gpu_dot(x, y, V, L, diff=1) == float(((x - y).astype(np.float64) ** 2).sum())
        xr = rng.uniform(-1, 1, k).astype(np.float32)
        yr = rng.uniform(-1, 1, k).astype(np.float32)
        exact = float(np.dot(xr.astype(np.float64), yr.astype(np.float64)))
        bound = k * np.finfo(np.float32).eps * float(np.abs(xr.astype(np.float64) * yr).sum())
        assert abs(oracle.gpu_dot(xr, yr, V, L) - exact) <= bound


def test_generic_stage_codes(oracle):
    g = graphs.tiny_er(20, 30, seed=2)
    k = 4
    X = graphs.features(20, k, 1); Y = graphs.features(20, k, 2); Z = np.zeros((20, k), np.float32)
    assert oracle.generic(0x11100, g, X, Y, Z) == 2            # VOP_NOOP is rejected
    assert oracle.generic(0x11108, g, X, Y, Z) == 2            # unknown VOP
    assert oracle.generic(0x11162, g, X, Y, Z) == 4            # unknown ROP
    assert oracle.generic(0x11202, g, X, Y, Z) == 16           # unknown SOP
    assert oracle.generic(0x13102, g, X, Y, Z) == 32           # unknown VSC
    assert oracle.generic(0x41102, g, X, Y, Z) == 8            # unknown AOP
    assert not Z.any()


def test_generic_tuples_equal_numpy(oracle):
    """A sweep of non-pattern tuples against a direct numpy statement of the five stages."""
    g = graphs.ragged(32, rows=23, cols=31, hub_deg=40)
    k = 6
    X = graphs.features(g["rows"], k, 1, -1, 1)
    Y = graphs.features(g["cols"], k, 2, -1, 1)
    vops = {1: lambda x, y: x, 2: lambda x, y: y, 3: lambda x, y: x + y, 4: lambda x, y: -x + y,
            5: lambda x, y: x - y, 6: np.maximum, 7: np.minimum}
    rops = {0x00: None, 0x10: lambda x, t: (x * t).sum(), 0x20: lambda x, t: x.sum(), 0x30: lambda x, t: t.sum(),
            0x40: lambda x, t: (x * x).sum(), 0x50: lambda x, t: (t * t).sum()}
    for vop, rop, sop, vsc, aop in [(5, 0x50, 0x100, 0x1000, 0x10000), (3, 0x10, 0x100, 0x2000, 0x20000),
                                    (4, 0x30, 0x000, 0x0000, 0x30000), (1, 0x20, 0x100, 0x1000, 0x10000),
                                    (6, 0x40, 0xF00, 0x1000, 0x10000), (7, 0x00, 0x100, 0x2000, 0x10000),
                                    (2, 0x10, 0x100, 0x1000, 0x00000)]:
        imsg = vop | rop | sop | vsc | aop
        Z0 = graphs.features(g["rows"], k, 5)
        Z = Z0.copy()
        assert oracle.generic(imsg, g, X, Y, Z, sop_kind=SOP_TDIST) == 0
        W = Z0.astype(np.float64)
        for i in range(g["rows"]):
            for j in range(g["pntrb"][i], g["pntre"][i]):
                x, y = X[i].astype(np.float64), Y[g["indx"][j]].astype(np.float64)
                t = vops[vop](x, y)
                s = float(g["val"][j]) if rops[rop] is None else rops[rop](x, t)
                d = max(-5.0, min(5.0, -2.0 / (1.0 + float(np.float32(s))))) if sop == 0xF00 else s
                if vsc == 0x1000: t = d * t
                elif vsc == 0x2000: t = d + t
                if aop == 0x10000: W[i] += t
                elif aop == 0x20000: W[i] = np.maximum(W[i], t)
                elif aop == 0x30000: W[i] = np.minimum(W[i], t)
        np.testing.assert_allclose(Z, W, rtol=2e-5, atol=2e-5, err_msg=hex(imsg))


def test_gpu_bin_expression_is_equivalent_for_every_float(oracle):
    """The kernels index the sigmoid table with one double multiply instead of
    the reference's multiply-then-divide.  Proven equal by visiting every float
    in [-5, 5]."""
    import ctypes as C
    seen = C.c_int64()
    oracle.lib.orc_count_bin_formula_mismatches.restype = C.c_int64
    bad = oracle.lib.orc_count_bin_formula_mismatches(C.byref(seen))
    assert seen.value == 2168455170
    assert bad == 0


def test_partition_hand_example_and_properties(oracle):
    """nnz-balanced contiguous row ranges (reference fusedMM.c:633-676).  The row
    that tips the running count over the quota OPENS the next thread's range."""
    deg = np.array([3, 1, 1, 1, 3, 1], np.int32)
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    rc, rb, re = oracle.partition(ptr[:-1], ptr[1:], 2)
    # Mnnz = 10, quota 5: running counts 3,4,5,6 -> row 3 is the first to exceed it
    assert rc == 0 and rb.tolist() == [0, 3] and re.tolist() == [3, 6]
    # three threads: quota 3; row 1 tips (4 > 3) -> thread 1 starts at 1 with quota (10-4)/2 = 3;
    # running 1,2,5 -> row 4 tips -> thread 2 starts at 4
    rc, rb, re = oracle.partition(ptr[:-1], ptr[1:], 3)
    assert rb.tolist() == [0, 1, 4] and re.tolist() == [1, 4, 6]
    # properties on random skewed degrees: ranges tile [0, m) in order, nobody is far over the mean
    rng = np.random.default_rng(1)
    for nthreads in (2, 7, 16):
        deg = np.minimum(rng.zipf(1.6, 5000), 400).astype(np.int64)
        ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
        rc, rb, re = oracle.partition(ptr[:-1], ptr[1:], nthreads)
        assert rc == 0 and rb[0] == 0
        used = [(b, e) for b, e in zip(rb, re) if e >= 0]
        assert used[-1][1] == 5000
        for (b0, e0), (b1, e1) in zip(used, used[1:]):
            assert e0 == b1 and b0 <= e0
        loads = [int(ptr[e] - ptr[b]) for b, e in used]
        assert max(loads) <= ptr[-1] / nthreads + 2 * 400 + ptr[-1] / nthreads * 0.5


@pytest.mark.parametrize("t,sk", [("s", SOP_SIGMOID), ("t", SOP_TDIST), ("m", 0), ("g", 0)])
def test_cpu_baseline_agrees_with_the_fp64_evaluation(t, sk):
    """The function bench.py times as its CPU leg (vectorised, thread-partitioned)."""
    from oracle_api import Oracle
    fast, ref = Oracle(fast=True), Oracle()
    g = graphs.with_values(graphs.tiny_er(500, 4000, 9))
    k = 64
    X = graphs.features(500, k, 1, -0.3, 0.3, 1)
    Y = graphs.features(500, k, 1, -0.3, 0.3, 2)
    for threads in (1, 3, 8):
        Z = graphs.features(500, k, 1, -1, 1, 3)
        assert fast.baseline(t, g, X, Y, Z, 0.0, sk, threads) == 0
        want = np.zeros((500, k), np.float32)
        ref.opt(t, g, X, Y, want, beta=0.0, sop_kind=sk, mode=1)
        tol = 2e-3 if t == "s" else 2e-5              # sigmoid: a table-bin flip between summation orders
        np.testing.assert_allclose(Z, want, rtol=tol, atol=tol)
