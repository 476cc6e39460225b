"""The CPU oracle against the golden fixtures written by the real reference
(tests/golden/make_golden.py).  Runs without the reference tree."""
import os

import numpy as np

import graphs
import pytest

from oracle_api import MSG, SOP_NAMES

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KIND_OF = {"s": "sigmoid", "t": "tdist", "f": "fr", "m": None, "g": None}


def bits_equal(a, b):
    return np.array_equal(np.asarray(a, np.float32).view(np.uint32), np.asarray(b, np.float32).view(np.uint32))


def graph_from(d, name, bits):
    it = np.int32 if bits == 32 else np.int64
    rows, cols = (int(v) for v in d[name + "_shape"])
    return {"rows": rows, "cols": cols, "nnz": int(d[name + "_indx"].size), "pntrb": d[name + "_pntrb"].astype(it),
            "pntre": d[name + "_pntre"].astype(it), "indx": d[name + "_indx"].astype(it), "val": d[name + "_val"]}


def test_table_and_sop_bodies_bit_equal(oracle):
    d = np.load(os.path.join(GOLD, "sop.npz"))
    assert bits_equal(oracle.table(), d["table"])
    v = d["probe"]
    for kind in ("sigmoid", "tdist", "fr", "ll", "fa"):
        arg = v if kind == "sigmoid" else np.abs(v) + np.float32(1e-3)
        assert bits_equal(oracle.sop(SOP_NAMES[kind], arg), d["sop_" + kind]), kind


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("gname", ["ragged", "er"])
@pytest.mark.parametrize("k", [16, 40])
@pytest.mark.parametrize("t", ["s", "t", "f", "m", "g"])
def test_ops_against_reference(oracle, bits, gname, k, t):
    d = np.load(os.path.join(GOLD, "ops_i%d.npz" % bits))
    g = graph_from(d, gname, bits)
    X, Y = d["%s_X%d" % (gname, k)], d["%s_Y%d" % (gname, k)]
    sk = SOP_NAMES[KIND_OF[t]] if KIND_OF[t] else 0
    want_f = d["%s_%s_k%d_fusedmm" % (gname, t, k)]
    want_t = d["%s_%s_k%d_trusted" % (gname, t, k)]
    # the reference's fusedMM_csr (general pipeline): bit for bit
    Z = np.zeros_like(want_f)
    assert oracle.generic(MSG[t], g, X, Y, Z, sop_kind=sk) == 0
    assert bits_equal(Z, want_f)
    # pattern kernels, sequential fp32: same bits as the general pipeline for these tuples
    ot = "t" if t == "f" else t
    Z = np.zeros_like(want_f)
    assert oracle.opt(ot, g, X, Y, Z, beta=0.0, sop_kind=sk, mode=0) == 0
    assert bits_equal(Z, want_f)
    # fp64 and wavefront-order modes: within the reference's own trusted-vs-test spread
    scale = np.abs(want_t).max() + 1.0
    for mode in (1, 2):
        Z = np.zeros_like(want_f)
        oracle.opt(ot, g, X, Y, Z, beta=0.0, sop_kind=sk, mode=mode, V=4, L=16, S=4)
        # a table-bin flip (sigmoid) shows up as <= 1.3e-3 * |Y|; anything else is rounding
        tol = 2e-3 if t == "s" else 2e-5
        assert np.abs(Z - want_t).max() <= tol * scale, (mode, np.abs(Z - want_t).max())


def test_tuple_sweep_bit_equal(oracle):
    d = np.load(os.path.join(GOLD, "tuples_i32.npz"))
    rows, cols = (int(v) for v in d["shape"])
    g = {"rows": rows, "cols": cols, "nnz": int(d["indx"].size), "pntrb": d["pntrb"], "pntre": d["pntre"],
         "indx": d["indx"], "val": d["val"]}
    for imsg, want in zip(d["msgs"], d["Z"]):
        Z = d["Z0"].copy()
        assert oracle.generic(int(imsg), g, d["X"], d["Y"], Z, sop_kind=SOP_NAMES["tdist"]) == 0
        if (int(imsg) & 0xF00) == 0x000 and (int(imsg) & 0xF000) != 0:
            continue   # SOP_NOOP feeding a VSC reads an uninitialised scalar in the reference
        assert bits_equal(Z, want), hex(int(imsg))


# ---- double precision (the reference's -DDREAL build) ------------------------------------

def bits_equal64(a, b):
    return np.array_equal(np.asarray(a, np.float64).view(np.uint64), np.asarray(b, np.float64).view(np.uint64))


@pytest.fixture(scope="module")
def oracle_d():
    from oracle_api import Oracle
    return Oracle(vbits=64)


def test_double_table_and_sop_bodies_bit_equal(oracle_d):
    d = np.load(os.path.join(GOLD, "sop.npz"))
    assert bits_equal64(oracle_d.table(), d["table_d"])
    v = d["probe_d"]
    for kind in ("sigmoid", "tdist", "fr", "ll", "fa"):
        arg = v if kind == "sigmoid" else np.abs(v) + 1e-3
        assert bits_equal64(oracle_d.sop(SOP_NAMES[kind], arg), d["sop_%s_d" % kind]), kind


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("t", ["s", "t", "f", "m", "g"])
def test_double_ops_against_reference(oracle_d, bits, t):
    d = np.load(os.path.join(GOLD, "ops_d_i%d.npz" % bits))
    g = graph_from(d, "ragged", bits)
    k = 24
    X, Y = d["ragged_X%d" % k], d["ragged_Y%d" % k]
    sk = SOP_NAMES[KIND_OF[t]] if KIND_OF[t] else 0
    want_f = d["ragged_%s_k%d_fusedmm" % (t, k)]
    want_t = d["ragged_%s_k%d_trusted" % (t, k)]
    Z = np.zeros_like(want_f)
    assert oracle_d.generic(MSG[t], g, X, Y, Z, sop_kind=sk) == 0
    assert bits_equal64(Z, want_f)
    ot = "t" if t == "f" else t
    Z = np.zeros_like(want_f)
    assert oracle_d.opt(ot, g, X, Y, Z, beta=0.0, sop_kind=sk, mode=0) == 0
    assert bits_equal64(Z, want_f)
    scale = np.abs(want_t).max() + 1.0
    for mode in (1, 2):
        Z = np.zeros_like(want_f)
        oracle_d.opt(ot, g, X, Y, Z, beta=0.0, sop_kind=sk, mode=mode, V=4, L=8, S=8)
        tol = 2e-3 if t == "s" else 1e-13          # sigmoid: a table-bin flip; otherwise rounding
        assert np.abs(Z - want_t).max() <= tol * scale, (mode, np.abs(Z - want_t).max())


def _rule(deg, nthreads, recompute=True, strict=True, tip_opens_next=True, restart=True):
    """The partition rule with each of its steps switchable, used only to show
    that the golden vectors tell the variants apart (all switches on = the rule
    as the reference has it)."""
    m = len(deg)
    total = int(deg.sum())
    quota = total // nthreads
    own = np.zeros(m, np.int64)
    cur = cum = 0
    tt = 0
    for i in range(m):
        cum += int(deg[i])
        cur += int(deg[i])
        own[i] = tt
        if (cur > quota if strict else cur >= quota) and tt + 1 < nthreads:
            tt += 1
            if tip_opens_next:
                own[i] = tt
            cur = 0 if restart else cur - quota
            if recompute:
                quota = (total - cum) // (nthreads - tt)
    return own


def _partition_golden():
    d = np.load(os.path.join(GOLD, "partition.npz"))
    for name in d["names"]:
        name = str(name)
        yield name, d[name + "_pntrb"], d[name + "_pntre"], int(d[name + "_m"]), \
            {t: d["%s_owner_t%d" % (name, t)].astype(np.int64) for t in (2, 3, 5, 8, 16)}


@pytest.mark.parametrize("bits", [32, 64])
def test_partition_equals_the_reference_row_for_row(oracle, bits):
    """orc_partition_rows against the thread the real reference (fusedMM.c:633-676,
    -DPTTIME -DLOAD_BALANCE -DNTHREADS=t) was seen to evaluate every row on."""
    from oracle_api import owners_from_ranges
    it = np.int32 if bits == 32 else np.int64
    checked = 0
    for name, pb, pe, m, owners in _partition_golden():
        for t, want in owners.items():
            rc, rb, re = oracle.partition(pb.astype(it), pe.astype(it), t, m=m)
            assert rc == 0, (name, t)
            got = owners_from_ranges(rb, re, m)
            assert got.min() >= 0, (name, t, "rows outside every range, or in two")
            seen = want >= 0                       # rows with edges: the reference showed their thread
            assert np.array_equal(got[seen], want[seen]), (name, t)
            # ranges are contiguous and ascending, so rows without edges are pinned wherever
            # they lie strictly between two rows of one thread
            assert np.all(np.diff(got) >= 0), (name, t)
            checked += int(seen.sum())
    assert checked > 40000


def test_partition_vectors_tell_the_rule_from_its_near_misses():
    """Each plausible slip (quota never recomputed, >= for >, the tipping row
    kept by the closing thread, the running count not restarted) disagrees with
    the reference's recorded ownership on some case; the rule itself never does."""
    variants = {"no_recompute": dict(recompute=False), "not_strict": dict(strict=False),
                "tip_stays": dict(tip_opens_next=False), "no_restart": dict(restart=False)}
    wrong = {v: 0 for v in variants}
    for name, pb, pe, m, owners in _partition_golden():
        deg = (pe - pb)[:m]
        for t, want in owners.items():
            seen = want >= 0
            assert np.array_equal(_rule(deg, t)[seen], want[seen]), (name, t)
            for v, kw in variants.items():
                wrong[v] += int(not np.array_equal(_rule(deg, t, **kw)[seen], want[seen]))
    assert all(n > 0 for n in wrong.values()), wrong


def _udef_case(d, bits, npv):
    it = np.int32 if bits == 32 else np.int64
    rows, cols = (int(v) for v in d["shape"])
    g = {"rows": rows, "cols": cols, "nnz": int(d["indx"].size), "pntrb": d["pntrb"].astype(it),
         "pntre": d["pntre"].astype(it), "indx": d["indx"].astype(it), "val": d["val"]}
    return g, d["X"].astype(npv), d["Y"].astype(npv), d["Z0"].astype(npv)


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("vbits", [32, 64])
def test_user_stage_tuples_bit_equal(oracle, oracle_d, bits, vbits):
    """Tuples in which VOP, ROP, VSC or AOP (and SOP) are the caller's functions: the oracle's
    restatement with those functions bound equals, bit for bit, what the real reference built
    with <STAGE>_UDEF_IMPL switched on wrote for the same inputs."""
    d = np.load(os.path.join(GOLD, "udef_stages.npz"))
    o, npv, key = (oracle, np.float32, "Z") if vbits == 32 else (oracle_d, np.float64, "Z_d")
    g, X, Y, Z0 = _udef_case(d, bits, npv)
    assert len(d["msgs"]) >= 60
    for imsg, want in zip(d["msgs"], d[key]):
        Z = Z0.copy()
        assert o.generic_udef(int(imsg), g, X, Y, Z, host_sop=True) == 0, hex(int(imsg))
        np.testing.assert_array_equal(Z.view(np.uint8), want.view(np.uint8), err_msg=hex(int(imsg)))
    # the accumulate stage is what writes Z: without one the call leaves it alone
    i = list(d["msgs"]).index(0xFFFFF & (0xF | 0xF0 | 0xF00 | 0xF000))
    np.testing.assert_array_equal(d[key][i], Z0)


def test_user_stage_without_a_function_is_undefined(oracle):
    """The reference's default build binds stubs that return FUSEDMM_UNDEFINED_USER_FUNCTION
    (fusedMM_internal.h:50-84); the oracle reports that code and leaves Z alone."""
    d = np.load(os.path.join(GOLD, "udef_stages.npz"))
    g, X, Y, Z0 = _udef_case(d, 32, np.float32)
    for imsg in (0x1110F, 0x111F2, 0x1F112, 0xF1112):
        Z = Z0.copy()
        assert oracle.generic(imsg, g, X, Y, Z) == 64
        np.testing.assert_array_equal(Z, Z0)


def same_values(a, b):
    """NaN in the same places, the same bits everywhere else (so a zero's sign counts)."""
    a, b = np.asarray(a), np.asarray(b)
    u = np.uint32 if a.dtype == np.float32 else np.uint64
    na, nb = np.isnan(a), np.isnan(b)
    return a.dtype == b.dtype and np.array_equal(na, nb) and np.array_equal(a.view(u)[~na], b.view(u)[~nb])


@pytest.mark.parametrize("vbits", [32, 64])
def test_max_and_min_stages_on_nan_infinities_and_signed_zeros(oracle, oracle_d, vbits):
    """The reference's fmax / fmin are macros, (x) > (y) ? (x) : (y) and (x) < (y) ? (x) : (y) (fusedMM.c:18-19),
    not the C library's: a NaN on the left loses, on the right wins; of two zeros the right one is kept.  The
    oracle's VOP_MAX / VOP_MIN / AOP_MAX / AOP_MIN against the real reference's output on such operands."""
    d = np.load(os.path.join(GOLD, "special_values.npz"))
    multi, single, X, Y, Z0, msgs = graphs.special_values_case(32)
    o, npv, sfx = (oracle, np.float32, "") if vbits == 32 else (oracle_d, np.float64, "_d")
    assert np.array_equal(msgs, d["msgs"]) and np.isnan(X).any() and np.signbit(Y[Y == 0]).any()
    seen_nan = seen_negzero = 0
    for gname, g in (("multi", multi), ("single", single)):
        for imsg, want in zip(msgs, d["Z_%s%s" % (gname, sfx)]):
            Z = Z0.astype(npv)
            assert o.generic(int(imsg), g, X.astype(npv), Y.astype(npv), Z) == 0
            assert same_values(Z, want), (gname, hex(int(imsg)))
            seen_nan += int(np.isnan(want).sum())
            seen_negzero += int((np.signbit(want) & (want == 0)).sum())
    assert seen_nan > 100 and seen_negzero > 20
    # the C library's fmax / fmin would differ on these operands (it never returns the NaN of a pair)
    a, b = np.float32(1.0), np.float32(np.nan)
    assert np.isnan(a if a > b else b) and not np.isnan(np.fmax(a, b))
