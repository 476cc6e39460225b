"""Live cross-check of the CPU oracle against the real reference, compiled from
/root/reference by `make -C oracle ref`.  Skipped where that build is absent."""
import numpy as np
import pytest

import graphs
from oracle_api import MSG, SOP_NAMES, Ref, ref_available

pytestmark = pytest.mark.skipif(not ref_available(), reason="oracle/_ref not built (needs /root/reference)")
KIND_OF = {"s": "sigmoid", "t": "tdist", "f": "fr", "m": "spmm", "g": "gcn"}


def bits_equal(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_table_bits(oracle):
    assert bits_equal(oracle.table(), Ref("sigmoid").table())


@pytest.mark.parametrize("kind", ["sigmoid", "tdist", "fr", "ll", "fa"])
def test_sop_bodies_bits(oracle, kind):
    rng = np.random.default_rng(3)
    v = rng.uniform(-6, 6, 100000).astype(np.float32)
    edges = (np.arange(2049) * 10.0 / 2048 - 5.0).astype(np.float32)
    v = np.concatenate([v, edges, np.nextafter(edges, np.float32(9)), np.nextafter(edges, np.float32(-9))])
    v = v[v != np.float32(5.0)]       # the reference indexes one past its table there
    if kind != "sigmoid":
        v = np.abs(v) + np.float32(1e-4)
    assert bits_equal(oracle.sop(SOP_NAMES[kind], v), Ref(kind).sop(v))


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("t", ["s", "t", "f", "m", "g"])
@pytest.mark.parametrize("k", [8, 33, 128])
def test_generic_path_bits(oracle, bits, t, k):
    kind = KIND_OF[t]
    r = Ref(kind, bits)
    sk = SOP_NAMES.get(kind, 0)
    for g in (graphs.ragged(bits), graphs.with_values(graphs.tiny_er(300, 2500, 4, bits))):
        X = graphs.features(g["rows"], k, 1, -1, 1, 1)
        Y = graphs.features(g["cols"], k, 1, -1, 1, 2)
        Z0 = graphs.features(g["rows"], k, 1, -1, 1, 3)
        A, B = Z0.copy(), Z0.copy()
        r.test(t, g, X, Y, A)
        assert oracle.generic(MSG[t], g, X, Y, B, sop_kind=sk) == 0
        assert bits_equal(A, B)
        # m < rows
        A, B = Z0.copy(), Z0.copy()
        r.test(t, g, X, Y, A, m=g["rows"] // 2)
        oracle.generic(MSG[t], g, X, Y, B, sop_kind=sk, m=g["rows"] // 2)
        assert bits_equal(A, B)


@pytest.mark.skipif(not ref_available("sigmoid", 32, 64), reason="double-precision reference not built")
@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("t", ["s", "t", "f", "m", "g"])
def test_double_generic_path_bits(bits, t):
    from oracle_api import Oracle
    od = Oracle(vbits=64)
    kind = KIND_OF[t]
    r = Ref(kind, bits, 64)
    sk = SOP_NAMES.get(kind, 0)
    g = graphs.with_values(graphs.tiny_er(300, 2500, 4, bits))
    for k in (8, 33):
        X = graphs.features(g["rows"], k, 1, -1, 1, 1).astype(np.float64)
        Y = graphs.features(g["cols"], k, 1, -1, 1, 2).astype(np.float64)
        Z0 = graphs.features(g["rows"], k, 1, -1, 1, 3).astype(np.float64)
        A, B = Z0.copy(), Z0.copy()
        r.test(t, g, X, Y, A)
        assert od.generic(MSG[t], g, X, Y, B, sop_kind=sk) == 0
        assert np.array_equal(A.view(np.uint64), B.view(np.uint64))
    assert np.array_equal(od.table().view(np.uint64), Ref("sigmoid", bits, 64).table().view(np.uint64))


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("nthreads", [2, 3, 5, 8, 16])
def test_partition_rows_live(oracle, bits, nthreads):
    """orc_partition_rows against the thread the real reference (fusedMM.c:633-676 built
    with -DPTTIME -DLOAD_BALANCE -DNTHREADS=n) is seen to evaluate each row on, for
    fresh random skewed degree sets."""
    from oracle_api import RefPartition, owners_from_ranges, ref_partition_available
    if not ref_partition_available(nthreads, bits):
        pytest.skip("oracle/_ref partition probe not built")
    it = np.int32 if bits == 32 else np.int64
    ref = RefPartition(nthreads, bits)
    rng = np.random.default_rng(100 * nthreads + bits)
    for rep in range(24):
        n = int(rng.integers(1, 3000))
        deg = np.minimum(rng.zipf(1.3 + 0.1 * (rep % 8), n), int(rng.integers(1, 1500)))
        deg[rng.random(n) < 0.1 * (rep % 5)] = 0
        ptr = np.concatenate([[0], np.cumsum(deg)]).astype(it)
        m = n if rep % 3 else max(1, n // 2)
        want, _ = ref.owners(ptr[:-1], ptr[1:], m)
        rc, rb, re = oracle.partition(ptr[:-1], ptr[1:], nthreads, m=m)
        assert rc == 0
        got = owners_from_ranges(rb, re, m)
        seen = want >= 0
        assert got.min() >= 0 and np.array_equal(got[seen], want[seen]), (rep, n, m)


@pytest.mark.parametrize("bits,vbits", [(32, 32), (64, 32), (32, 64), (64, 64)])
def test_user_stage_tuples_live(bits, vbits):
    """Every tuple with a user stage (1344 of them: all built-in neighbours, every precision
    and index width) through the real reference built with <STAGE>_UDEF_IMPL switched on and
    through the oracle's restatement bound to the same caller-side functions: same status,
    same bits.  (SOP_NOOP with a scaling stage is left out: the reference passes an
    uninitialised scalar there, fusedMM.c:212-216.)"""
    import itertools
    from oracle_api import Oracle, RefUdef, ref_udef_available
    if not ref_udef_available(bits, vbits):
        pytest.skip("oracle/_ref/libref_udefstages not built")
    npv = np.float32 if vbits == 32 else np.float64
    o, r = Oracle(vbits=vbits), RefUdef(bits, vbits)
    g = graphs.with_values(graphs.ragged(bits, seed=17, hub_deg=70))
    k = 20
    X = graphs.features(g["rows"], k, 5, -0.5, 0.5, 1).astype(npv)
    Y = graphs.features(g["cols"], k, 5, -0.5, 0.5, 2).astype(npv)
    Z0 = graphs.features(g["rows"], k, 5, -1, 1, 3).astype(npv)
    n = 0
    for v, rp, sp, vs, ap in itertools.product((1, 2, 3, 4, 5, 6, 7, 0xF), (0x00, 0x10, 0x20, 0x30, 0x40, 0x50, 0xF0),
                                               (0x000, 0x100, 0xF00), (0x0000, 0x1000, 0x2000, 0xF000),
                                               (0x00000, 0x10000, 0x20000, 0x30000, 0xF0000)):
        if not (v == 0xF or rp == 0xF0 or vs == 0xF000 or ap == 0xF0000) or (sp == 0x000 and vs != 0x0000):
            continue
        msg = v | rp | sp | vs | ap
        za, zb = Z0.copy(), Z0.copy()
        assert r.fusedMM_csr(msg, g, X, Y, za) == o.generic_udef(msg, g, X, Y, zb, host_sop=True) == 0, hex(msg)
        assert np.array_equal(za.view(np.uint8), zb.view(np.uint8)), hex(msg)
        n += 1
    assert n == 1344


@pytest.mark.parametrize("vbits", [32, 64])
def test_max_min_on_special_values_live(vbits):
    """Fresh operands with NaN, infinities and signed zeros through the real reference's general pipeline and
    the oracle's: NaN for NaN, bit for bit elsewhere (the committed vectors are tests/golden/special_values.npz)."""
    from oracle_api import Oracle, Ref, ref_available
    if not ref_available("tdist", 32, vbits):
        pytest.skip("oracle/_ref not built")
    npv, u = (np.float32, np.uint32) if vbits == 32 else (np.float64, np.uint64)
    o, r = Oracle(vbits=vbits), Ref("tdist", 32, vbits)
    for seed in (41, 42, 43):
        multi, single, X, Y, Z0, msgs = graphs.special_values_case(32, seed)
        for g in (multi, single):
            for imsg in msgs:
                Za, Zb = Z0.astype(npv), Z0.astype(npv)
                assert o.generic(int(imsg), g, X.astype(npv), Y.astype(npv), Za) == 0
                assert r.fusedMM_csr(int(imsg), g, X.astype(npv), Y.astype(npv), Zb) == 0
                na, nb = np.isnan(Za), np.isnan(Zb)
                assert np.array_equal(na, nb) and np.array_equal(Za.view(u)[~na], Zb.view(u)[~nb]), (seed, hex(int(imsg)))
