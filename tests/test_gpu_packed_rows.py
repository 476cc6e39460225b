"""Short rows walked one per sub-wave (K <= 64): which rows are taken that way follows a rule on the row
pointers alone, the CPU mirror applies the same rule and sums such a row in one accumulator, and the results
must agree bit for bit; switched off, the same call must give the plain wavefront order's bits."""
import numpy as np
import pytest

import checks
import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES, Oracle

pytestmark = pytest.mark.gpu

KINDS = [("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist"), ("f", "fr")]


def _inputs(g, k, tkern, seed=1, npv=np.float32):
    lo, hi = (-0.5, 0.5) if tkern in ("s", "g", "m") else (-1.0, 1.0)
    X = graphs.features(g["rows"], k, seed, lo, hi, stream=1).astype(npv)
    Y = graphs.features(g["cols"], k, seed, lo, hi, stream=2).astype(npv)
    Z0 = graphs.features(g["rows"], k, seed, -1.0, 1.0, stream=3).astype(npv)
    return X, Y, Z0


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("k", [32, 64, 48, 20, 8])
@pytest.mark.parametrize("tkern,kind", KINDS)
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_packed_rows_match_the_mirror(tkern, kind, k, bits, beta):
    oracle = Oracle()
    g = graphs.boundary_graph(bits)
    X, Y, Z0 = _inputs(g, k, tkern)
    sk = SOP_NAMES[kind] if kind else 0
    print("case", tkern, k, bits, beta, flush=True)
    gpu_api.set_kind(sk, bits)
    heavy_deg, seg_len = gpu_api.default_split(k)
    m = g["rows"] - 1                                       # the last row stays out: m is not a multiple of the group
    rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=bits, m=m)
    assert rc == 0
    want = gpu_api.oracle_mirror(oracle, tkern, g, X, Y, Z0, beta, sk, k, heavy_deg, seg_len, m=m)
    assert gpu_api.packed_rows(g, m, k, 32, heavy_deg).sum() > 100
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))
    np.testing.assert_array_equal(Z[m:], Z0[m:])            # the row past m is untouched
    # and within tolerance of the double-precision evaluation, like any other row
    ot = "t" if tkern == "f" else tkern
    Z64 = Z0.copy()
    oracle.opt(ot, g, X, Y, Z64, beta=beta, sop_kind=sk, mode=1, m=m)
    extra = checks.sigmoid_flip_slack(oracle.table(), g, X, Y)[0] if tkern == "s" else None
    rtol = 1e-5 if tkern in ("g", "m") else 1e-4
    checks.assert_close(Z[:m], Z64[:m], rtol, 1e-6, None if extra is None else extra[:m], "%s k=%d" % (tkern, k))


@pytest.mark.parametrize("k", [32, 64])
def test_switched_off_gives_the_plain_wavefront_order(k):
    """fusedMM_amd_set_pack_rows(0): every row is walked by the whole wavefront again (the mirror with
    pack=False); switched back on, the packed bits return.  The two differ in rounding only."""
    oracle = Oracle()
    g = graphs.boundary_graph()
    X, Y, Z0 = _inputs(g, k, "t")
    gpu_api.set_kind(SOP_NAMES["tdist"], 32)
    lib = fa.load(32)
    split = gpu_api.default_split(k)
    try:
        assert lib.fusedMM_amd_set_pack_rows(0) == 1
        rc, Zoff = gpu_api.run(MSG["t"], g, X, Y, Z0)
        assert rc == 0
        want = gpu_api.oracle_mirror(oracle, "t", g, X, Y, Z0, 0.0, 2, k, *split, pack=False)
        np.testing.assert_array_equal(Zoff.view(np.uint32), want.view(np.uint32))
    finally:
        assert lib.fusedMM_amd_set_pack_rows(1) == 0
    rc, Zon = gpu_api.run(MSG["t"], g, X, Y, Z0)
    assert rc == 0
    want = gpu_api.oracle_mirror(oracle, "t", g, X, Y, Z0, 0.0, 2, k, *split)
    np.testing.assert_array_equal(Zon.view(np.uint32), want.view(np.uint32))
    assert (Zon.view(np.uint32) != Zoff.view(np.uint32)).any()          # the order of summation did change
    np.testing.assert_allclose(Zon, Zoff, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("tkern,kind", [("m", None), ("s", "sigmoid"), ("t", "tdist")])
def test_packed_rows_in_double_precision(tkern, kind, bits):
    od = Oracle(vbits=64)
    g = graphs.boundary_graph(bits)
    k = 32
    X, Y, Z0 = _inputs(g, k, tkern, npv=np.float64)
    sk = SOP_NAMES[kind] if kind else 0
    gpu_api.set_kind(sk, bits, 64)
    for beta in (0.0, 1.0):
        rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=bits, vbits=64)
        assert rc == 0
        want = gpu_api.oracle_mirror(od, tkern, g, X, Y, Z0, beta, sk, k, *gpu_api.default_split(k, 64))
        np.testing.assert_array_equal(Z.view(np.uint64), want.view(np.uint64))
    assert 0 < gpu_api.packed_rows(g, g["rows"], k, 64, 4096).sum() < gpu_api.packed_rows(g, g["rows"], k, 32, 4096).sum()


def test_general_pipeline_over_packed_rows():
    """Tuples that match no optimised kernel take the same walk; they are held to the reference's general
    pipeline (the oracle's restatement of it, bit-equal to the real one) within rounding."""
    oracle = Oracle()
    g = graphs.boundary_graph()
    k = 32
    X, Y, Z0 = _inputs(g, k, "t")
    gpu_api.set_kind(SOP_NAMES["tdist"], 32)
    for imsg in (fa.VOP_SUBR | fa.ROP_NORMR | fa.SOP_UDEF | fa.VSC_MUL | fa.AOP_MAX,
                 fa.VOP_ADD | fa.ROP_DOT | fa.SOP_COPY | fa.VSC_ADD | fa.AOP_ADD,
                 fa.VOP_MIN | fa.ROP_ADD_RHS | fa.SOP_COPY | fa.VSC_MUL | fa.AOP_MIN,
                 fa.VOP_COPY_LHS | fa.ROP_NOOP | fa.SOP_COPY | fa.VSC_MUL | fa.AOP_ADD,
                 fa.VOP_COPY_RHS | fa.ROP_NOOP | fa.SOP_NOOP | fa.VSC_NOOP | fa.AOP_NOOP):
        rc, Z = gpu_api.run(imsg, g, X, Y, Z0, beta=0.0)
        assert rc == 0
        want = Z0.copy()
        assert oracle.generic(imsg, g, X, Y, want, sop_kind=2) == 0
        np.testing.assert_allclose(Z, want, rtol=3e-5, atol=3e-5, err_msg=hex(imsg))


def test_noalloc_entry_point_packs_the_same_rows():
    import torch
    g = graphs.boundary_graph()
    k = 32
    X, Y, Z0 = _inputs(g, k, "s")
    lib = fa.load(32)
    lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_SIGMOID)
    assert lib.fusedMM_amd_init_noalloc() == 0
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    d = [t(g["val"]), t(g["indx"]), t(g["pntrb"]), t(g["pntre"]), t(X), t(Y)]
    Za, Zb = t(Z0), t(Z0)
    st = torch.cuda.current_stream().cuda_stream
    args = lambda Z: (fa.MSG_SIGMOID, g["rows"], g["cols"], k, 1.0, g["nnz"], g["rows"], g["cols"], d[0], d[1], d[2], d[3],
                      d[4], k, d[5], k, 1.0, Z, k)
    assert fa.fusedMM_csr(*args(Za), stream=st) == 0
    assert fa.fusedMM_csr(*args(Zb), stream=st, noalloc=True) == 0
    torch.cuda.synchronize()
    assert torch.equal(Za, Zb)
    want = gpu_api.oracle_mirror(Oracle(), "s", g, X, Y, Z0, 1.0, 1, k, *gpu_api.default_split(k))
    np.testing.assert_array_equal(Zb.cpu().numpy().view(np.uint32), want.view(np.uint32))
