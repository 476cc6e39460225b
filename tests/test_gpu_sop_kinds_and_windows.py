"""The plain t-distribution weight 1/(1+s) as a device SOP body (the benchmark list's wording of the t-dist op;
the reference's tester has the same weight times -2), and host-function stages over a window of rows that lies
high in the CSR arrays (their per-edge buffers cover the window's edge slots, indexed from its first one)."""
import ctypes as C

import numpy as np
import pytest

import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, Oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits,vbits", [(32, 32), (64, 32), (32, 64)])
@pytest.mark.parametrize("k", [32, 64, 128, 40])
def test_plain_tdist_body_on_the_device(k, bits, vbits):
    npv = np.float32 if vbits == 32 else np.float64
    ubits = np.uint32 if vbits == 32 else np.uint64
    o = Oracle(vbits=vbits)
    g = graphs.ragged(bits, hub_deg=700)
    X = graphs.features(g["rows"], k, 3, -1, 1, 1).astype(npv)
    Y = graphs.features(g["cols"], k, 3, -1, 1, 2).astype(npv)
    Z0 = graphs.features(g["rows"], k, 3, -1, 1, 3).astype(npv)
    split = (40, 16)
    gpu_api.set_split(*split, bits, vbits)
    try:
        assert gpu_api.set_kind(fa.SOP_KIND_TDIST_PLAIN, bits, vbits) >= -1
        rc, Zp = gpu_api.run(MSG["t"], g, X, Y, Z0, beta=0.0, bits=bits, vbits=vbits)
        assert rc == 0 and gpu_api.last_split(bits, vbits)[1] > 0          # the hub row went through segments
        want = gpu_api.oracle_mirror(o, "t", g, X, Y, Z0, 0.0, fa.SOP_KIND_TDIST_PLAIN, k, *split, vec_ok=(k % 4 == 0))
        np.testing.assert_array_equal(Zp.view(ubits), want.view(ubits))
        # the tester's t-dist body is -2 times this weight, and a factor of -2 is exact through every fused
        # multiply-add and every sum: the two ops' results differ by exactly that factor
        gpu_api.set_kind(fa.SOP_KIND_TDIST, bits, vbits)
        rc, Zt = gpu_api.run(MSG["t"], g, X, Y, Z0, beta=0.0, bits=bits, vbits=vbits)
        assert rc == 0
        # (+ 0: the empty rows' zeros come out of the multiplication with the other sign)
        np.testing.assert_array_equal((npv(-2) * Zp + npv(0)).view(ubits), (Zt + npv(0)).view(ubits))
        # closed form in double precision from the definition
        deg = (g["pntre"] - g["pntrb"]).astype(np.int64)
        Zd = np.zeros((g["rows"], k))
        for i in np.nonzero(deg)[0][:40]:
            cols = g["indx"][g["pntrb"][i]:g["pntre"][i]]
            d = X[i].astype(np.float64) - Y[cols].astype(np.float64)
            Zd[i] = (d / (1.0 + (d * d).sum(1))[:, None]).sum(0)
            np.testing.assert_allclose(Zp[i], Zd[i], rtol=1e-4, atol=1e-5)
        # identical embeddings: weight 1, difference 0
        gpu_api.set_kind(fa.SOP_KIND_TDIST_PLAIN, bits, vbits)
        E = np.tile(X[:1], (max(g["rows"], g["cols"]), 1))
        rc, Z = gpu_api.run(MSG["t"], g, E[:g["rows"]], E[:g["cols"]], Z0, beta=0.0, bits=bits, vbits=vbits)
        assert rc == 0 and not Z.any()
    finally:
        gpu_api.set_split(0, 0, bits, vbits)


def test_plain_tdist_device_body_equals_the_same_weight_as_a_host_function():
    """What a caller of the reference would write as SOP_UDEF_FUNC, (VALUETYPE)(1.0 / (1.0 + val)), evaluated on
    the host between the GPU passes, against the device body: same per-edge scalars; the host-function path
    multiplies then adds where the fused kernel fuses, so rounding-level differences only."""
    g = graphs.ragged(32, hub_deg=90)
    k = 64
    X = graphs.features(g["rows"], k, 4, -1, 1, 1)
    Y = graphs.features(g["cols"], k, 4, -1, 1, 2)
    Z0 = graphs.features(g["rows"], k, 4, -1, 1, 3)
    lib = fa.load(32)
    SOPFN = C.CFUNCTYPE(C.c_int, C.c_float, C.POINTER(C.c_float))

    def sop(val, out):
        out[0] = 1.0 / (1.0 + float(val))
        return 0

    cb = SOPFN(sop)
    try:
        lib.fusedMM_amd_set_sop_callback(C.cast(cb, C.c_void_p))
        lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_HOST)
        rc, Zh = gpu_api.run(MSG["t"], g, X, Y, Z0, beta=1.0)
        assert rc == 0
        lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_TDIST_PLAIN)
        rc, Zd = gpu_api.run(MSG["t"], g, X, Y, Z0, beta=1.0)
        assert rc == 0
        np.testing.assert_allclose(Zd, Zh, rtol=2e-6, atol=2e-6)
        assert np.abs(Zd - Z0).max() > 0.1
    finally:
        lib.fusedMM_amd_set_sop_callback(None)


@pytest.mark.parametrize("where", ["device", "host"])
def test_host_function_stages_over_a_window_high_in_the_arrays(where):
    """Rows [lo, hi) of a larger matrix, passed as the reference's API allows (pntrb + lo, pntre + lo, X + lo*ldx,
    Z + lo*ldz, m = hi - lo): edge slots start far from zero.  A tuple with user stages and the host SOP_UDEF
    path must give those rows exactly what the whole-matrix call gives them."""
    o = Oracle()
    g = graphs.with_values(graphs.ragged(32, rows=300, cols=200, hub_deg=120, hub_rows=(11, 250)))
    k = 12
    X = graphs.features(g["rows"], k, 5, -1, 1, 1)
    Y = graphs.features(g["cols"], k, 5, -1, 1, 2)
    Z0 = graphs.features(g["rows"], k, 5, -1, 1, 3)
    lo, hi = 232, 296      # whole groups of 8 rows: which short rows share a wavefront is decided per such group
    assert g["pntrb"][lo] > 0.5 * g["nnz"]
    sub = dict(g)
    sub.update(rows=hi - lo, pntrb=np.ascontiguousarray(g["pntrb"][lo:hi]), pntre=np.ascontiguousarray(g["pntre"][lo:hi]))
    lib = fa.load(32)
    ptr = lambda st: o.stage_fn(st, 32)
    lib.fusedMM_amd_set_stage_callbacks(ptr("VOP"), ptr("ROP"), ptr("VSC"), ptr("AOP"))
    lib.fusedMM_amd_set_sop_callback(ptr("SOP"))
    lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_HOST)
    try:
        for imsg in (0xF | 0xF0 | 0xF00 | 0xF000 | 0xF0000, 0x5 | 0x50 | 0xF00 | 0x1000 | 0xF0000,
                     0xF | 0x10 | 0x100 | 0x2000 | 0x20000, MSG["t"], MSG["s"]):
            rc, Zfull = gpu_api.run(imsg, g, X, Y, Z0, beta=1.0, where=where)
            assert rc == 0, hex(imsg)
            rc, Zwin = gpu_api.run(imsg, sub, X[lo:hi], Y, Z0[lo:hi], beta=1.0, where=where)
            assert rc == 0, hex(imsg)
            np.testing.assert_array_equal(Zwin.view(np.uint32), Zfull[lo:hi].view(np.uint32), err_msg=hex(imsg))
            if imsg not in (MSG["t"], MSG["s"]):
                want = Z0.copy()
                assert o.generic_udef(imsg, g, X, Y, want, host_sop=True) == 0
                np.testing.assert_array_equal(Zfull.view(np.uint32), want.view(np.uint32), err_msg=hex(imsg))
    finally:
        lib.fusedMM_amd_set_stage_callbacks(None, None, None, None)
        lib.fusedMM_amd_set_sop_callback(None)
