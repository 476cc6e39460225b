"""SOP_UDEF served by the caller's host function (the reference's binding,
fusedMM.h:139): GPU reduce pass -> host function per edge -> GPU accumulate pass."""
import ctypes as C
import math

import numpy as np
import pytest

import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, SOP_SIGMOID

pytestmark = pytest.mark.gpu
SOPFN = C.CFUNCTYPE(C.c_int, C.c_float, C.POINTER(C.c_float))


@pytest.fixture
def host_kind():
    libs = [fa.load(32), fa.load(64)]
    prev = [l.fusedMM_amd_set_sop_kind(fa.SOP_KIND_HOST) for l in libs]
    yield
    for l, p in zip(libs, prev):
        l.fusedMM_amd_set_sop_kind(p)
        l.fusedMM_amd_set_sop_callback(None)


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("where", ["device", "host"])
def test_host_sigmoid_callback_equals_device_body(oracle, host_kind, bits, where):
    g = graphs.ragged(bits, hub_deg=300)
    k = 64
    X = graphs.features(g["rows"], k, 1, -0.5, 0.5, 1)
    Y = graphs.features(g["cols"], k, 1, -0.5, 0.5, 2)
    Z0 = graphs.features(g["rows"], k, 1, -1, 1, 3)
    table = oracle.table()

    def sop(val, out):     # the reference tester's sigmoid body (test/fusedMMtime.cpp:628-632)
        if val > 5.0:
            t = 1.0
        elif val < -5.0:
            t = 0.0
        else:
            t = float(table[min(2047, int((val + 5.0) * 2048 / 10.0))])
        out[0] = 1.0 - t
        return 0

    cb = SOPFN(sop)
    lib = fa.load(bits)
    lib.fusedMM_amd_set_sop_callback(C.cast(cb, C.c_void_p))
    for beta in (0.0, 1.0):
        rc, Z = gpu_api.run(MSG["s"], g, X, Y, Z0, beta=beta, bits=bits, where=where)
        assert rc == 0
        want = Z0.copy()
        oracle.opt("s", g, X, Y, want, beta=beta, sop_kind=SOP_SIGMOID, mode=2, V=4, L=16, S=4)
        # same per-edge scalars (same wavefront order, same table bins); the accumulate pass
        # multiplies then adds where the fused kernel uses fma: rounding-level differences only
        np.testing.assert_allclose(Z, want, rtol=2e-6, atol=2e-6)


def test_arbitrary_user_function(oracle, host_kind):
    """A SOP no built-in body covers: d = tanh(s) on the t-dist tuple."""
    g = graphs.tiny_er(120, 500, 3)
    k = 24
    X = graphs.features(120, k, 2, -1, 1, 1)
    Y = graphs.features(120, k, 2, -1, 1, 2)

    def sop(val, out):
        out[0] = math.tanh(val)
        return 0

    cb = SOPFN(sop)
    fa.load(32).fusedMM_amd_set_sop_callback(C.cast(cb, C.c_void_p))
    rc, Z = gpu_api.run(MSG["t"], g, X, Y, np.zeros((120, k), np.float32), beta=0.0)
    assert rc == 0
    want = np.zeros((120, k))
    for i in range(120):
        for j in range(g["pntrb"][i], g["pntre"][i]):
            d = X[i].astype(np.float64) - Y[g["indx"][j]].astype(np.float64)
            want[i] += math.tanh(float(np.float32(d @ d))) * d
    np.testing.assert_allclose(Z, want, rtol=1e-4, atol=1e-5)


def test_no_host_function_is_reported(host_kind):
    g = graphs.tiny_er(20, 40, 3)
    X = graphs.features(20, 8, 2)
    rc, _ = gpu_api.run(MSG["s"], g, X, X, np.zeros((20, 8), np.float32))
    assert rc == fa.UNDEFINED_USER_FUNCTION       # python has no SOP_UDEF_FUNC symbol and none was registered
