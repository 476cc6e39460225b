"""Op tuples in which VOP, ROP, VSC or AOP is the caller's host function.  The library's
own stages of such a tuple run on the GPU in the reference's order, the caller's
functions on the host, so the result is held to the reference's bits: the golden Z of
the real reference built with those stages switched on, and the oracle's restatement."""
import ctypes as C
import os

import numpy as np
import pytest

import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import Oracle

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _register(o, bits, vbits, which=("VOP", "ROP", "VSC", "AOP"), sop=True):
    lib = fa.load(bits, vbits)
    ptr = lambda st: o.stage_fn(st, bits) if st in which else C.c_void_p(None)
    lib.fusedMM_amd_set_stage_callbacks(ptr("VOP"), ptr("ROP"), ptr("VSC"), ptr("AOP"))
    lib.fusedMM_amd_set_sop_callback(o.stage_fn("SOP", bits) if sop else None)
    lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_HOST)          # SOP_UDEF through the host function
    return lib


def _unregister(lib):
    lib.fusedMM_amd_set_stage_callbacks(None, None, None, None)
    lib.fusedMM_amd_set_sop_callback(None)


def _case(d, bits, npv):
    it = np.int32 if bits == 32 else np.int64
    rows, cols = (int(v) for v in d["shape"])
    g = {"rows": rows, "cols": cols, "nnz": int(d["indx"].size), "pntrb": d["pntrb"].astype(it),
         "pntre": d["pntre"].astype(it), "indx": d["indx"].astype(it), "val": d["val"]}
    return g, d["X"].astype(npv), d["Y"].astype(npv), d["Z0"].astype(npv)


@pytest.mark.parametrize("where", ["device", "host"])
@pytest.mark.parametrize("bits,vbits", [(32, 32), (64, 32), (32, 64), (64, 64)])
def test_user_stage_tuples_equal_the_reference(where, bits, vbits):
    d = np.load(os.path.join(GOLD, "udef_stages.npz"))
    npv, key = (np.float32, "Z") if vbits == 32 else (np.float64, "Z_d")
    o = Oracle(vbits=vbits)
    g, X, Y, Z0 = _case(d, bits, npv)
    lib = _register(o, bits, vbits)
    try:
        for imsg, want in zip(d["msgs"], d[key]):
            imsg = int(imsg)
            print("tuple", hex(imsg), where, bits, vbits, flush=True)
            rc, Z = gpu_api.run(imsg, g, X, Y, Z0, bits=bits, vbits=vbits, where=where)
            assert rc == 0, hex(imsg)
            np.testing.assert_array_equal(Z.view(np.uint8), want.view(np.uint8), err_msg=hex(imsg))
    finally:
        _unregister(lib)


def test_user_stages_on_a_ragged_graph_with_a_device_sop_body():
    """m < rows, rows with gaps between pntre and the next pntrb, leading dimensions larger
    than k, a hub row, and SOP_UDEF as a device body between two host stages."""
    o = Oracle()
    g = graphs.split_pointers(graphs.with_values(graphs.ragged(32, rows=150, cols=400, hub_deg=700)))
    k, ldx, ldy, ldz, m = 20, 24, 28, 32, 131
    X = graphs.features(g["rows"], ldx, 3, -0.5, 0.5, 1)
    Y = graphs.features(g["cols"], ldy, 3, -0.5, 0.5, 2)
    Z0 = graphs.features(g["rows"], ldz, 3, -1, 1, 3)
    lib = _register(o, 32, 32, sop=False)
    try:
        lib.fusedMM_amd_set_sop_kind(2)      # t-dist body on the device
        for imsg in (0xF | 0x50 | 0xF00 | 0xF000 | 0x10000, 0x5 | 0xF0 | 0xF00 | 0x1000 | 0xF0000,
                     0x3 | 0x10 | 0xF00 | 0xF000 | 0x20000):
            for where in ("device", "host"):
                rc, Z = gpu_api.run(imsg, g, X, Y, Z0, bits=32, where=where, m=m, k=k, ldx=ldx, ldy=ldy, ldz=ldz)
                assert rc == 0
                want = Z0.copy()
                assert o.generic_udef(imsg, g, X, Y, want, sop_kind=2, m=m, k=k, ldx=ldx, ldy=ldy, ldz=ldz) == 0
                np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32), err_msg="%s %s" % (hex(imsg), where))
                np.testing.assert_array_equal(Z[m:], Z0[m:])             # rows beyond m untouched
                np.testing.assert_array_equal(Z[:, k:], Z0[:, k:])       # columns beyond k untouched
    finally:
        lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_HOST)
        _unregister(lib)


def test_a_user_stage_without_a_function_is_undefined():
    """No function registered and none defined in the process: the code of the reference's
    stubs (fusedMM_internal.h:50-84), Z untouched; with only some registered, the tuples
    that need the others still fail; the stream entry point cannot serve them."""
    import torch
    o = Oracle()
    d = np.load(os.path.join(GOLD, "udef_stages.npz"))
    g, X, Y, Z0 = _case(d, 32, np.float32)
    lib = fa.load(32)
    _unregister(lib)
    for imsg in (0x1110F, 0x111F2, 0x1F112, 0xF1112):
        for where in ("device", "host"):
            rc, Z = gpu_api.run(imsg, g, X, Y, Z0, where=where)
            assert rc == fa.UNDEFINED_USER_FUNCTION
            np.testing.assert_array_equal(Z, Z0)
    lib = _register(o, 32, 32, which=("VOP",))
    try:
        rc, Z = gpu_api.run(0x1110F, g, X, Y, Z0)
        want = Z0.copy()
        assert rc == 0 and o.generic_udef(0x1110F, g, X, Y, want) == 0
        np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))
        assert gpu_api.run(0x111FF, g, X, Y, Z0)[0] == fa.UNDEFINED_USER_FUNCTION      # ROP_UDEF has no function
        t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
        Zd = t(Z0)
        rc = fa.fusedMM_csr(0x1110F, g["rows"], g["cols"], X.shape[1], 1.0, g["nnz"], g["rows"], g["cols"], t(g["val"]),
                            t(g["indx"]), t(g["pntrb"]), t(g["pntre"]), t(X), X.shape[1], t(Y), Y.shape[1], 0.0, Zd,
                            Z0.shape[1], stream=torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert rc == fa.UNDEFINED_USER_FUNCTION and np.array_equal(Zd.cpu().numpy(), Z0)
    finally:
        _unregister(lib)
