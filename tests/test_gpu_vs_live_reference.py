"""The GPU path side by side with the REAL reference (its general fusedMM_csr and
its tester's trusted kernels, compiled from the reference tree into oracle/_ref)
on the same seeded inputs.  Skipped where that build is absent."""
import numpy as np
import pytest

import checks
import gpu_api
import graphs
from fusedmm_amd import synth
from oracle_api import MSG, SOP_NAMES, Oracle, Ref, ref_available

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not ref_available("sigmoid", 32), reason="oracle/_ref not built (needs the reference tree)")]
KINDS = [("s", "sigmoid"), ("t", "tdist"), ("f", "fr"), ("m", "spmm"), ("g", "gcn")]


@pytest.mark.parametrize("vbits", [32, 64])
@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("tkern,kind", KINDS)
def test_gpu_equals_reference_within_tolerance(tkern, kind, bits, vbits):
    if not ref_available(kind, bits, vbits):
        pytest.skip("this reference variant is not built")
    np_v = np.float32 if vbits == 32 else np.float64
    n, k = 20000, 128
    g = synth.er_graph(n, 8 * n, 21, bits)
    g["val"] = synth.edge_values(g["nnz"], 21)
    lo, hi = (-0.5, 0.5) if tkern == "s" else (-1.0, 1.0)
    X = synth.uniform_matrix(n, k, lo, hi, 21, 1).astype(np_v)
    Y = synth.uniform_matrix(n, k, lo, hi, 21, 2).astype(np_v)
    Z0 = np.zeros((n, k), np_v)
    sk = SOP_NAMES.get(kind, 0)
    r = Ref(kind, bits, vbits)
    Zref = Z0.copy()
    r.test(tkern, g, X, Y, Zref)                      # the reference's fusedMM_csr (general pipeline)
    Ztru = Z0.copy()
    r.trusted(tkern, g, X, Y, Ztru)                   # its tester's trusted kernel
    gpu_api.set_kind(sk, bits, vbits)
    rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=0.0, bits=bits, vbits=vbits)
    assert rc == 0
    if vbits == 32:
        rtol, atol = (1e-5, 1e-6) if tkern in ("g", "m") else (1e-4, 1e-6)
        deg_term = 32 * checks.EPS32            # both sides are fp32 sums of ~16 terms of size <= 1
    else:
        rtol, atol, deg_term = 1e-12, 1e-13, 0.0
    extra = deg_term
    if tkern == "s":   # an edge whose dot sits on a table-bin boundary may take the neighbouring entry
        extra = extra + checks.sigmoid_flip_slack(Oracle(vbits=vbits).table().astype(np.float32), g, X, Y)[0]
    checks.assert_close(Z, Zref, rtol, atol, extra, "vs reference fusedMM_csr")
    checks.assert_close(Z, Ztru, rtol, atol, extra, "vs reference trusted kernel")
