"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle."""
import numpy as np
import pytest

import checks
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES, Oracle

pytestmark = pytest.mark.gpu

KINDS = [("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist"), ("f", "fr")]


def _inputs(g, k, tkern, seed=1):
    lo, hi = (-0.5, 0.5) if tkern in ("s", "g", "m") else (-1.0, 1.0)
    X = graphs.features(g["rows"], k, seed, lo, hi, stream=1)
    Y = graphs.features(g["cols"], k, seed, lo, hi, stream=2)
    Z0 = graphs.features(g["rows"], k, seed, -1.0, 1.0, stream=3)
    return X, Y, Z0


def _tol(tkern):
    return (1e-5, 1e-6) if tkern in ("g", "m") else (1e-4, 1e-6)


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("k", [32, 64, 128, 256, 512, 48, 20, 130])
@pytest.mark.parametrize("tkern,kind", KINDS)
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_pattern_ops_match_oracle(oracle, tkern, kind, k, bits, beta):
    """Light rows only (hub below the split threshold): the result must equal the
    oracle's wavefront-order evaluation bit for bit, and sit within tolerance of
    the fp64 evaluation."""
    g = graphs.ragged(bits, hub_deg=60)
    X, Y, Z0 = _inputs(g, k, tkern)
    sk = SOP_NAMES[kind] if kind else 0
    print("case", tkern, k, bits, beta, flush=True)
    gpu_api.set_kind(sk, bits)
    rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=bits)
    assert rc == 0
    ot = "t" if tkern == "f" else tkern
    Zw = gpu_api.oracle_mirror(oracle, tkern, g, X, Y, Z0, beta, sk, k, *gpu_api.default_split(k), vec_ok=(k % 4 == 0))
    np.testing.assert_array_equal(Z.view(np.uint32), Zw.view(np.uint32))
    Z64 = Z0.copy()
    oracle.opt(ot, g, X, Y, Z64, beta=beta, sop_kind=sk, mode=1)
    rtol, atol = _tol(tkern)
    extra = None
    if tkern == "s":
        extra, _ = checks.sigmoid_flip_slack(oracle.table(), g, X, Y)
    checks.assert_close(Z, Z64, rtol, atol, extra, "%s k=%d" % (tkern, k))


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("tkern,kind", KINDS)
def test_host_operands(oracle, tkern, kind, bits):
    """The drop-in call with plain host arrays (staged inside the library)."""
    g = graphs.ragged(bits, hub_deg=60)
    k = 64
    X, Y, Z0 = _inputs(g, k, tkern)
    sk = SOP_NAMES[kind] if kind else 0
    gpu_api.set_kind(sk, bits)
    rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=0.0, bits=bits, where="host")
    assert rc == 0
    Zw = gpu_api.oracle_mirror(oracle, tkern, g, X, Y, Z0, 0.0, sk, k, *gpu_api.default_split(k))
    np.testing.assert_array_equal(Z.view(np.uint32), Zw.view(np.uint32))
