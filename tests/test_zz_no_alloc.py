"""fusedMM_csr_stream_noalloc, the entry point whose work queues live in a static
device array: same bits as fusedMM_csr_stream, call after call on one GPU, the
second call smaller than the first (the array keeps the first call's contents)."""
import numpy as np
import pytest

import bench
import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import SOP_NAMES

pytestmark = pytest.mark.gpu


def _device_operands(g, X, Y, Z0, vbits=32):
    import torch
    dev = torch.device("cuda:0")
    np_v = np.float32 if vbits == 32 else np.float64
    up = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    val = None if g["val"] is None else g["val"].astype(np_v)
    return dict(val=up(val), indx=up(g["indx"]), pb=up(g["pntrb"]), pe=up(g["pntre"]), X=up(X), Y=up(Y), Z0=up(Z0))


def _call(imsg, g, d, k, beta, Z, bits, vbits, noalloc, nnz=None):
    import torch
    rc = fa.fusedMM_csr(imsg, g["rows"], g["cols"], k, 1.0, g["nnz"] if nnz is None else nnz, g["rows"], g["cols"],
                        d["val"], d["indx"], d["pb"], d["pe"], d["X"], k, d["Y"], k, beta, Z, k, index_bits=bits,
                        stream=torch.cuda.current_stream().cuda_stream, value_bits=vbits, noalloc=noalloc)
    torch.cuda.synchronize()
    return rc


def _both_ways(imsg, sk, g, X, Y, Z0, beta, bits=32, vbits=32):
    """(Z of fusedMM_csr_stream, Z of fusedMM_csr_stream_noalloc, split counters of the latter)."""
    k = Y.shape[1]
    d = _device_operands(g, X, Y, Z0, vbits)
    gpu_api.set_kind(sk, bits, vbits)
    Za, Zb = d["Z0"].clone(), d["Z0"].clone()
    assert _call(imsg, g, d, k, beta, Za, bits, vbits, False) == 0
    assert _call(imsg, g, d, k, beta, Zb, bits, vbits, True) == 0
    return Za, Zb, gpu_api.last_split(bits, vbits)


def test_two_calls_in_a_row_second_smaller():
    import torch
    # first call: power-law graph at K=512 with library-default thresholds; its hubs are split,
    # so the heavy-row queue, the segment descriptors and the partial results are all in use
    g, X, Y = bench.make_workload("c5", 5)
    deg = np.diff(g["rowptr"])
    heavy_deg, seg_len = gpu_api.default_split(512)
    print("first call: rows", g["rows"], "nnz", g["nnz"], "rows split", int((deg > heavy_deg).sum()), flush=True)
    assert (deg > heavy_deg).sum() >= 2
    Z0 = np.zeros((g["rows"], 512), np.float32)
    Za, Zb, (h, s, o) = _both_ways(fa.MSG_SIGMOID, SOP_NAMES["sigmoid"], g, X, Y, Z0, 0.0)
    assert h == int((deg > heavy_deg).sum()) and s > h and o == 0
    assert torch.equal(Za, Zb)
    assert float(Za.abs().max()) > 0

    # second call, smaller, another op, accumulating into a non-zero Z: the array still holds
    # the first call's queue, bitmap and counters
    g2 = graphs.ragged(32, rows=64, cols=5000, hub_deg=40000)
    k2 = 64
    Y2 = graphs.features(g2["cols"], k2, 2, -0.5, 0.5, 2)
    Z02 = graphs.features(g2["rows"], k2, 2, -1, 1, 3)
    print("second call: rows", g2["rows"], "nnz", g2["nnz"], flush=True)
    Za, Zb, (h, s, o) = _both_ways(fa.MSG_SPMM, 0, g2, None, Y2, Z02, 1.0)
    hd2, sl2 = gpu_api.default_split(k2)
    assert (h, s, o) == (1, -(-40000 // sl2), 0)
    assert torch.equal(Za, Zb)

    # third: no row long enough to split (the bitmap of the call before must have been cleared)
    g3 = graphs.with_values(graphs.tiny_er(3000, 20000, 5))
    X3 = graphs.features(3000, 128, 3, -0.5, 0.5, 1)
    Y3 = graphs.features(3000, 128, 3, -0.5, 0.5, 2)
    print("third call: rows", g3["rows"], "nnz", g3["nnz"], flush=True)
    Za, Zb, (h, s, o) = _both_ways(fa.MSG_SIGMOID, SOP_NAMES["sigmoid"], g3, X3, Y3, np.zeros((3000, 128), np.float32), 0.0)
    assert (h, s, o) == (0, 0, 0)
    assert torch.equal(Za, Zb)


@pytest.mark.parametrize("bits,vbits", [(64, 32), (32, 64)])
def test_other_index_and_value_widths(bits, vbits):
    """Every library has its own copy of the array; forced low thresholds split most rows."""
    import torch
    np_v = np.float32 if vbits == 32 else np.float64
    g = graphs.ragged(bits, hub_deg=3000)
    k = 48
    X = graphs.features(g["rows"], k, 1, -1, 1, 1).astype(np_v)
    Y = graphs.features(g["cols"], k, 1, -1, 1, 2).astype(np_v)
    Z0 = graphs.features(g["rows"], k, 1, -1, 1, 3).astype(np_v)
    gpu_api.set_split(10, 7, bits, vbits)
    try:
        for beta in (0.0, 1.0):
            print("widths", bits, vbits, "beta", beta, flush=True)
            Za, Zb, (h, s, o) = _both_ways(fa.MSG_TDIST, SOP_NAMES["tdist"], g, X, Y, Z0, beta, bits, vbits)
            assert h > 10 and o == 0
            assert torch.equal(Za, Zb)
    finally:
        gpu_api.set_split(0, 0, bits, vbits)


def test_sizes_beyond_the_array_are_refused_and_touch_nothing():
    import torch
    lib = fa.load(32)
    assert lib.fusedMM_amd_noalloc_capacity() == 32 << 20
    g = graphs.with_values(graphs.tiny_er(500, 3000, 6))
    k = 512
    Y = graphs.features(500, k, 4, -0.5, 0.5, 2)
    Z0 = graphs.features(500, k, 4, -1, 1, 3)
    d = _device_operands(g, None, Y, Z0)
    gpu_api.set_kind(0)
    Z = d["Z0"].clone()
    # a caller-stated nnz of 10^9 at K=512 asks for ~6 GB of partial results
    assert _call(fa.MSG_SPMM, g, d, k, 0.0, Z, 32, 32, True, nnz=10 ** 9) == fa.NOT_ENOUGH_MEM
    assert torch.equal(Z, d["Z0"])
    # the allocating entry point serves the same call
    assert _call(fa.MSG_SPMM, g, d, k, 0.0, Z, 32, 32, False, nnz=g["nnz"]) == 0
    Zn = d["Z0"].clone()
    assert _call(fa.MSG_SPMM, g, d, k, 0.0, Zn, 32, 32, True) == 0
    assert torch.equal(Z, Zn)
    # rows wider than one kernel instance holds are refused as well
    kw = 2052
    Yw = graphs.features(500, kw, 4, -0.5, 0.5, 2)
    dw = _device_operands(g, None, Yw, np.zeros((500, kw), np.float32))
    Zw = dw["Z0"].clone()
    assert _call(fa.MSG_SPMM, g, dw, kw, 0.0, Zw, 32, 32, True) == fa.NOT_ENOUGH_MEM
    assert not bool(Zw.any())
