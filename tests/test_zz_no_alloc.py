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


def test_calls_leave_device_memory_as_they_found_it_and_match_the_oracle():
    """The property the entry point exists for: after the set-up call that allocates nothing either
    (fusedMM_amd_init_noalloc) and one warm-up call, a series of calls of different sizes, ops and K -- one of
    them splitting rows -- changes the free device memory by not one byte.  Run on a library whose grown queues
    were released (fusedMM_amd_finalize), so that a fall-back to the growing path would show as an allocation.
    One of the results is also held to the CPU oracle's mirror of the kernels, bit for bit."""
    import torch
    from oracle_api import Oracle
    lib = fa.load(32)
    # (the static array is part of the library's code object: it comes into being when the runtime loads that
    # object, on the library's first use in the process -- make sure that lies behind us)
    assert lib.fusedMM_amd_init_noalloc() == 0
    torch.cuda.synchronize()
    lib.fusedMM_amd_finalize()                       # nothing grown is left; the static array stays (it is not an allocation)
    free0 = torch.cuda.mem_get_info()[0]
    assert lib.fusedMM_amd_init_noalloc() == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0     # the set-up call allocated no device memory

    cases = []
    g1 = graphs.with_values(graphs.tiny_er(3000, 20000, 5))
    cases.append(("s", fa.MSG_SIGMOID, 1, g1, graphs.features(3000, 128, 3, -0.5, 0.5, 1), graphs.features(3000, 128, 3, -0.5, 0.5, 2), 0.0))
    g2 = graphs.ragged(32, rows=64, cols=5000, hub_deg=40000)      # its hub row is cut into segments
    cases.append(("m", fa.MSG_SPMM, 0, g2, None, graphs.features(5000, 64, 2, -0.5, 0.5, 2), 1.0))
    g3 = graphs.boundary_graph()                                      # short rows, walked one per sub-wave
    cases.append(("t", fa.MSG_TDIST, 2, g3, graphs.features(g3["rows"], 32, 4, -1, 1, 1), graphs.features(g3["cols"], 32, 4, -1, 1, 2), 0.0))
    g4 = graphs.ragged(32, hub_deg=300)
    cases.append(("g", fa.MSG_GCN, 0, g4, None, graphs.features(g4["cols"], 512, 6, -0.5, 0.5, 2), 0.0))
    ops = []
    for tkern, imsg, sk, g, X, Y, beta in cases:      # every operand resident before the measurement starts
        Z0 = graphs.features(g["rows"], Y.shape[1], 9, -1, 1, 3)
        ops.append((tkern, imsg, sk, g, X, Y, Z0, beta, _device_operands(g, X, Y, Z0)))
    outs = [o[8]["Z0"].clone() for o in ops]
    # warm-up (module loading, first launch of each kernel instance), then the measured series
    for (tkern, imsg, sk, g, X, Y, Z0, beta, d), Z in zip(ops, outs):
        gpu_api.set_kind(sk)
        assert _call(imsg, g, d, Y.shape[1], beta, Z, 32, 32, True) == 0
    torch.cuda.synchronize()
    free1 = torch.cuda.mem_get_info()[0]
    for rep in range(3):
        for (tkern, imsg, sk, g, X, Y, Z0, beta, d), Z in zip(ops, outs):
            Z.copy_(d["Z0"])
            gpu_api.set_kind(sk)
            assert _call(imsg, g, d, Y.shape[1], beta, Z, 32, 32, True) == 0
            if tkern == "m":
                assert gpu_api.last_split()[1] > 1
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free1      # not one byte allocated or freed by twelve calls
    oracle = Oracle()
    for (tkern, imsg, sk, g, X, Y, Z0, beta, d), Z in zip(ops, outs):
        k = Y.shape[1]
        want = gpu_api.oracle_mirror(oracle, tkern, g, X, Y, Z0, beta, sk, k, *gpu_api.default_split(k))
        np.testing.assert_array_equal(Z.cpu().numpy().view(np.uint32), want.view(np.uint32), err_msg=tkern)
