"""General op tuples on the GPU, and the corners of the fusedMM_csr contract."""
import os

import numpy as np
import pytest

import checks
import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_tuple_sweep_against_reference_golden(oracle):
    """168 op tuples: the reference's general pipeline (golden Z) vs the GPU's
    runtime-switched kernel.  Sums differ in order only; max/min are exact."""
    d = np.load(os.path.join(GOLD, "tuples_i32.npz"))
    rows, cols = (int(v) for v in d["shape"])
    g = {"rows": rows, "cols": cols, "nnz": int(d["indx"].size), "pntrb": d["pntrb"], "pntre": d["pntre"],
         "indx": d["indx"], "val": d["val"]}
    gpu_api.set_kind(SOP_NAMES["tdist"], 32)
    lib = fa.load(32)
    prev = lib.fusedMM_amd_set_opt(0)      # the golden Z comes from the general pipeline: always accumulates
    try:
        for imsg, want in zip(d["msgs"], d["Z"]):
            imsg = int(imsg)
            print("tuple", hex(imsg), flush=True)
            rc, Z = gpu_api.run(imsg, g, d["X"], d["Y"], d["Z0"], bits=32)
            assert rc == 0, hex(imsg)
            checks.assert_close(Z, want, 3e-5, 1e-5 * float(np.abs(want).max()), None, hex(imsg))
    finally:
        lib.fusedMM_amd_set_opt(prev)


@pytest.mark.parametrize("bits", [32, 64])
def test_general_pipeline_always_accumulates(oracle, bits):
    """opt off: the pattern tuples follow the general rule (beta ignored)."""
    g = graphs.ragged(bits, hub_deg=50)
    k = 32
    Y = graphs.features(g["cols"], k, 4, -0.5, 0.5, 2)
    Z0 = graphs.features(g["rows"], k, 4, -1, 1, 3)
    lib = fa.load(bits)
    prev = lib.fusedMM_amd_set_opt(0)
    try:
        rc, Z = gpu_api.run(MSG["m"], g, None, Y, Z0, beta=0.0, bits=bits)
    finally:
        lib.fusedMM_amd_set_opt(prev)
    assert rc == 0
    want = Z0.copy()
    oracle.generic(MSG["m"], g, None, Y, want)
    np.testing.assert_allclose(Z, want, rtol=1e-5, atol=1e-5)
    assert np.abs(Z[0] - Z0[0]).max() == 0            # empty row untouched


@pytest.mark.parametrize("where", ["device", "host"])
def test_m_smaller_than_rows_and_split_pointers(oracle, where):
    g = graphs.split_pointers(graphs.ragged(32, hub_deg=70))
    k = 64
    X = graphs.features(g["rows"], k, 5, -0.5, 0.5, 1)
    Y = graphs.features(g["cols"], k, 5, -0.5, 0.5, 2)
    Z0 = graphs.features(g["rows"], k, 5, -1, 1, 3)
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32)
    m = 41
    rc, Z = gpu_api.run(MSG["s"], g, X, Y, Z0, beta=0.0, bits=32, where=where, m=m)
    assert rc == 0
    want = gpu_api.oracle_mirror(oracle, "s", g, X, Y, Z0, 0.0, 1, k, *gpu_api.default_split(k), m=m)
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))
    np.testing.assert_array_equal(Z[m:], Z0[m:])      # rows beyond m untouched


@pytest.mark.parametrize("where", ["device", "host"])
def test_leading_dimensions_larger_than_k(oracle, where):
    g = graphs.ragged(32, hub_deg=70)
    k, ldx, ldy, ldz = 48, 52, 64, 56
    X = graphs.features(g["rows"], ldx, 6, -0.5, 0.5, 1)
    Y = graphs.features(g["cols"], ldy, 6, -0.5, 0.5, 2)
    Z0 = graphs.features(g["rows"], ldz, 6, -1, 1, 3)
    gpu_api.set_kind(SOP_NAMES["tdist"], 32)
    rc, Z = gpu_api.run(MSG["t"], g, X, Y, Z0, beta=1.0, bits=32, where=where, k=k)
    assert rc == 0
    want = gpu_api.oracle_mirror(oracle, "t", g, X, Y, Z0, 1.0, 2, k, *gpu_api.default_split(k))
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))
    np.testing.assert_array_equal(Z[:, k:], Z0[:, k:])   # padding columns untouched


def test_unaligned_operands_take_the_scalar_layout(oracle):
    """ldy not a multiple of 4: 16-byte gathers are impossible; the 4-byte layout is used."""
    g = graphs.ragged(32, hub_deg=70)
    k, ldy = 64, 65
    X = graphs.features(g["rows"], k, 7, -0.5, 0.5, 1)
    Y = graphs.features(g["cols"], ldy, 7, -0.5, 0.5, 2)
    Z0 = np.zeros((g["rows"], k), np.float32)
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32)
    rc, Z = gpu_api.run(MSG["s"], g, X, Y, Z0, bits=32, k=k)
    assert rc == 0
    want = Z0.copy()
    oracle.opt("s", g, X, Y, want, sop_kind=1, mode=2, V=1, L=64, S=1, k=k)
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))


def test_x_and_y_are_the_same_buffer(oracle):
    """Embedding training passes A = B (config 1 of the benchmark list)."""
    import torch
    g = graphs.tiny_er(300, 2400, 12)
    k = 32
    E = graphs.features(300, k, 8, -1, 1, 1)
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    dE, Z = t(E), torch.zeros((300, k), device=dev)
    val, indx, pb, pe = t(g["val"]), t(g["indx"]), t(g["pntrb"]), t(g["pntre"])
    gpu_api.set_kind(SOP_NAMES["fr"], 32)
    rc = fa.fusedMM_csr(fa.MSG_FR, 300, 300, k, 1.0, g["nnz"], 300, 300, val, indx, pb, pe, dE, k, dE, k, 0.0, Z, k)
    assert rc == 0
    torch.cuda.synchronize()
    want = gpu_api.oracle_mirror(oracle, "t", g, E, E, np.zeros((300, k), np.float32), 0.0, 3, k, *gpu_api.default_split(k))
    np.testing.assert_array_equal(Z.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert np.isfinite(want).all()                    # no self loops => no 1/0


def test_empty_inputs():
    k = 16
    Y = graphs.features(5, k, 9)
    Z0 = graphs.features(4, k, 9, stream=3)
    empty = {"rows": 4, "cols": 5, "nnz": 0, "pntrb": np.zeros(4, np.int32), "pntre": np.zeros(4, np.int32),
             "indx": np.zeros(1, np.int32), "val": np.zeros(1, np.float32)}
    rc, Z = gpu_api.run(MSG["m"], empty, None, Y, Z0, beta=0.0)
    assert rc == 0 and not Z.any()                    # beta == 0 overwrites even empty rows
    rc, Z = gpu_api.run(MSG["m"], empty, None, Y, Z0, beta=1.0)
    assert rc == 0 and np.array_equal(Z, Z0)
    rc, Z = gpu_api.run(MSG["m"], empty, None, Y, Z0, beta=0.0, m=0)
    assert rc == 0 and np.array_equal(Z, Z0)          # m == 0: nothing happens


@pytest.mark.parametrize("k", [2052, 4100, 2049])
@pytest.mark.parametrize("tkern,kind", [("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist")])
def test_rows_wider_than_one_kernel_instance(oracle, tkern, kind, k):
    """k > 2048: processed in column slabs of 2048; tuples that reduce over the
    whole row assemble the per-edge scalar from the slabs first."""
    g = graphs.ragged(32, rows=40, cols=60, hub_deg=300)
    amp = 0.05 if tkern in ("s", "t") else 0.5          # keep dots inside the sigmoid table's range
    X = graphs.features(g["rows"], k, 4, -amp, amp, 1)
    Y = graphs.features(g["cols"], k, 4, -amp, amp, 2)
    Z0 = graphs.features(g["rows"], k, 4, -1, 1, 3)
    sk = SOP_NAMES[kind] if kind else 0
    gpu_api.set_kind(sk, 32)
    for beta, where in ((0.0, "device"), (1.0, "host")):
        rc, Z = gpu_api.run(MSG[tkern], g, X, Y, Z0, beta=beta, bits=32, where=where)
        assert rc == 0
        want = Z0.copy()
        oracle.opt(tkern, g, X, Y, want, beta=beta, sop_kind=sk, mode=1)
        extra = checks.sigmoid_flip_slack(oracle.table(), g, X, Y)[0] if tkern == "s" else None
        checks.assert_close(Z, want, 1e-4, 1e-5, extra, "%s k=%d" % (tkern, k))


@pytest.mark.parametrize("bits", [32, 64])
def test_golden_ops_on_gpu(oracle, bits):
    """The reference's own outputs (golden fixtures) within the stated tolerances."""
    d = np.load(os.path.join(GOLD, "ops_i%d.npz" % bits))
    it = np.int32 if bits == 32 else np.int64
    for gname in ("ragged", "er"):
        rows, cols = (int(v) for v in d[gname + "_shape"])
        g = {"rows": rows, "cols": cols, "nnz": int(d[gname + "_indx"].size), "pntrb": d[gname + "_pntrb"].astype(it),
             "pntre": d[gname + "_pntre"].astype(it), "indx": d[gname + "_indx"].astype(it), "val": d[gname + "_val"]}
        deg = (g["pntre"] - g["pntrb"]).astype(np.int64)
        for k in (16, 40):
            X, Y = d["%s_X%d" % (gname, k)], d["%s_Y%d" % (gname, k)]
            for t, kind in (("s", "sigmoid"), ("t", "tdist"), ("f", "fr"), ("m", None), ("g", None)):
                sk = SOP_NAMES[kind] if kind else 0
                gpu_api.set_kind(sk, bits)
                rc, Z = gpu_api.run(MSG[t], g, X, Y, np.zeros((rows, k), np.float32), bits=bits)
                assert rc == 0
                want = d["%s_%s_k%d_fusedmm" % (gname, t, k)]
                rtol, atol = (1e-5, 1e-6) if t in ("g", "m") else (1e-4, 1e-6)
                es = np.zeros(int(g["pntre"].max()), np.float32)
                tmp = np.zeros((rows, k), np.float32)
                oracle.opt("t" if t == "f" else t, g, X, Y, tmp, sop_kind=sk, mode=1, edge_s=es if kind else None)
                r_, slots = checks.edge_rows(g)
                d_abs = np.ones(slots.size) if t == "g" else (np.abs(g["val"][slots]).astype(np.float64) if t == "m"
                                                               else np.abs(oracle.sop(sk, es[slots])).astype(np.float64))
                # the golden Z is itself a sequential fp32 sum over deg edges
                extra = 2 * checks.EPS32 * np.maximum(deg, 1)[:, None] * checks.abs_term_sum(t, g, X, Y, d_abs)
                if t == "s":
                    extra = extra + checks.sigmoid_flip_slack(oracle.table(), g, X, Y)[0]
                checks.assert_close(Z, want, rtol, atol, extra, "%s %s k=%d" % (gname, t, k))


def test_stream_entry_can_be_captured_in_a_hip_graph(oracle):
    """fusedMM_csr_stream enqueues kernels only (no memset, no allocation once the
    work queues exist): a caller may capture it and replay it.  Every replay is
    checked against the eager result, with eager work in between; the graph has
    split rows, so all three kernels and the queue reset are replayed."""
    import torch
    g = graphs.ragged(32, rows=200, cols=3000, hub_deg=5000)
    k = 128
    X = graphs.features(g["rows"], k, 3, -0.5, 0.5, 1)
    Y = graphs.features(g["cols"], k, 3, -0.5, 0.5, 2)
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    val, indx, pb, pe, dX, dY = t(g["val"]), t(g["indx"]), t(g["pntrb"]), t(g["pntre"]), t(X), t(Y)
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32)

    def enqueue(Z):
        rc = fa.fusedMM_csr(fa.MSG_SIGMOID, g["rows"], g["cols"], k, 1.0, g["nnz"], g["rows"], g["cols"], val, indx,
                            pb, pe, dX, k, dY, k, 0.0, Z, k, stream=torch.cuda.current_stream().cuda_stream)
        assert rc == 0

    Zeager = torch.zeros((g["rows"], k), device=dev)
    enqueue(Zeager)                                   # also sizes the work queues
    torch.cuda.synchronize()
    assert gpu_api.last_split(32)[1] > 0
    Zg = torch.full((g["rows"], k), 9.0, device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue(Zg)
    for rep in range(4):
        Zg.fill_(float(rep))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Zg, Zeager), rep
        dY2 = dY * 2.0                                # eager work between replays
        Ze2 = torch.zeros_like(Zeager)
        rc = fa.fusedMM_csr(fa.MSG_SIGMOID, g["rows"], g["cols"], k, 1.0, g["nnz"], g["rows"], g["cols"], val, indx,
                            pb, pe, dX, k, dY2, k, 0.0, Ze2, k)
        assert rc == 0


def test_operand_check_rejects_bad_csr_instead_of_reading_outside_y():
    """With the optional check on, a column id >= n or a row with pntre < pntrb
    returns FUSEDMM_FAIL_RETURN before any kernel dereferences it."""
    lib = fa.load(32)
    prev = lib.fusedMM_amd_set_validate(1)
    try:
        g = graphs.tiny_er(50, 120, 2)
        k = 32
        Y = graphs.features(50, k, 2)
        Z0 = np.zeros((50, k), np.float32)
        rc, _ = gpu_api.run(MSG["g"], g, None, Y, Z0)
        assert rc == 0                                   # clean operands pass
        bad = dict(g)
        bad["indx"] = g["indx"].copy()
        bad["indx"][7] = 50                              # one past the last row of Y
        for where in ("device", "host"):
            rc, Z = gpu_api.run(MSG["g"], bad, None, Y, Z0, where=where)
            assert rc == fa.FAIL and not Z.any()
        bad = dict(g)
        bad["pntre"] = g["pntre"].copy()
        bad["pntre"][3] = g["pntrb"][3] - 1
        rc, _ = gpu_api.run(MSG["g"], bad, None, Y, Z0)
        assert rc == fa.FAIL
    finally:
        lib.fusedMM_amd_set_validate(prev)


def test_mixed_host_and_device_operands_are_refused():
    import torch
    g = graphs.tiny_er(50, 120, 2)
    k = 32
    Y = graphs.features(50, k, 2)
    dev = torch.device("cuda:0")
    Zd = torch.zeros((50, k), device=dev)
    rc = fa.fusedMM_csr(fa.MSG_GCN, 50, 50, k, 1.0, g["nnz"], 50, 50, g["val"], g["indx"], np.ascontiguousarray(g["pntrb"]),
                        np.ascontiguousarray(g["pntre"]), None, k, Y, k, 0.0, Zd, k)       # Z on the GPU, the rest on the host
    assert rc == fa.FAIL
    torch.cuda.synchronize()
    assert not Zd.any()


def test_finalize_releases_and_the_library_recovers(oracle):
    """fusedMM_amd_finalize() frees every buffer the library holds; the next call
    sets everything up again (table, counters, queues)."""
    g = graphs.ragged(32, hub_deg=5000)
    k = 64
    X = graphs.features(g["rows"], k, 3, -0.5, 0.5, 1)
    Y = graphs.features(g["cols"], k, 3, -0.5, 0.5, 2)
    Z0 = np.zeros((g["rows"], k), np.float32)
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32)
    rc, Za = gpu_api.run(MSG["s"], g, X, Y, Z0)
    assert rc == 0
    fa.load(32).fusedMM_amd_finalize()
    fa.load(32).fusedMM_amd_finalize()          # twice is harmless
    rc, Zb = gpu_api.run(MSG["s"], g, X, Y, Z0, where="host")
    assert rc == 0
    np.testing.assert_array_equal(Za.view(np.uint32), Zb.view(np.uint32))


def _same_special(Z, want, imsg, u, what):
    """NaN for NaN; elsewhere the same bits -- except where the tuple sums over the row's elements (a ROP), whose
    order differs between the wavefront and the reference's loop: there, infinities equal and the rest to rounding."""
    nz, nw = np.isnan(Z), np.isnan(want)
    np.testing.assert_array_equal(nz, nw, err_msg=what)
    if (imsg & 0xF0) == 0:
        np.testing.assert_array_equal(Z.view(u)[~nz], want.view(u)[~nw], err_msg=what)
    else:
        np.testing.assert_allclose(Z[~nz], want[~nw], rtol=1e-5, atol=1e-6, err_msg=what)


@pytest.mark.parametrize("where", ["device", "host"])
@pytest.mark.parametrize("bits,vbits", [(32, 32), (64, 32), (32, 64)])
def test_max_and_min_stages_on_nan_and_signed_zeros_match_the_reference(where, bits, vbits):
    """VOP_MAX / VOP_MIN / AOP_MAX / AOP_MIN on operands salted with NaN, infinities and zeros of both signs,
    rows with at most one edge (with more, what a NaN term leaves behind depends on the order of the edges,
    in the reference as here): the reference's own output, NaN for NaN and bit for bit elsewhere.  Its fmax /
    fmin are the ternaries of fusedMM.c:18-19 -- a NaN on the right wins, the right one of two zeros is kept --
    and so are the kernels'; where sub-wave accumulators are combined a NaN is kept."""
    import os
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "special_values.npz"))
    multi, single, X, Y, Z0, msgs = graphs.special_values_case(bits)
    npv, sfx, u = (np.float32, "", np.uint32) if vbits == 32 else (np.float64, "_d", np.uint64)
    for imsg, want in zip(msgs, d["Z_single" + sfx]):
        rc, Z = gpu_api.run(int(imsg), single, X.astype(npv), Y.astype(npv), Z0.astype(npv), bits=bits, vbits=vbits, where=where)
        assert rc == 0
        _same_special(Z, want, int(imsg), u, hex(int(imsg)))
    # the same operands with the packing of short rows switched off: every row goes through the merge of
    # the sub-wave accumulators, which must keep what the single edge left
    lib = fa.load(bits, vbits)
    prev = lib.fusedMM_amd_set_pack_rows(0)
    try:
        for imsg, want in zip(msgs, d["Z_single" + sfx]):
            rc, Z = gpu_api.run(int(imsg), single, X.astype(npv), Y.astype(npv), Z0.astype(npv), bits=bits, vbits=vbits, where=where)
            assert rc == 0
            _same_special(Z, want, int(imsg), u, "unpacked " + hex(int(imsg)))
    finally:
        lib.fusedMM_amd_set_pack_rows(prev)
