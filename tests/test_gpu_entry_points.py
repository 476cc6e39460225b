"""Entry points and switches around fusedMM_csr: the reference's second-level
entry sgfusedMM_csr / dgfusedMM_csr (kernels/src/kernels.c:456-631), the device
copy of the sigmoid table, the operand check on every path, calls on several
streams, and inputs at the edge of what the reference defines."""
import ctypes as C

import numpy as np
import pytest

import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES

pytestmark = pytest.mark.gpu
GOLD = __import__("os").path.join(__import__("os").path.dirname(__import__("os").path.abspath(__file__)), "golden")


def _dev(a):
    import torch
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(torch.device("cuda:0"))


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("vbits", [32, 64])
def test_second_level_entry_equals_fusedmm_csr(bits, vbits):
    """sgfusedMM_csr('g'|'m'|'s'|'t', ...) called through its own symbol gives the
    bits of fusedMM_csr with the matching op tuple, for beta 0 and 1, host and
    device operands; an unknown letter prints and leaves C alone (kernels.c:627-629)."""
    import torch
    np_v = np.float32 if vbits == 32 else np.float64
    it, ct = (np.int32, C.c_int32) if bits == 32 else (np.int64, C.c_int64)
    cv = C.c_float if vbits == 32 else C.c_double
    lib = fa.load(bits, vbits)
    gf = lib.sgfusedMM_csr if vbits == 32 else lib.dgfusedMM_csr
    g = graphs.ragged(bits, hub_deg=900)
    k = 64
    X = graphs.features(g["rows"], k, 1, -0.5, 0.5, 1).astype(np_v)
    Y = graphs.features(g["cols"], k, 1, -0.5, 0.5, 2).astype(np_v)
    Z0 = graphs.features(g["rows"], k, 1, -1, 1, 3).astype(np_v)
    val = g["val"].astype(np_v)
    d = dict(val=_dev(val), indx=_dev(g["indx"]), pb=_dev(g["pntrb"]), pe=_dev(g["pntre"]), X=_dev(X), Y=_dev(Y))

    def second_level(letter, beta, where):
        if where == "host":
            Z = Z0.copy()
            ops = [val, g["indx"], g["pntrb"], g["pntre"], X, Y, Z]
            addr = [o.ctypes.data for o in ops]
        else:
            Zd = _dev(Z0)
            ops = [d["val"], d["indx"], d["pb"], d["pe"], d["X"], d["Y"], Zd]
            addr = [o.data_ptr() for o in ops]
        gf(C.c_char(letter.encode()), ct(g["rows"]), ct(g["cols"]), ct(k), cv(1.0), ct(g["nnz"]), ct(g["rows"]),
           ct(g["cols"]), addr[0], addr[1], addr[2], addr[3], addr[4], ct(k), addr[5], ct(k), cv(beta), addr[6], ct(k))
        if where == "host":
            return Z
        torch.cuda.synchronize()
        return Zd.cpu().numpy()

    for letter, kind in (("g", None), ("m", None), ("s", "sigmoid"), ("t", "tdist")):
        gpu_api.set_kind(SOP_NAMES[kind] if kind else 0, bits, vbits)
        for beta in (0.0, 1.0):
            for where in ("device", "host"):
                print("case", letter, beta, where, bits, vbits, flush=True)
                rc, want = gpu_api.run(MSG[letter], g, X, Y, Z0, beta=beta, bits=bits, where=where, vbits=vbits)
                assert rc == 0
                got = second_level(letter, beta, where)
                np.testing.assert_array_equal(got.view(np.uint8), want.view(np.uint8))
                assert not np.array_equal(got, Z0)
    for where in ("device", "host"):
        got = second_level("q", 0.0, where)                  # "unknown kernel type!" on stderr, nothing else
        np.testing.assert_array_equal(got.view(np.uint8), Z0.view(np.uint8))


@pytest.mark.parametrize("vbits", [32, 64])
def test_device_sigmoid_table_equals_the_reference_table(vbits):
    """The table the kernels index, read back through the kernels themselves:
    2048 one-edge rows, Y = 1, X[i] = centre of bin i in column 0, sigmoid tuple
    => Z[i, 0] = 1 - table[i].  Compared bit for bit with the table of the real
    reference's tester (test/fusedMMtime.cpp:594-604, stored in golden/sop.npz)."""
    np_v = np.float32 if vbits == 32 else np.float64
    d = np.load(__import__("os").path.join(GOLD, "sop.npz"))
    table = d["table" if vbits == 32 else "table_d"]
    assert table.dtype == np_v and table.size == 2048
    n, k = 2048, 4
    it = np.int32
    g = {"rows": n, "cols": 1, "nnz": n, "val": np.ones(n, np.float32), "indx": np.zeros(n, it),
         "pntrb": np.arange(n, dtype=it), "pntre": np.arange(1, n + 1, dtype=it)}
    X = np.zeros((n, k), np_v)
    X[:, 0] = ((np.arange(n) + 0.5) * 10.0 / 2048 - 5.0).astype(np_v)     # exact in binary: (2i+1) * 5/2048 - 5
    Y = np.ones((1, k), np_v)
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32, vbits)
    for where in ("device", "host"):
        rc, Z = gpu_api.run(MSG["s"], g, X, Y, np.zeros((n, k), np_v), bits=32, where=where, vbits=vbits)
        assert rc == 0
        want = (np_v(1.0) - table).astype(np_v)
        np.testing.assert_array_equal(np.ascontiguousarray(Z[:, 0]).view(np.uint8), want.view(np.uint8))
        np.testing.assert_array_equal(np.ascontiguousarray(Z[:, 3]).view(np.uint8), want.view(np.uint8))
    # and through the entry point whose table lives in the static array
    import torch
    dv = [_dev(g["val"].astype(np_v)), _dev(g["indx"]), _dev(g["pntrb"]), _dev(g["pntre"]), _dev(X), _dev(Y)]
    Zd = _dev(np.zeros((n, k), np_v))
    rc = fa.fusedMM_csr(MSG["s"], n, 1, k, 1.0, n, n, 1, dv[0], dv[1], dv[2], dv[3], dv[4], k, dv[5], k, 0.0, Zd, k,
                        stream=torch.cuda.current_stream().cuda_stream, value_bits=vbits, noalloc=True)
    assert rc == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(np.ascontiguousarray(Zd.cpu().numpy()[:, 0]).view(np.uint8), want.view(np.uint8))


SOPFN = C.CFUNCTYPE(C.c_int, C.c_float, C.POINTER(C.c_float))


def test_operand_check_covers_the_host_function_path():
    """FUSEDMM_VALIDATE with SOP_UDEF served by the caller's host function: the
    first pass gathers Y rows by column id and the host walks the row pointers, so
    bad CSR must be turned away before either happens."""
    lib = fa.load(32)
    prev_kind = lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_HOST)
    prev = lib.fusedMM_amd_set_validate(1)
    calls = [0]

    def sop(val, out):
        calls[0] += 1
        out[0] = val
        return 0

    cb = SOPFN(sop)
    lib.fusedMM_amd_set_sop_callback(C.cast(cb, C.c_void_p))
    try:
        g = graphs.tiny_er(50, 120, 2)
        k = 32
        X = graphs.features(50, k, 2, -0.5, 0.5, 1)
        Y = graphs.features(50, k, 2, -0.5, 0.5, 2)
        Z0 = np.zeros((50, k), np.float32)
        for where in ("device", "host"):
            rc, Z = gpu_api.run(MSG["s"], g, X, Y, Z0, where=where)
            assert rc == 0 and Z.any()
        seen = calls[0]
        assert seen == 2 * g["nnz"]
        bad_col = dict(g)
        bad_col["indx"] = g["indx"].copy()
        bad_col["indx"][7] = 50                              # one past the last row of Y
        bad_end = dict(g)
        bad_end["pntre"] = g["pntre"].copy()
        bad_end["pntre"][3] = g["pntrb"][3] - 1
        bad_start = dict(g)
        bad_start["pntrb"] = g["pntrb"].copy()
        bad_start["pntrb"][0] = -4
        for bad in (bad_col, bad_end, bad_start):
            for where in ("device", "host"):
                rc, Z = gpu_api.run(MSG["s"], bad, X, Y, Z0, where=where)
                assert rc == fa.FAIL and not Z.any()
        assert calls[0] == seen                              # the user function was never reached
    finally:
        lib.fusedMM_amd_set_validate(prev)
        lib.fusedMM_amd_set_sop_kind(prev_kind)
        lib.fusedMM_amd_set_sop_callback(None)


def test_host_arrays_allocated_exactly_as_far_as_the_reference_reads(oracle):
    """ld > k with X, Y and Z ending at the last element the reference touches,
    (rows - 1) * ld + k, each placed at the very end of its own page-aligned
    mapping so that reading one element further would fault."""
    import mmap
    g = graphs.ragged(32, hub_deg=70)
    k, ldx, ldy, ldz = 48, 52, 64, 56

    def tight(rows, ld, seed, lo, hi):
        full = graphs.features(rows, ld, 6, lo, hi, seed)
        used = (rows - 1) * ld + k
        nbytes = used * 4
        pages = -(-nbytes // mmap.PAGESIZE)
        buf = mmap.mmap(-1, (pages + 1) * mmap.PAGESIZE)
        base = np.frombuffer(buf, np.uint8)
        # make the page after the data inaccessible
        libc = C.CDLL(None, use_errno=True)
        addr = base.ctypes.data
        assert libc.mprotect(C.c_void_p(addr + pages * mmap.PAGESIZE), C.c_size_t(mmap.PAGESIZE), 0) == 0
        off = pages * mmap.PAGESIZE - nbytes
        flat = base[off:off + nbytes].view(np.float32)
        flat[:] = full.reshape(-1)[:used]
        return full, flat, buf

    X, Xt, kx = tight(g["rows"], ldx, 1, -0.5, 0.5)
    Y, Yt, ky = tight(g["cols"], ldy, 2, -0.5, 0.5)
    Z0, Zt, kz = tight(g["rows"], ldz, 3, -1, 1)
    gpu_api.set_kind(SOP_NAMES["tdist"], 32)
    rc = fa.fusedMM_csr(MSG["t"], g["rows"], g["cols"], k, 1.0, g["nnz"], g["rows"], g["cols"], g["val"], g["indx"],
                        np.ascontiguousarray(g["pntrb"]), np.ascontiguousarray(g["pntre"]), Xt, ldx, Yt, ldy, 1.0, Zt, ldz)
    assert rc == 0
    want = gpu_api.oracle_mirror(oracle, "t", g, X, Y, Z0, 1.0, 2, k, *gpu_api.default_split(k))
    used = (g["rows"] - 1) * ldz + k
    np.testing.assert_array_equal(np.array(Zt).view(np.uint32), want.reshape(-1)[:used].view(np.uint32))


def test_calls_on_different_streams_share_the_queues_safely(oracle):
    """Every call on a GPU uses that GPU's one set of work queues.  Calls issued
    back to back on different (non-blocking) streams, with split rows, must each
    give the single-stream result: the library orders them."""
    import torch
    g = graphs.ragged(32, rows=300, cols=4000, hub_deg=30000)
    k = 128
    X = graphs.features(g["rows"], k, 3, -0.5, 0.5, 1)
    Ys = [graphs.features(g["cols"], k, 3 + i, -0.5, 0.5, 2) for i in range(4)]
    d = dict(val=_dev(g["val"]), indx=_dev(g["indx"]), pb=_dev(g["pntrb"]), pe=_dev(g["pntre"]), X=_dev(X))
    dY = [_dev(y) for y in Ys]
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32)

    def enqueue(Y, Z, stream, noalloc):
        rc = fa.fusedMM_csr(fa.MSG_SIGMOID, g["rows"], g["cols"], k, 1.0, g["nnz"], g["rows"], g["cols"], d["val"],
                            d["indx"], d["pb"], d["pe"], d["X"], k, Y, k, 0.0, Z, k, stream=stream, noalloc=noalloc)
        assert rc == 0

    for noalloc in (False, True):
        want = []
        for y in dY:
            Z = torch.zeros((g["rows"], k), device="cuda:0")
            enqueue(y, Z, torch.cuda.current_stream().cuda_stream, noalloc)
            torch.cuda.synchronize()
            want.append(Z)
        assert gpu_api.last_split(32)[1] > 0
        streams = [torch.cuda.Stream() for _ in range(4)]
        torch.cuda.synchronize()
        for rep in range(3):
            got = [torch.full((g["rows"], k), 5.0, device="cuda:0") for _ in range(4)]
            for i in range(4):
                enqueue(dY[i], got[i], streams[i].cuda_stream, noalloc)
            torch.cuda.synchronize()
            for i in range(4):
                assert torch.equal(got[i], want[i]), (noalloc, rep, i)


def test_nan_dot_product_takes_the_first_table_bin(oracle):
    """A NaN in X makes the dot NaN; neither saturation test holds for it and the
    reference converts it to an integer (undefined).  Here the index is clamped to
    bin 0 on the GPU and in the oracle alike, so the row stays finite."""
    g = graphs.tiny_er(64, 300, 4)
    k = 32
    X = graphs.features(64, k, 5, -0.5, 0.5, 1)
    Y = graphs.features(64, k, 5, -0.5, 0.5, 2)
    X[10, 3] = np.nan
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32)
    rc, Z = gpu_api.run(MSG["s"], g, X, Y, np.zeros((64, k), np.float32))
    assert rc == 0
    want = gpu_api.oracle_mirror(oracle, "s", g, X, Y, np.zeros((64, k), np.float32), 0.0, 1, k, *gpu_api.default_split(k))
    np.testing.assert_array_equal(Z.view(np.uint32), want.view(np.uint32))
    assert np.isfinite(Z).all() and g["pntre"][10] > g["pntrb"][10]
    t0 = oracle.table()[0]
    cols = g["indx"][g["pntrb"][10]:g["pntre"][10]]
    np.testing.assert_allclose(Z[10], ((np.float32(1) - t0) * Y[cols].astype(np.float64)).sum(0), rtol=1e-5, atol=1e-6)


def test_cmake_consumer_runs():
    """The executable the consumer CMake project builds against target `fusedmm`
    (fusedmm_amd/consumer, built in-tree by __graft_entry__.build()) runs its call on the GPU."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fusedmm_amd", "cmake_build", "xconsumer")
    if not os.path.exists(exe):
        pytest.skip("fusedmm_amd/cmake_build not built")
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout


def test_host_arrays_larger_than_the_pinned_staging_buffers(oracle):
    """Host-pointer mode moves operands through 16 MiB pinned buffers, a chunk at a
    time.  Arrays of several chunks and odd sizes arrive and return intact: same bits
    as the same call on device operands."""
    n, k = 70001, 132                       # Y and Z: 36.96 MB each, not a multiple of the chunk
    g = graphs.with_values(graphs.tiny_er(n, 6 * n, 21))
    X = graphs.features(n, k, 9, -0.5, 0.5, 1)
    Y = graphs.features(n, k, 9, -0.5, 0.5, 2)
    Z0 = graphs.features(n, k, 9, -1, 1, 3)
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32)
    for beta in (0.0, 1.0):
        rc, Zd = gpu_api.run(MSG["s"], g, X, Y, Z0, beta=beta, where="device")
        assert rc == 0
        rc, Zh = gpu_api.run(MSG["s"], g, X, Y, Z0, beta=beta, where="host")
        assert rc == 0
        np.testing.assert_array_equal(Zh.view(np.uint32), Zd.view(np.uint32))
    lib = fa.load(32)
    up, kern, down = C.c_double(), C.c_double(), C.c_double()
    assert lib.fusedMM_amd_last_host_phases(C.byref(up), C.byref(kern), C.byref(down)) == 0
    assert up.value > 0 and kern.value > 0 and down.value > 0
    # X == Y (one buffer): uploaded once, used for both
    rc, Zd = gpu_api.run(MSG["t"], g, Y, Y, Z0, beta=1.0, where="device")
    gpu_api.set_kind(SOP_NAMES["tdist"], 32)
    rc, Zd = gpu_api.run(MSG["t"], g, Y, Y, Z0, beta=1.0, where="device")
    rc2, Zh = gpu_api.run(MSG["t"], g, Y, Y, Z0, beta=1.0, where="host")
    assert rc == 0 and rc2 == 0
    np.testing.assert_array_equal(Zh.view(np.uint32), Zd.view(np.uint32))


def test_device_mirrors_of_host_operands_are_opt_in_and_invalidated_on_request():
    """Default: every host-pointer call re-uploads, so a changed Y is seen.  With
    fusedMM_amd_set_cache(1) the read-only operands are mirrored on the GPU and a
    changed Y is NOT seen until fusedMM_amd_invalidate() -- the documented contract."""
    lib = fa.load(32)
    g = graphs.with_values(graphs.tiny_er(400, 3000, 8))
    k = 64
    Y = graphs.features(400, k, 4, -0.5, 0.5, 2)
    Z0 = np.zeros((400, k), np.float32)
    gpu_api.set_kind(0, 32)
    run = lambda: gpu_api.run(MSG["m"], g, None, Y, Z0, where="host")[1]
    fresh = lambda: gpu_api.run(MSG["m"], g, None, Y.copy(), Z0, where="device")[1]
    a = run()
    Y *= 2.0
    np.testing.assert_array_equal(run(), fresh())            # default: the change is seen
    prev = lib.fusedMM_amd_set_cache(1)
    try:
        assert prev == 0
        b = run()                                            # uploads and keeps mirrors
        np.testing.assert_array_equal(b, fresh())
        Y *= 0.5                                             # back to the first values, in place
        np.testing.assert_array_equal(run(), b)              # mirror still holds the doubled Y
        lib.fusedMM_amd_invalidate()
        np.testing.assert_array_equal(run(), a)              # re-uploaded
    finally:
        lib.fusedMM_amd_set_cache(prev)
        lib.fusedMM_amd_invalidate()


def test_capture_refuses_what_would_block(oracle):
    """A device's first call (blocking set-up copies, allocations) and a call with operand
    validation switched on (reads a flag back) cannot be recorded into a HIP graph: both
    are refused with FUSEDMM_FAIL_RETURN before anything is enqueued, and the same calls
    succeed once the set-up has been done outside the capture and validation is off."""
    import torch
    lib = fa.load(64)
    g = graphs.with_values(graphs.tiny_er(300, 2000, 21, bits=64))
    k = 32
    Y = graphs.features(300, k, 6, -0.5, 0.5, 2)
    d = dict(val=_dev(g["val"]), indx=_dev(g["indx"]), pb=_dev(g["pntrb"]), pe=_dev(g["pntre"]), Y=_dev(Y))
    dev = torch.device("cuda:0")

    def enqueue(Z, noalloc):
        return fa.fusedMM_csr(fa.MSG_SPMM, g["rows"], g["cols"], k, 1.0, g["nnz"], g["rows"], g["cols"], d["val"], d["indx"],
                              d["pb"], d["pe"], None, k, d["Y"], k, 0.0, Z, k, index_bits=64,
                              stream=torch.cuda.current_stream().cuda_stream, noalloc=noalloc)

    torch.cuda.synchronize()
    lib.fusedMM_amd_finalize()                                # this library now knows nothing of the device
    Z1 = torch.full((g["rows"], k), 7.0, device=dev)
    Z2 = torch.full((g["rows"], k), 7.0, device=dev)
    Zwarm = torch.zeros((g["rows"], k), device=dev)
    first = torch.cuda.CUDAGraph()
    with torch.cuda.graph(first):
        rc_grown = enqueue(Z1, False)
        rc_static = enqueue(Z2, True)
        Zwarm.add_(1.0)                                       # something to record, so the graph is not empty
    assert rc_grown == fa.FAIL and rc_static == fa.FAIL
    assert lib.fusedMM_amd_init() == 0
    Zeager = torch.zeros((g["rows"], k), device=dev)
    assert enqueue(Zeager, False) == 0                        # sizes the grown queues
    torch.cuda.synchronize()
    second = torch.cuda.CUDAGraph()
    with torch.cuda.graph(second):
        prev = lib.fusedMM_amd_set_validate(1)
        rc_val = enqueue(Z1, False)
        rc_val_static = enqueue(Z2, True)
        lib.fusedMM_amd_set_validate(prev)
        rc_ok = enqueue(Z1, False)
        rc_ok_static = enqueue(Z2, True)
    assert rc_val == fa.FAIL and rc_val_static == fa.FAIL and rc_ok == 0 and rc_ok_static == 0
    for rep in range(2):
        Z1.fill_(float(rep) + 2.0)
        Z2.fill_(float(rep) + 3.0)
        second.replay()
        torch.cuda.synchronize()
        assert torch.equal(Z1, Zeager) and torch.equal(Z2, Zeager), rep


def test_a_call_is_not_ordered_after_a_stream_that_entered_capture(oracle):
    """Calls on different streams are ordered by an event recorded on the earlier call's stream.  When that
    stream has meanwhile entered a capture, such a record would become a node of the caller's graph: the new call
    is refused (FUSEDMM_FAIL_RETURN, nothing enqueued, no device-wide wait), the capture stays valid, and the
    same call goes through once the capture has ended."""
    import torch
    lib = fa.load(64)
    assert lib.fusedMM_amd_init() == 0
    g = graphs.with_values(graphs.tiny_er(300, 2000, 22, bits=64))
    k = 32
    Y = graphs.features(300, k, 6, -0.5, 0.5, 2)
    d = dict(val=_dev(g["val"]), indx=_dev(g["indx"]), pb=_dev(g["pntrb"]), pe=_dev(g["pntre"]), Y=_dev(Y))
    dev = torch.device("cuda:0")

    def enqueue(Z, stream):
        return fa.fusedMM_csr(fa.MSG_SPMM, g["rows"], g["cols"], k, 1.0, g["nnz"], g["rows"], g["cols"], d["val"], d["indx"],
                              d["pb"], d["pe"], None, k, d["Y"], k, 0.0, Z, k, index_bits=64, stream=stream.cuda_stream)

    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    Za = torch.zeros((g["rows"], k), device=dev)
    Zb = torch.full((g["rows"], k), 5.0, device=dev)
    Zw = torch.zeros(16, device=dev)
    torch.cuda.synchronize()
    assert enqueue(Za, s1) == 0                                # eager, on s1: the queues' last user
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s1):                   # s1 enters a capture
        Zw.add_(1.0)
        rc_refused = enqueue(Zb, s2)                           # would have to record an event on s1
    assert rc_refused == fa.FAIL
    torch.cuda.synchronize()
    assert float(Zb.min()) == 5.0 and float(Zb.max()) == 5.0   # nothing ran
    graph.replay()                                             # the capture was left intact
    torch.cuda.synchronize()
    assert float(Zw.sum()) == 16.0
    assert enqueue(Zb, s2) == 0                                # the capture has ended: ordered and run
    torch.cuda.synchronize()
    assert torch.equal(Za, Zb) and float(Za.abs().max()) > 0


def test_capture_never_reallocates_work_queues(oracle):
    """Under HIP graph capture fusedMM_csr_stream refuses a call whose work queues
    would have to grow (replacing them would leave earlier graphs with freed
    addresses); fusedMM_csr_stream_noalloc takes a size it has never seen, because
    its queues are the static array.  Replays are checked against eager results,
    with eager work in between."""
    import torch
    lib = fa.load(64)                                         # a library no other test has given big queues
    assert lib.fusedMM_amd_init() == 0                        # one-time set-up, outside the capture
    g = graphs.ragged(64, rows=300, cols=4000, hub_deg=9000)
    k = 256
    Y = graphs.features(g["cols"], k, 5, -0.5, 0.5, 2)
    d = dict(val=_dev(g["val"]), indx=_dev(g["indx"]), pb=_dev(g["pntrb"]), pe=_dev(g["pntre"]), Y=_dev(Y))
    dev = torch.device("cuda:0")

    def enqueue(Z, noalloc, nnz):
        return fa.fusedMM_csr(fa.MSG_SPMM, g["rows"], g["cols"], k, 1.0, nnz, g["rows"], g["cols"], d["val"], d["indx"],
                              d["pb"], d["pe"], None, k, d["Y"], k, 0.0, Z, k, index_bits=64,
                              stream=torch.cuda.current_stream().cuda_stream, noalloc=noalloc)

    Zeager = torch.zeros((g["rows"], k), device=dev)
    assert enqueue(Zeager, False, g["nnz"]) == 0              # sizes the grown queues for this nnz
    torch.cuda.synchronize()
    assert gpu_api.last_split(64)[1] > 0
    Zg = torch.full((g["rows"], k), 9.0, device=dev)
    Zn = torch.full((g["rows"], k), 9.0, device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        big = enqueue(Zg, False, 50 * g["nnz"])               # would need larger queues: refused, nothing enqueued
        ok = enqueue(Zg, False, g["nnz"])                     # fits what exists
        na = enqueue(Zn, True, g["nnz"])                      # static array: nothing to allocate
    assert big == fa.NOT_ENOUGH_MEM and ok == 0 and na == 0
    for rep in range(3):
        Zg.fill_(float(rep))
        Zn.fill_(float(-rep))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Zg, Zeager) and torch.equal(Zn, Zeager), rep
        Ze2 = torch.zeros_like(Zeager)                        # eager work between replays, both kinds of queues
        assert enqueue(Ze2, False, g["nnz"]) == 0 and enqueue(Ze2, True, g["nnz"]) == 0
        torch.cuda.synchronize()
        assert torch.equal(Ze2, Zeager)


def test_two_host_threads_calling_at_once(oracle):
    """The entry points may be called from several host threads (the reference is
    re-entrant); the library serialises the enqueueing and orders the calls on the
    GPU.  Each thread uses its own stream, operands and output; every result must
    equal the single-threaded one."""
    import threading
    import torch
    g = graphs.ragged(32, rows=400, cols=6000, hub_deg=20000)
    k = 64
    X = graphs.features(g["rows"], k, 3, -0.5, 0.5, 1)
    Ys = [graphs.features(g["cols"], k, 30 + i, -0.5, 0.5, 2) for i in range(3)]
    d = dict(val=_dev(g["val"]), indx=_dev(g["indx"]), pb=_dev(g["pntrb"]), pe=_dev(g["pntre"]), X=_dev(X))
    dY = [_dev(y) for y in Ys]
    gpu_api.set_kind(SOP_NAMES["sigmoid"], 32)

    def enqueue(Y, Z, stream):
        return fa.fusedMM_csr(fa.MSG_SIGMOID, g["rows"], g["cols"], k, 1.0, g["nnz"], g["rows"], g["cols"], d["val"],
                              d["indx"], d["pb"], d["pe"], d["X"], k, Y, k, 0.0, Z, k, stream=stream)

    want = []
    for y in dY:
        Z = torch.zeros((g["rows"], k), device="cuda:0")
        assert enqueue(y, Z, torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        want.append(Z)
    streams = [torch.cuda.Stream() for _ in dY]
    got = [[torch.full((g["rows"], k), 3.0, device="cuda:0") for _ in range(20)] for _ in dY]
    errors = []

    def worker(i):
        for rep in range(20):
            rc = enqueue(dY[i], got[i][rep], streams[i].cuda_stream)
            if rc != 0:
                errors.append((i, rep, rc))

    torch.cuda.synchronize()
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(dY))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for i in range(len(dY)):
        for rep in range(20):
            assert torch.equal(got[i][rep], want[i]), (i, rep)


def test_probes_take_what_they_document(oracle):
    """The measuring aids (copy, read-stream and gather probes) run on well-formed
    arguments and refuse the rest without launching anything."""
    import torch
    lib = fa.load_probes()                                                  # a library of their own
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    src = torch.arange(1 << 20, dtype=torch.float32, device=dev)            # 4 MiB
    dst = torch.zeros_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    assert lib.fusedMM_amd_copy_probe(dst.data_ptr(), src.data_ptr(), src.numel() * 4, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
    assert lib.fusedMM_amd_copy_probe(dst.data_ptr(), src.data_ptr(), 24, st) == fa.FAIL           # not a multiple of 16
    for nt in (0, 1):
        assert lib.fusedMM_amd_read_probe(src.data_ptr(), src.numel() * 4, 4, 8, nt, sink.data_ptr(), st) == 0
    assert lib.fusedMM_amd_read_probe(src.data_ptr() + 4, 1024, 4, 8, 0, sink.data_ptr(), st) == fa.FAIL   # misaligned
    for row_bytes in (16, 128, 256, 1024, 2048):
        rows = src.numel() * 4 // row_bytes
        ids = torch.randint(0, rows, (5000,), device=dev, dtype=torch.int64).to(torch.int32)
        for nt in (0, 1):
            for in_flight in (4, 8, 16):
                assert lib.fusedMM_amd_gather_probe(src.data_ptr(), row_bytes, ids.data_ptr(), ids.numel(), 2, in_flight, nt,
                                                    sink.data_ptr(), st) == 0
    ids = torch.zeros(8, dtype=torch.int32, device=dev)
    for bad in (0, 8, 48, 4096):
        assert lib.fusedMM_amd_gather_probe(src.data_ptr(), bad, ids.data_ptr(), 8, 2, 8, 0, sink.data_ptr(), st) == fa.FAIL
    assert lib.fusedMM_amd_gather_probe(src.data_ptr(), 256, ids.data_ptr(), 0, 2, 8, 0, sink.data_ptr(), st) == fa.FAIL
    torch.cuda.synchronize()
    assert int(sink.abs().sum()) == 0                                       # the probes store nothing
