"""Edge slots at the end of the index type's range.  The CSR arrays of the
reference's API are addressed by INDEXTYPE slot numbers; the largest int32 slot
range ends at 2^31 - 1, and an int64 library must not squeeze a slot number
through 32 bits anywhere.  The index (and value) arrays are allocated at full
length on the GPU, uninitialised, and only the slots the rows use are filled."""
import numpy as np
import pytest

import fusedmm_amd as fa
import gpu_api
import graphs
from oracle_api import MSG, SOP_NAMES

pytestmark = pytest.mark.gpu


def _case(bits, end_slot, oracle, tkern, kind, k, split=None, validate=False):
    import torch
    dev = torch.device("cuda:0")
    it = np.int32 if bits == 32 else np.int64
    tt = torch.int32 if bits == 32 else torch.int64
    base = graphs.ragged(bits, rows=60, cols=500, hub_deg=4000)          # rows of 0..23 edges and one of 4000
    deg = (base["pntre"] - base["pntrb"]).astype(np.int64)
    used = int(deg.sum())
    first = end_slot - used                                              # the rows occupy slots [first, end_slot)
    assert first > 0
    rowptr = first + np.concatenate([[0], np.cumsum(deg)])
    assert rowptr[-1] == end_slot and end_slot <= np.iinfo(it).max
    pb, pe = rowptr[:-1].astype(it), rowptr[1:].astype(it)
    # device arrays of the full length; everything below `first` stays uninitialised and must never be read
    indx = torch.empty(end_slot, dtype=tt, device=dev)
    val = torch.empty(end_slot, dtype=torch.float32, device=dev)
    cols = np.concatenate([base["indx"][base["pntrb"][r]:base["pntre"][r]] for r in range(base["rows"])]).astype(it)
    vals = np.concatenate([base["val"][base["pntrb"][r]:base["pntre"][r]] for r in range(base["rows"])])
    indx[first:] = torch.from_numpy(cols).to(dev)
    val[first:] = torch.from_numpy(vals).to(dev)
    if first > 1000:                                                     # poison the neighbourhood just below
        indx[first - 1000:first] = 2 ** 30
    X = graphs.features(base["rows"], k, 3, -0.5, 0.5, 1)
    Y = graphs.features(base["cols"], k, 3, -0.5, 0.5, 2)
    Z0 = graphs.features(base["rows"], k, 3, -1, 1, 3)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    dX, dY, dpb, dpe = up(X), up(Y), up(pb), up(pe)
    sk = SOP_NAMES[kind] if kind else 0
    gpu_api.set_kind(sk, bits)
    lib = fa.load(bits)
    if split:
        gpu_api.set_split(*split, bits)
    prev = lib.fusedMM_amd_set_validate(1 if validate else 0)
    # the same rows with pointers starting at zero, for the oracle
    g0 = dict(base)
    g0.update(indx=cols, val=vals, pntrb=(rowptr[:-1] - first).astype(it), pntre=(rowptr[1:] - first).astype(it), nnz=used)
    try:
        for beta in (0.0, 1.0):
            print("case", bits, end_slot, tkern, k, split, "beta", beta, flush=True)
            Z = up(Z0)
            rc = fa.fusedMM_csr(MSG[tkern], base["rows"], base["cols"], k, 1.0, used, base["rows"], base["cols"], val, indx,
                                dpb, dpe, dX, k, dY, k, beta, Z, k, index_bits=bits)
            assert rc == 0
            torch.cuda.synchronize()
            heavy_deg, seg_len = split if split else gpu_api.default_split(k)
            want = gpu_api.oracle_mirror(oracle, tkern, g0, X, Y, Z0, beta, sk, k, heavy_deg, seg_len)
            np.testing.assert_array_equal(Z.cpu().numpy().view(np.uint32), want.view(np.uint32))
    finally:
        lib.fusedMM_amd_set_validate(prev)
        gpu_api.set_split(0, 0, bits)
    del indx, val
    torch.cuda.empty_cache()


@pytest.mark.parametrize("tkern,kind,k,split,validate", [
    ("s", "sigmoid", 128, None, False),          # hub row split at the library's thresholds
    ("m", None, 32, (10, 7), True),              # most rows split into 7-edge segments; operand check on
    ("t", "tdist", 48, None, False),             # masked last slice
])
def test_int32_slots_up_to_the_largest_int32(oracle, tkern, kind, k, split, validate):
    _case(32, 2 ** 31 - 1, oracle, tkern, kind, k, split, validate)


@pytest.mark.parametrize("tkern,kind,k,split,validate", [
    ("s", "sigmoid", 128, None, False),
    ("m", None, 32, (10, 7), True),
])
def test_int64_slots_beyond_32_bits(oracle, tkern, kind, k, split, validate):
    _case(64, 2 ** 32 + 12345, oracle, tkern, kind, k, split, validate)
