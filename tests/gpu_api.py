"""Helpers for the GPU parity tests: run the C ABI on device or host operands
and mirror the library's choice of wavefront layout so the oracle can be asked
for the same summation order."""
import numpy as np

import fusedmm_amd as fa

TKERN_MSG = {"g": fa.MSG_GCN, "m": fa.MSG_SPMM, "s": fa.MSG_SIGMOID, "t": fa.MSG_TDIST, "f": fa.MSG_FR}


def layout_for(k, vec_ok=True):
    """(V, L, S): floats per load, lanes per neighbour row, sub-waves per wave --
    the rule of pick_shape in fusedmm_dispatch.hip."""
    if vec_ok and k % 4 == 0:
        if k <= 32:
            L = 8
        elif k <= 64:
            L = 16
        elif k <= 128:
            L = 32
        else:
            L = 64
        return 4, L, 64 // L
    return 1, 64, 1


MAX_SEGS_PER_ROW = 512   # kMaxSegsPerRow of the kernels: longer rows get longer segments
ROWS_PER_CLAIM = 8       # kRowsPerClaim


def packed_rows(g, m, k, vbits, heavy_deg, vec_ok=True, pack=True):
    """Which of the first m rows the library walks one per sub-wave (packed_group of the kernels): for sub-waves
    of 8 or 16 lanes (K <= 64, 16-byte layout), a group of S = 64/L consecutive rows, groups aligned at multiples
    of S, whose longest row has md <= S*U edges (and is not split) and ceil(md / U) <= (non-empty rows of the
    group).  U is the number of gathers a sub-wave keeps in flight: 8, or 4 in double precision.  Such a row is
    summed over its edges in order in one accumulator."""
    V, L, S = layout_for(k, vec_ok)
    out = np.zeros(m, bool)
    if not pack or V != 4 or L > 16 or m == 0:
        return out
    U = 8 if vbits == 32 else 4
    deg = (g["pntre"][:m].astype(np.int64) - g["pntrb"][:m].astype(np.int64))
    deg = np.maximum(deg, 0)
    pad = (-m) % S
    d2 = np.concatenate([deg, np.zeros(pad, np.int64)]).reshape(-1, S)
    md = d2.max(1)
    nz = (d2 > 0).sum(1)
    ok = (nz > 0) & (md <= S * U) & (md <= heavy_deg) & (-(-md // U) <= nz)
    return np.repeat(ok, S)[:m]


def default_split(k, vbits=32):
    """(heavy_deg, seg_len) defaults of the library for feature width k."""
    seg = max(64, min(2048, 1048576 // ((vbits // 8) * k)))
    return 2 * seg, seg


def run(imsg, g, X, Y, Z, beta=0.0, bits=32, where="device", m=None, k=None, ldx=None, ldy=None, ldz=None,
        nnz=None, vbits=32):
    """Call fusedMM_csr.  where='device': operands copied to the GPU with torch
    and passed as device addresses; 'host': numpy arrays passed as they are.
    Returns (status, Z as numpy)."""
    m = g["rows"] if m is None else m
    k = Y.shape[1] if k is None else k
    ldx = (X.shape[1] if X is not None else k) if ldx is None else ldx
    ldy = Y.shape[1] if ldy is None else ldy
    ldz = Z.shape[1] if ldz is None else ldz
    nnz = g["nnz"] if nnz is None else nnz
    np_v = np.float32 if vbits == 32 else np.float64
    gval = g["val"] if g["val"] is None or g["val"].dtype == np_v else g["val"].astype(np_v)
    assert Y.dtype == np_v and Z.dtype == np_v and (X is None or X.dtype == np_v)
    if where == "host":
        Zh = np.ascontiguousarray(Z).copy()
        rc = fa.fusedMM_csr(imsg, m, g["cols"], k, 1.0, nnz, g["rows"], g["cols"], gval, g["indx"],
                            np.ascontiguousarray(g["pntrb"]), np.ascontiguousarray(g["pntre"]),
                            X, ldx, Y, ldy, beta, Zh, ldz, index_bits=bits, value_bits=vbits)
        return rc, Zh
    import torch
    dev = torch.device("cuda:0")
    t = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    val, indx, pb, pe = t(gval), t(g["indx"]), t(g["pntrb"]), t(g["pntre"])
    Xd, Yd, Zd = t(X), t(Y), t(Z)
    rc = fa.fusedMM_csr(imsg, m, g["cols"], k, 1.0, nnz, g["rows"], g["cols"], val, indx, pb, pe,
                        Xd, ldx, Yd, ldy, beta, Zd, ldz, index_bits=bits, value_bits=vbits)
    torch.cuda.synchronize()
    return rc, Zd.cpu().numpy()


def set_kind(kind, bits=32, vbits=32):
    return fa.load(bits, vbits).fusedMM_amd_set_sop_kind(kind)


def last_split(bits=32, vbits=32):
    import ctypes as C
    h, s, o = C.c_uint(), C.c_uint(), C.c_uint()
    rc = fa.load(bits, vbits).fusedMM_amd_last_split(C.byref(h), C.byref(s), C.byref(o))
    assert rc == 0
    return h.value, s.value, o.value


def oracle_mirror(oracle, tkern, g, X, Y, Z0, beta, sop_kind, k, heavy_deg, seg_len, vec_ok=True, m=None, pack=True, packed=None):
    """What the library computes, operation for operation: rows up to heavy_deg
    edges in wavefront order (short rows that the library walks one per sub-wave, packed_rows(), with a
    single accumulator); longer rows cut into seg_len-edge segments (at
    most MAX_SEGS_PER_ROW per row), each reduced in wavefront order; the merge
    block's G thread groups fold segments g, g+G, ... in ascending order from
    zero, the group sums are added in ascending g, then Z is added when beta != 0."""
    m = g["rows"] if m is None else m
    V, L, S = layout_for(k, vec_ok)
    ot = "t" if tkern == "f" else tkern
    Z = Z0.copy()
    vbits = 32 if Z0.dtype == np.float32 else 64
    if packed is None:      # (a caller checking a window of rows passes the window's part of the whole matrix's mask)
        packed = packed_rows(g, m, k, vbits, heavy_deg, vec_ok, pack)
    if packed.all() and m > 0:
        oracle.opt(ot, g, X, Y, Z, beta=beta, sop_kind=sop_kind, mode=2, V=V, L=L, S=1, m=m, k=k)
    else:
        oracle.opt(ot, g, X, Y, Z, beta=beta, sop_kind=sop_kind, mode=2, V=V, L=L, S=S, m=m, k=k)
        if packed.any():
            # the rows walked one per sub-wave, as a sub-problem of their own: same operands, one accumulator per row
            rows = np.nonzero(packed)[0]
            gp = dict(g)
            gp.update(rows=rows.size, pntrb=np.ascontiguousarray(g["pntrb"][rows]), pntre=np.ascontiguousarray(g["pntre"][rows]))
            Xp = None if X is None else np.ascontiguousarray(X[rows])
            Zp = np.ascontiguousarray(Z0[rows])
            oracle.opt(ot, gp, Xp, Y, Zp, beta=beta, sop_kind=sop_kind, mode=2, V=V, L=L, S=1, k=k)
            Z[rows] = Zp
    deg = (g["pntre"][:m].astype(np.int64) - g["pntrb"][:m].astype(np.int64))
    heavy = np.nonzero(deg > heavy_deg)[0]
    if heavy.size == 0:
        return Z
    pb, pe, owner = [], [], []
    for r in heavy:
        b, e = int(g["pntrb"][r]), int(g["pntre"][r])
        sl = seg_len if (e - b) <= seg_len * MAX_SEGS_PER_ROW else -(-(e - b) // MAX_SEGS_PER_ROW)
        for s0 in range(b, e, sl):
            pb.append(s0)
            pe.append(min(e, s0 + sl))
            owner.append(r)
    it = g["indx"].dtype
    g2 = dict(g)
    g2.update(rows=len(pb), pntrb=np.array(pb, it), pntre=np.array(pe, it))
    X2 = None if X is None else np.ascontiguousarray(X[np.array(owner)])
    np_v = Z0.dtype.type
    P = np.zeros((len(pb), k), np_v)
    oracle.opt(ot, g2, X2, Y, P, beta=0.0, sop_kind=sop_kind, mode=2, V=V, L=L, S=S, k=k)
    owner = np.array(owner)
    G = max(1, 256 // min(k, 256))          # merge kernel: groups of a 256-thread block
    for r in heavy:
        mine = np.nonzero(owner == r)[0]
        total = None
        for grp in range(G):
            a = np.zeros(k, np_v)
            for q in mine[grp::G]:
                a = (a + P[q]).astype(np_v)
            total = a if total is None else (total + a).astype(np_v)
        Z[r, :k] = total if beta == 0.0 else (Z0[r, :k] + total).astype(np_v)
    return Z


def set_split(heavy_deg, seg_len, bits=32, vbits=32):
    fa.load(bits, vbits).fusedMM_amd_set_split(heavy_deg, seg_len)
