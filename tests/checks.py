"""Tolerance rules of the parity tests.

dot/sum ops (gcn, spmm):   |dz| <= 1e-6 + 1e-5 |z|   (+ a degree-scaled rounding
                           term, because a sequential fp32 sum over d edges
                           carries an error of about d * eps * sum|terms|)
sigmoid / t-dist / FR:     |dz| <= 1e-6 + 1e-4 |z|   likewise, and for the table
                           sigmoid an edge whose dot product lies within the
                           rounding uncertainty of a table-bin boundary may
                           take the neighbouring entry.
"""
import numpy as np

EPS32 = float(np.finfo(np.float32).eps)


def edge_rows(g, m=None):
    m = g["rows"] if m is None else m
    pb = np.asarray(g["pntrb"][:m], np.int64)
    pe = np.asarray(g["pntre"][:m], np.int64)
    deg = pe - pb
    rows = np.repeat(np.arange(m, dtype=np.int64), deg)
    # slot index of every edge of every processed row
    start = np.repeat(pb - np.concatenate([[0], np.cumsum(deg)[:-1]]), deg)
    slots = np.arange(int(deg.sum()), dtype=np.int64) + start
    return rows, slots


def abs_term_sum(tkern, g, X, Y, d_abs, m=None):
    """sum over edges of |d_j| * |vector_j| per row: the scale of the rounding error."""
    rows, slots = edge_rows(g, m)
    cols = np.asarray(g["indx"], np.int64)[slots]
    m = g["rows"] if m is None else m
    out = np.zeros((m, Y.shape[1]), np.float64)
    vec = np.abs(Y[cols].astype(np.float64))
    if tkern in ("t", "f"):
        vec = np.abs(X[rows].astype(np.float64) - Y[cols].astype(np.float64))
    np.add.at(out, rows, vec * d_abs[:, None])
    return out


def sigmoid_flip_slack(table, g, X, Y, m=None):
    """Per element: how much Z may move if every edge whose fp64 dot lies within
    the fp32 rounding uncertainty of a bin boundary took the neighbouring entry."""
    rows, slots = edge_rows(g, m)
    cols = np.asarray(g["indx"], np.int64)[slots]
    m = g["rows"] if m is None else m
    k = Y.shape[1]
    xr = X[rows].astype(np.float64)
    yc = Y[cols].astype(np.float64)
    s = np.einsum("ij,ij->i", xr, yc)
    unc = (k + 8) * EPS32 * np.einsum("ij,ij->i", np.abs(xr), np.abs(yc)) + 1e-7
    pos = (s + 5.0) * 204.8
    frac = pos - np.floor(pos)
    dist = np.minimum(frac, 1.0 - frac) / 204.8          # distance to a boundary, in s units
    near = (dist <= unc) & (np.abs(s) <= 5.0 + unc)
    b = np.clip(np.floor(pos).astype(np.int64), 0, 2047)
    t = table.astype(np.float64)
    lo = np.clip(b - 1, 0, 2047)
    hi = np.clip(b + 1, 0, 2047)
    jump = np.maximum(np.abs(t[b] - t[lo]), np.abs(t[hi] - t[b]))
    # at the +-5 ends the neighbour is the saturated branch (0 or 1)
    jump = np.where(np.abs(s) > 5.0 - unc, np.maximum(jump, 0.0067), jump)
    slack = np.zeros((m, k), np.float64)
    np.add.at(slack, rows[near], jump[near, None] * np.abs(yc[near]))
    return slack, int(near.sum())


def assert_close(z, zref, rtol, atol, extra=None, what=""):
    z = np.asarray(z, np.float64)
    zref = np.asarray(zref, np.float64)
    bound = atol + rtol * np.abs(zref)
    if extra is not None:
        bound = bound + extra
    bad = ~(np.abs(z - zref) <= bound)
    if bad.any():
        i = np.argwhere(bad)[0]
        raise AssertionError("%s: %d elements outside tolerance; first at %s: got %r want %r (bound %g)" % (
            what, int(bad.sum()), tuple(i), z[tuple(i)], zref[tuple(i)], bound[tuple(i)]))
