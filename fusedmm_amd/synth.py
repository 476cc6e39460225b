"""Seeded synthetic graphs and embeddings for the benchmark configurations.

Everything is drawn from numpy's counter-based Philox generator, so the same
(seed, shape) gives the same bytes on any host.  Graphs come back as a dict:

    rows, cols, nnz   sizes of the sparse matrix
    rowptr            [rows+1] row pointer;  pntrb = rowptr[:-1], pntre = rowptr[1:]
    indx              [nnz] column ids, ascending inside each row
    val               [nnz] fp32 edge values

Column ids ascending per row, duplicates removed, no self-loops: the layout the
reference's loader produces for a symmetric pattern file
(test/include/IO.h:127-143, CSR.h:154-186).
"""
import numpy as np


def _rng(seed, stream=0):
    return np.random.Generator(np.random.Philox(key=[int(seed), int(stream)]))


def graph_from_rowptr(rows, cols, rowptr, indx, val=None, index_bits=32):
    it = np.int32 if index_bits == 32 else np.int64
    rowptr = np.ascontiguousarray(rowptr, it)
    indx = np.ascontiguousarray(indx, it)
    nnz = int(indx.size)
    if val is None:
        val = np.ones(nnz, np.float32)
    return {"rows": int(rows), "cols": int(cols), "nnz": nnz, "rowptr": rowptr,
            "pntrb": rowptr[:-1], "pntre": rowptr[1:], "indx": indx,
            "val": np.ascontiguousarray(val, np.float32)}


def _csr_from_keys(n, keys, index_bits):
    """keys = row*n + col, unique and sorted -> CSR with ascending columns."""
    r = keys // n
    c = keys - r * n
    counts = np.bincount(r, minlength=n)
    rowptr = np.zeros(n + 1, np.int64)
    np.cumsum(counts, out=rowptr[1:])
    return graph_from_rowptr(n, n, rowptr, c, None, index_bits)


def _symmetrise(n, u, v, index_bits):
    keep = u != v
    u, v = u[keep].astype(np.int64), v[keep].astype(np.int64)
    keys = np.concatenate([u * n + v, v * n + u])
    keys = np.unique(keys)
    return _csr_from_keys(n, keys, index_bits)


def er_graph(n, undirected_pairs, seed, index_bits=32):
    """Symmetric Erdos-Renyi G(n, M): exactly `undirected_pairs` distinct pairs
    u != v, so nnz = 2 * undirected_pairs."""
    rng = _rng(seed)
    have = np.empty(0, np.int64)
    while have.size < undirected_pairs:
        need = undirected_pairs - have.size
        draw = int(need * 1.05) + 16
        u = rng.integers(0, n, draw, dtype=np.int64)
        v = rng.integers(0, n, draw, dtype=np.int64)
        ok = u != v
        lo = np.minimum(u[ok], v[ok])
        hi = np.maximum(u[ok], v[ok])
        new = np.unique(hi * n + lo)
        if have.size:
            new = new[~np.isin(new, have, assume_unique=True)]
        if new.size > need:  # drop a seeded random subset, not the largest keys
            new = new[np.sort(rng.permutation(new.size)[:need])]
        have = np.union1d(have, new)
    hi = have // n
    lo = have - hi * n
    return _symmetrise(n, hi, lo, index_bits)


def rmat_graph(scale, edge_factor, seed, a=0.57, b=0.19, c=0.19, d=0.05, index_bits=32,
               chunk=1 << 24):
    """R-MAT: edge_factor * 2^scale sampled edges, self-loops dropped,
    symmetrised, duplicates removed, columns sorted."""
    n = 1 << scale
    total = edge_factor * n
    rng = _rng(seed)
    parts = []
    done = 0
    while done < total:
        cnt = min(chunk, total - done)
        u = np.zeros(cnt, np.int64)
        v = np.zeros(cnt, np.int64)
        for _ in range(scale):
            r = rng.random(cnt, dtype=np.float32)
            right = (r >= a) & (r < a + b) | (r >= a + b + c)  # quadrants b, d
            down = r >= a + b                                  # quadrants c, d
            u = (u << 1) | down
            v = (v << 1) | right
        keep = u != v
        u, v = u[keep], v[keep]
        parts.append(np.unique(np.concatenate([u * n + v, v * n + u])))
        done += cnt
    keys = parts[0] if len(parts) == 1 else np.unique(np.concatenate(parts))
    return _csr_from_keys(n, keys, index_bits)


def zipf_graph(n, exponent, cap, target_nnz, seed, index_bits=32, n_hubs=4):
    """Power-law out-degrees: deg_i ~ Zipf(exponent) capped at `cap`, the
    mid-range rescaled so the total is about target_nnz; `n_hubs` rows are set
    to the cap so the load-balance stress is always present.  Neighbours are
    uniform, distinct within a row, never the row itself, sorted."""
    rng = _rng(seed)
    cap = min(cap, n - 1)
    deg = np.minimum(rng.zipf(exponent, n).astype(np.int64), cap)
    hubs = np.sort(rng.choice(n, n_hubs, replace=False))
    deg[hubs] = 0
    tot = int(deg.sum())
    budget = max(n, target_nnz - n_hubs * cap)
    if tot > budget:
        deg = np.maximum(1, (deg * (budget / tot)).astype(np.int64))
    deg[hubs] = 0
    rows_rep = np.repeat(np.arange(n, dtype=np.int64), deg)
    draw = rng.integers(0, n - 1, rows_rep.size, dtype=np.int64)
    draw += draw >= rows_rep                       # skip the diagonal
    parts = [np.unique(rows_rep * n + draw)]       # duplicates inside a row collapse
    for h in hubs:
        pick = rng.permutation(n - 1)[:cap].astype(np.int64)
        pick += pick >= h
        parts.append(h * n + np.sort(pick))
    keys = np.sort(np.concatenate(parts))
    return _csr_from_keys(n, keys, index_bits)


def uniform_degree_graph(n, m, degree, seed, index_bits=32):
    """m rows of exactly `degree` uniformly random neighbours among n columns
    (unsorted, repeats possible): every row costs the same, so what a row
    length costs can be read off a run."""
    rng = _rng(seed)
    indx = rng.integers(0, n, m * degree, dtype=np.int64)
    rowptr = np.arange(m + 1, dtype=np.int64) * degree
    return graph_from_rowptr(m, n, rowptr, indx, None, index_bits)


def uniform_matrix(n, k, lo, hi, seed, stream=1):
    rng = _rng(seed, stream)
    out = rng.random((n, k), dtype=np.float32)
    out *= np.float32(hi - lo)
    out += np.float32(lo)
    return out


def normal_matrix(n, k, seed, stream=1):
    return _rng(seed, stream).standard_normal((n, k), dtype=np.float32)


def edge_values(nnz, seed, stream=2):
    """fp32 uniform on (0, 1]."""
    return (np.float32(1.0) - _rng(seed, stream).random(nnz, dtype=np.float32)).astype(np.float32)


def write_mtx_symmetric(path, g):
    """Write the lower triangle of a symmetric pattern graph as a MatrixMarket
    `coordinate pattern symmetric` file (1-based, row > col)."""
    n = g["rows"]
    rowid = np.repeat(np.arange(n, dtype=np.int64), np.diff(g["rowptr"]).astype(np.int64))
    col = g["indx"].astype(np.int64)
    low = rowid > col
    r, c = rowid[low] + 1, col[low] + 1
    with open(path, "w") as f:
        f.write("%%MatrixMarket matrix coordinate pattern symmetric\n")
        f.write("%d %d %d\n" % (n, n, r.size))
        np.savetxt(f, np.stack([r, c], 1), fmt="%d")


def algorithmic_bytes(kind, m, k, nnz, index_bytes=4, beta_nonzero=False, value_bytes=4):
    """Bytes one call must move if nothing is reused: every edge gathers a full
    Y row plus its column id (and value for spmm); every row reads X once (ops
    that use X), both row pointers, and writes Z once."""
    F = value_bytes
    vb = F if kind == "m" else 0
    xb = F * k if kind in ("s", "t", "f") else 0
    zb = F * k * (2 if beta_nonzero else 1)
    return nnz * (F * k + index_bytes + vb) + m * (xb + zb + 2 * index_bytes)


def algorithmic_flops(kind, k, nnz):
    """Flop convention of the reference's tester (test/fusedMMtime.cpp:806-831)."""
    per_edge = {"s": 4 * k, "t": 5 * k, "f": 5 * k, "m": 2 * k, "g": k}[kind]
    return per_edge * nnz
