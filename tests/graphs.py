"""Small seeded graphs shared by the CPU and GPU tests, with the edge cases the
reference's API allows: empty rows, duplicate edges, a hub row, rectangular
matrices, m < rows, and pntrb/pntre that are not rowptr / rowptr+1."""
import numpy as np

from fusedmm_amd import synth


def tiny_er(n=200, pairs=800, seed=11, bits=32):
    return synth.er_graph(n, pairs, seed, bits)


def with_values(g, seed=7):
    g = dict(g)
    g["val"] = synth.edge_values(g["nnz"], seed)
    return g


def ragged(bits=32, seed=3, rows=97, cols=131, hub_deg=600, hub_rows=(11,)):
    """Rectangular, rows 0 and 5 and the last one empty, a duplicate column in
    row 2, one hub row much longer than the rest (with repeats), unsorted row 7."""
    rng = np.random.Generator(np.random.Philox(key=[seed, 0]))
    it = np.int32 if bits == 32 else np.int64
    lists = []
    for r in range(rows):
        if r in (0, 5, rows - 1):
            lists.append(np.empty(0, np.int64))
        elif r == 2:
            lists.append(np.array([4, 9, 9, 30], np.int64) % cols)
        elif r == 7:
            lists.append(np.array([50, 3, 77, 12, 3], np.int64) % cols)
        elif r in hub_rows:
            lists.append(rng.integers(0, cols, hub_deg, dtype=np.int64))
        else:
            d = int(rng.integers(1, 24))
            lists.append(np.sort(rng.choice(cols, d, replace=False)).astype(np.int64))
    deg = np.array([len(x) for x in lists], np.int64)
    rowptr = np.zeros(rows + 1, np.int64)
    np.cumsum(deg, out=rowptr[1:])
    indx = np.concatenate(lists)
    g = synth.graph_from_rowptr(rows, cols, rowptr, indx, None, bits)
    g["val"] = synth.edge_values(g["nnz"], seed)
    assert g["indx"].dtype == it
    return g


def split_pointers(g, seed=5):
    """Same rows, but stored with gaps and in shuffled order: pntrb[i]/pntre[i]
    point into a longer indx/val with junk between rows (pntre[i] != pntrb[i+1])."""
    rng = np.random.Generator(np.random.Philox(key=[seed, 1]))
    rows = g["rows"]
    deg = (g["pntre"] - g["pntrb"]).astype(np.int64)
    order = rng.permutation(rows)
    gap = rng.integers(0, 4, rows)
    total = int(deg.sum() + gap.sum()) + 3
    indx = np.full(total, 0, g["indx"].dtype)       # junk points at a valid row of Y
    val = np.full(total, np.float32(1e30))          # ... but would wreck Z if read
    pb = np.zeros(rows, g["indx"].dtype)
    pe = np.zeros(rows, g["indx"].dtype)
    pos = 3
    for r in order:
        pos += int(gap[r])
        pb[r] = pos
        d = int(deg[r])
        indx[pos:pos + d] = g["indx"][g["pntrb"][r]:g["pntre"][r]]
        val[pos:pos + d] = g["val"][g["pntrb"][r]:g["pntre"][r]]
        pos += d
        pe[r] = pos
    out = dict(g)
    out.update(indx=indx, val=val, pntrb=pb, pntre=pe, nnz=total)
    out.pop("rowptr", None)
    return out


def features(n, k, seed, lo=-0.5, hi=0.5, stream=1):
    return synth.uniform_matrix(n, k, lo, hi, seed, stream)


def partition_cases():
    """Row-degree sets for the nnz-balanced row partition (reference
    fusedMM.c:633-676), as (name, pntrb, pntre, m) with int64 pointers.  Chosen so
    that each step of the rule decides some case: the quota recomputed after
    every closed range, the strict comparison, the tipping row opening the next
    range, the running count restarting at zero, empty rows on either side of a
    boundary, fewer ranges than threads, m < rows, pointers with gaps."""
    cases = []

    def add(name, deg, m=None):
        deg = np.asarray(deg, np.int64)
        ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
        cases.append((name, ptr[:-1].copy(), ptr[1:].copy(), len(deg) if m is None else m))

    add("front_heavy", [10] + [1] * 10)              # quota shrinks after the first range
    add("back_heavy", [1] * 10 + [10])
    add("hand", [3, 1, 1, 1, 3, 1])
    add("hub_last_row", [0, 0, 0, 5])                # fewer ranges than threads
    add("one_row", [7])
    add("all_empty", [0] * 9)
    add("ones16", [1] * 16)
    add("ones17", [1] * 17)
    add("exact_quota", [2, 2, 2, 2, 2, 2])           # running count EQUAL to the quota does not close a range
    add("empties_at_boundaries", [4, 0, 0, 4, 0, 0, 4, 0, 0, 4, 0, 0, 4, 0])
    add("empties_then_tip", [3, 0, 0, 0, 2, 0, 0, 3, 0, 1, 0, 0, 5, 0, 0, 1])
    add("staircase", list(range(1, 40)))
    add("staircase_down", list(range(39, 0, -1)))
    add("m_less_than_rows", [5, 1, 1, 7, 2, 2, 9, 1, 1, 1, 30, 30], m=9)
    rng = np.random.Generator(np.random.Philox(key=[77, 0]))
    for n, cap in ((60, 50), (300, 80), (1000, 400), (2500, 2000)):
        for rep in range(3):
            deg = np.minimum(rng.zipf(1.5 + 0.2 * rep, n), cap)
            deg[rng.random(n) < 0.3] = 0             # R-MAT graphs leave a third of the rows empty
            add("zipf_n%d_%d" % (n, rep), deg)
    for rep in range(3):
        add("geometric_%d" % rep, rng.geometric(0.08, 500) - 1)
    # rows stored with gaps and out of order: only pntre[i] - pntrb[i] may matter
    deg = np.minimum(rng.zipf(1.7, 200), 60)
    order = rng.permutation(200)
    pb, pe = np.zeros(200, np.int64), np.zeros(200, np.int64)
    pos = 3
    for r in order:
        pos += int(rng.integers(0, 4))
        pb[r], pe[r] = pos, pos + int(deg[r])
        pos = int(pe[r])
    cases.append(("gapped_pointers", pb, pe, 200))
    return cases


def udef_stage_tuples():
    """Op tuples in which at least one of VOP, ROP, VSC, AOP is a user function: every
    single such stage with built-in neighbours of each kind, pairs, and all of them
    together, with SOP as a copy, as a user function and absent.  (SOP_NOOP is only
    paired with VSC_NOOP: the reference leaves the scalar uninitialised otherwise,
    fusedMM.c:212-216.)"""
    msgs = []
    builtin = [(0x2, 0x10, 0x100, 0x1000, 0x10000),    # spmm-like with a dot
               (0x5, 0x50, 0xF00, 0x1000, 0x10000),    # the distance tuple
               (0x3, 0x00, 0x100, 0x2000, 0x20000),    # edge value as the scalar, max
               (0x1, 0x30, 0x000, 0x0000, 0x30000),    # no scaling, min
               (0x7, 0x20, 0xF00, 0x2000, 0x10000)]
    udef = (0xF, 0xF0, None, 0xF000, 0xF0000)
    for base in builtin:
        for mask in range(1, 16):
            stages = list(base)
            pos = [0, 1, 3, 4]
            for b in range(4):
                if (mask >> b) & 1:
                    stages[pos[b]] = udef[pos[b]]
            if stages[2] == 0x000 and stages[3] != 0x0000:
                continue
            msgs.append(stages[0] | stages[1] | stages[2] | stages[3] | stages[4])
    msgs.append(0xF | 0xF0 | 0xF00 | 0xF000 | 0x00000)   # no accumulate stage: Z untouched
    return np.array(sorted(set(msgs)), np.int32)


def boundary_graph(bits=32, cols=500, seed=21):
    """For the rule that walks short rows one per sub-wave (gpu_api.packed_rows).  Groups of 8 (and of 4) consecutive rows built around every edge of the rule: all rows at the longest
    length that still packs, one row one edge too long, a single long row among empty ones, all empty, all
    one edge, lengths 1..8 and 57..64, a group that straddles the end of the matrix (the row count is not a
    multiple of 8), and Poisson-like lengths in between."""
    rng = np.random.Generator(np.random.Philox(key=[seed, 0]))
    groups = [
        [64] * 8, [65] + [64] * 7, [64, 0, 0, 0, 0, 0, 0, 0], [8, 0, 0, 0, 0, 0, 0, 0], [9, 0, 0, 0, 0, 0, 0, 0],
        [16, 16, 0, 0, 0, 0, 0, 0], [17, 16, 0, 0, 0, 0, 0, 0], [0] * 8, [1] * 8, [1, 2, 3, 4, 5, 6, 7, 8],
        [57, 58, 59, 60, 61, 62, 63, 64], [32, 32, 32, 32, 0, 0, 0, 0], [33, 32, 32, 32, 1, 1, 1, 1],
        [32, 1, 1, 1, 32, 0, 0, 0], [24, 24, 24, 0, 24, 24, 0, 0], [40, 3, 0, 0, 0, 12, 12, 12],
    ]
    for _ in range(30):
        groups.append(list(rng.poisson(16, 8)))
    for _ in range(10):
        groups.append(list(rng.poisson(4, 8)))
    groups.append([5, 9, 13])              # the last claim is short: rows past m must stay untouched
    deg = np.array([d for grp in groups for d in grp], np.int64)
    rowptr = np.zeros(deg.size + 1, np.int64)
    np.cumsum(deg, out=rowptr[1:])
    indx = rng.integers(0, cols, int(rowptr[-1]), dtype=np.int64)
    g = synth.graph_from_rowptr(deg.size, cols, rowptr, indx, None, bits)
    g["val"] = synth.edge_values(g["nnz"], seed)
    return g


def special_values_case(bits=32, seed=31):
    """Inputs with NaN, infinities and zeros of both signs, for the MAX / MIN stages (the reference's own
    fmax / fmin are the ternaries (x) > (y) ? (x) : (y) and (x) < (y) ? (x) : (y), fusedMM.c:18-19, so a NaN
    on the left loses and a NaN on the right wins, and of two zeros the right one is kept).  Two graphs over
    the same operands: `multi` with ordinary rows (the order of edges matters once a NaN is involved) and
    `single` with at most one edge per row (no order to depend on).  Returns (multi, single, X, Y, Z0, tuples)."""
    rng = np.random.Generator(np.random.Philox(key=[seed, 0]))
    rows, cols, k = 40, 30, 8
    multi = ragged(bits, seed=seed, rows=rows, cols=cols, hub_deg=50)
    deg1 = (rng.random(rows) < 0.8).astype(np.int64)
    rowptr = np.zeros(rows + 1, np.int64)
    np.cumsum(deg1, out=rowptr[1:])
    single = synth.graph_from_rowptr(rows, cols, rowptr, rng.integers(0, cols, int(rowptr[-1]), dtype=np.int64), None, bits)
    single["val"] = synth.edge_values(single["nnz"], seed)
    special = np.array([np.nan, -0.0, 0.0, np.inf, -np.inf, 1.0, -1.0], np.float32)

    def salted(n, stream):
        a = features(n, k, seed, -1, 1, stream)
        hit = rng.random((n, k)) < 0.35
        a[hit] = special[rng.integers(0, special.size, int(hit.sum()))]
        return a
    X, Y, Z0 = salted(rows, 1), salted(cols, 2), salted(rows, 3)
    tuples = []
    for vop in (0x6, 0x7, 0x2):                    # VOP_MAX, VOP_MIN, VOP_COPY_RHS
        for aop in (0x10000, 0x20000, 0x30000):    # AOP_ADD, AOP_MAX, AOP_MIN
            if vop == 0x2 and aop == 0x10000:
                continue
            tuples.append(vop | 0x00 | 0x000 | 0x0000 | aop)        # ROP_NOOP, SOP_NOOP, VSC_NOOP: T goes straight to AOP
            tuples.append(vop | 0x30 | 0x100 | 0x1000 | aop)        # ROP_ADD_RHS, SOP_COPY, VSC_MUL
    return multi, single, X, Y, Z0, np.array(tuples, np.int32)
