#!/usr/bin/env python3
"""Benchmark of the fused SDDMM+SpMM hot path (fusedMM_csr) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2]

A step is one fusedMM_csr call over the whole synthetic graph, operands already
resident in HBM.  Prints ONE JSON line.  The default workload is the one the
headline metric is quoted on: the sigmoid graph-embedding op at K=128 on a
symmetric Erdos-Renyi graph with 2^20 nodes and 2^24 edges, int32 indices.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBPS = 8000.0

# Bytes per call that crossed the L2 <-> data-fabric boundary, from rocprofv3 --pmc
# FETCH_SIZE and WRITE_SIZE, each scaled by the same counter's reading for a plain
# 1 GiB copy: measured, not computed, and kept in the rocprofv3 summary of each
# workload under profiles/ (the line "traffic_bytes_per_call: N"), where this reads it.
# These counters sit at the L2: what they count is served by HBM or by the 256 MiB
# last-level (Infinity) cache behind the fabric, so on a workload whose Y partly fits
# that cache (c2: 512 MiB) the figure is an upper bound on HBM bytes, not HBM bytes.
TRAFFIC_IS = ("L2-miss (fabric) bytes per call: FETCH_SIZE + WRITE_SIZE scaled by a 1 GiB copy; served by HBM or by the "
              "256 MiB last-level cache, so an upper bound on HBM bytes")
# Extra workloads of the default run, measured after the headline one and reported under "also":
# the second configuration with a bandwidth target (gcn K=256), then the skewed ones, then the middle of the reference's
# own sweep of feature widths at HBM scale (K=128 on 2^23 nodes: nothing to reuse, nothing that fits a cache).
ALSO_DEFAULT = ("c3g", "c3", "c4", "c5", "k128er")   # c3g and c3 share a graph
PROFILE_OF = {"c2": "fused_kernel_sigmoid_k128_c2.md", "c3": "spmm_k256_c3_rmat22.md",
              "c3g": "gcn_k256_c3g_rmat22.md", "c4": "tdist_k64_c4_rmat24.md", "c5": "sigmoid_k512_c5_zipf.md",
              "k32er": "tdist_k32_k32er.md", "k64er": "tdist_k64_k64er.md", "k128er": "tdist_k128_k128er.md",
              "k256er": "tdist_k256_k256er.md"}


def measured_traffic_bytes(workload):
    """(bytes per call, profile file) from the committed rocprofv3 summary, or (None, None)."""
    name = PROFILE_OF.get(workload)
    path = os.path.join(ROOT, "profiles", name) if name else None
    if not path or not os.path.exists(path):
        return None, None
    for line in open(path):
        if line.startswith("traffic_bytes_per_call:"):
            return int(line.split(":")[1].split()[0]), "profiles/" + name
    return None, None

WORKLOADS = {
    # name: (description, op letter, K, sop kind)
    "c1": ("fr K=32, ER n=16384 nnz=262144 (cache-resident plumbing case)", "f", 32, "fr"),
    "c2": ("sigmoid K=128, ER n=2^20 nnz=2^24, int32", "s", 128, "sigmoid"),
    "c3": ("spmm K=256, R-MAT scale 22 edge factor 16, symmetrised", "m", 256, None),
    "c3g": ("gcn K=256, R-MAT scale 22 edge factor 16, symmetrised", "g", 256, None),
    "c4": ("tdist K=64, R-MAT scale 24 edge factor 16, symmetrised", "t", 64, "tdist"),
    "c4g": ("gcn K=64 on the c4 graph (same gathers, no reduction or scalar op)", "g", 64, None),
    "c5": ("sigmoid K=512, Zipf(1.8) degrees n=2^21 nnz~4e7, hubs to 1e6", "s", 512, "sigmoid"),
}
# The reference's own sweep is K = 32 ... 256 in steps of 32 (runtime.sh:21-25), on graphs of its users' choosing.  Here, at
# HBM scale: t-dist over an ER graph of 2^23 nodes with 2^27 edges, Y of K/32 GiB (K=32: 128-byte rows out of 1 GiB):
# nothing fits a cache.  k32er and k64er are the narrow rows, a wavefront holding 8 and 4 neighbour rows at a time.
for _k in range(32, 257, 32):
    WORKLOADS["k%der" % _k] = ("tdist K=%d, ER n=2^23 nnz=2^27 (%d-byte rows, Y of %g GiB)" % (_k, 4 * _k, _k / 32.0),
                               "t", _k, "tdist")
    # the same graph and embeddings under the gcn tuple (gathers and adds only) and the sigmoid tuple
    WORKLOADS["g%der" % _k] = ("gcn K=%d on the k%der graph" % (_k, _k), "g", _k, None)
    WORKLOADS["s%der" % _k] = ("sigmoid K=%d on the k%der graph" % (_k, _k), "s", _k, "sigmoid")
# What a row length costs: sigmoid K=512 over a Y of 2^21 rows (c5's), every row with the
# same number of uniformly random neighbours, min(2^21, 2^25 / degree) rows.
for _d in (1, 4, 16, 64, 512):
    WORKLOADS["u512d%d" % _d] = ("sigmoid K=512, %d rows of %d uniform neighbours each among 2^21" % (
        min(1 << 21, (1 << 25) // _d), _d), "s", 512, "sigmoid")


def make_workload(name, scale_down=0):
    """Graph + embeddings of a benchmark configuration.  scale_down shrinks the
    node count by 2^scale_down (used by the tests, never by the default bench)."""
    from fusedmm_amd import synth
    sd = scale_down
    if name == "c1":
        n = 16384 >> sd
        g = synth.er_graph(n, 8 * n, 1)
        X = synth.uniform_matrix(n, 32, -1.0, 1.0, 1)
        return g, X, X
    if name == "c2":
        n = (1 << 20) >> sd
        g = synth.er_graph(n, 8 * n, 2)
        return g, synth.uniform_matrix(n, 128, -0.5, 0.5, 2, 1), synth.uniform_matrix(n, 128, -0.5, 0.5, 2, 2)
    if name in ("c3", "c3g"):
        g = synth.rmat_graph(22 - sd, 16, 3)
        g["val"] = synth.edge_values(g["nnz"], 3)
        return g, None, synth.normal_matrix(g["rows"], 256, 3)
    if name in ("c4", "c4g"):
        g = synth.rmat_graph(24 - sd, 16, 4)
        n = g["rows"]
        return g, synth.uniform_matrix(n, 64, -1.0, 1.0, 4, 1), synth.uniform_matrix(n, 64, -1.0, 1.0, 4, 2)
    if name == "c5":
        n = (1 << 21) >> sd
        g = synth.zipf_graph(n, 1.8, min(1000000, n // 2), 40000000 >> sd, 5)
        return g, synth.uniform_matrix(n, 512, -0.5, 0.5, 5, 1), synth.uniform_matrix(n, 512, -0.5, 0.5, 5, 2)
    if name[0] in "kgs" and name.endswith("er") and name[1:-2].isdigit():
        n = (1 << 23) >> sd
        k = int(name[1:-2])
        g = synth.er_graph(n, 8 * n, 7)
        lim = 1.0 if name[0] != "s" else 2.0 / np.sqrt(k)          # sigmoid: keep the dots inside the table's range
        return g, synth.uniform_matrix(n, k, -lim, lim, 7, 1), synth.uniform_matrix(n, k, -lim, lim, 7, 2)
    if name.startswith("u512d"):
        d = int(name[5:])
        n = (1 << 21) >> sd
        m = min(n, ((1 << 25) >> sd) // d)
        g = synth.uniform_degree_graph(n, m, d, 6)
        return g, synth.uniform_matrix(m, 512, -0.5, 0.5, 6, 1), synth.uniform_matrix(n, 512, -0.5, 0.5, 6, 2)
    raise SystemExit("unknown workload %s" % name)


def physical_cores():
    """Physical cores of this host as lscpu counts them (sockets x cores per socket), or None."""
    import subprocess
    try:
        txt = subprocess.run(["lscpu"], stdout=subprocess.PIPE, text=True, timeout=10).stdout
        f = {}
        for line in txt.splitlines():
            if ":" in line:
                a, b = line.split(":", 1)
                f[a.strip()] = b.strip()
        return int(f["Socket(s)"]) * int(f["Core(s) per socket"])
    except Exception:
        return None


def sample_problem(g, X, edge_budget, seed=17):
    """A sub-problem of about edge_budget edges for the CPU legs: the whole graph when it is that small, else rows
    drawn uniformly at random (seeded) from all over the matrix, kept in ascending order, with their X rows; Y and
    the CSR arrays are the workload's own (pntrb / pntre of the chosen rows: m < rows and separate row pointers are
    part of the API).  Returns (graph dict, X, rows chosen or None)."""
    rows = g["rows"]
    if g["nnz"] <= edge_budget:
        return g, X, None
    deg = (g["pntre"][:rows].astype(np.int64) - g["pntrb"][:rows].astype(np.int64))
    order = np.random.Generator(np.random.Philox(key=[seed, 0])).permutation(rows)
    take = int(np.searchsorted(np.cumsum(deg[order]), edge_budget, side="right"))
    pick = np.sort(order[:max(1, take)])
    sub = dict(g)
    sub.update(rows=int(pick.size), pntrb=np.ascontiguousarray(g["pntrb"][pick]), pntre=np.ascontiguousarray(g["pntre"][pick]))
    sub.pop("rowptr", None)
    return sub, (None if X is None else np.ascontiguousarray(X[pick])), pick


def cpu_baseline(name, g, X, Y, tkern, kind_id, k, budget_s=12.0):
    """The CPU legs, timed on this host's cores on a bounded sample of the same workload (sample_problem):
    the oracle's OpenMP port of the optimised semantics (the headline CPU figure), and beside it the real
    reference's general fusedMM_csr where oracle/_ref was built, both on the same number of threads.
    Checker-side code: used here only to report a baseline."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from oracle_api import Oracle, Ref, ref_available, ref_threads_for
    from fusedmm_amd import synth
    orc = Oracle(fast=True)
    cores = physical_cores()
    # the threads this process may use: OpenMP's own limit (OMP_NUM_THREADS, cgroup share), not above the physical cores
    threads = orc.max_threads()
    if cores:
        threads = max(1, min(threads, cores))
    rows = g["rows"]
    # about 5e7 edges/s on 8 cores at K=128: size the sample for a few calls inside the budget
    gs, Xs, pick = sample_problem(g, X, int(2.5e9 / k))
    m = gs["rows"]
    nnz_s = int((gs["pntre"][:m].astype(np.int64) - gs["pntrb"][:m].astype(np.int64)).sum())
    Z = np.zeros((m, k), np.float32)
    ot = "t" if tkern == "f" else tkern
    orc.baseline(ot, gs, Xs, Y, Z, 0.0, kind_id, threads, m=m)  # warm-up, untimed
    t_all = []
    t0 = time.time()
    while (len(t_all) < 3 or time.time() - t0 < budget_s) and len(t_all) < 200:
        t1 = time.time()
        orc.baseline(ot, gs, Xs, Y, Z, 0.0, kind_id, threads, m=m)
        t_all.append(time.time() - t1)
    t, t_min = float(np.mean(t_all)), float(np.min(t_all))
    flops = synth.algorithmic_flops(tkern, k, nnz_s)
    what = ("the whole graph" if pick is None else
            "%d of %d rows drawn uniformly at random from the whole matrix (seed 17), in ascending order" % (m, rows))
    out = {"value": flops / t / 1e9, "unit": "GFLOP/s", "cores": threads, "kind": "port",
           "value_best_call": flops / t_min / 1e9,
           "sample": "%s: %d of %d edges, %d calls, mean %.4f s/call, min %.4f; OpenMP restatement of the optimised "
                     "semantics built -O3 -march=%s" % (what, nnz_s, g["nnz"], len(t_all), t, t_min, orc.isa),
           "omp_max_threads": orc.max_threads(), "lscpu_physical_cores": cores,
           "s_per_call": {"mean": t, "min": t_min},
           "edges_per_s": nnz_s / t,
           "alg_GBps": synth.algorithmic_bytes(tkern, m, k, nnz_s) / t / 1e9}
    # the real reference's general pipeline (fusedMM.c compiled where it lies; its build bakes the OpenMP team size
    # in, so the library built for the thread count used above is loaded) on the same sample
    ref_kind = {"s": "sigmoid", "t": "tdist", "f": "fr", "m": "spmm", "g": "gcn"}[tkern]
    ref_threads = ref_threads_for(threads)
    if ref_available(ref_kind, 32, 32, ref_threads):
        from oracle_api import MSG
        ref = Ref(ref_kind, 32, 32, ref_threads)
        Zr = np.zeros((m, k), np.float32)
        Xr = Xs if Xs is not None else Y
        ref.fusedMM_csr(MSG[tkern], gs, Xr, Y, Zr, 0.0, m=m)       # warm-up
        tr = []
        t0 = time.time()
        while (len(tr) < 2 or time.time() - t0 < 0.6 * budget_s) and len(tr) < 50:
            Zr[:] = 0
            t1 = time.time()
            ref.fusedMM_csr(MSG[tkern], gs, Xr, Y, Zr, 0.0, m=m)
            tr.append(time.time() - t1)
        tm, tmin = float(np.mean(tr)), float(np.min(tr))
        out["reference_general"] = {"kind": "reference-general", "value": flops / tm / 1e9, "unit": "GFLOP/s",
                                    "value_best_call": flops / tmin / 1e9,
                                    "cores": ref_threads, "edges_per_s": nnz_s / tm, "s_per_call": {"mean": tm, "min": tmin},
                                    "sample": "same sample; the reference's general fusedMM_csr (five indirect stage calls "
                                              "per edge, built -fopenmp -O3 with NTHREADS=%d), %d calls, mean %.4f s/call, "
                                              "min %.4f; its optimised kernels are generated code and are not built here"
                                              % (ref_threads, len(tr), tm, tmin)}
    return out


def parse_args(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS),
                    help="c1-c5: the benchmark configurations (c2 is the one the metric is quoted on); c3g, c4g: the gcn "
                         "tuple on the c3 and c4 graphs; k<K>er, K = 32 ... 256: the reference's sweep of feature widths at HBM scale; u512d<D>: uniform-degree "
                         "rows at c5's row size (a measuring aid)")
    ap.add_argument("--also", default="auto",
                    help="comma-separated workloads measured after the headline one and reported, compactly, under "
                         "\"also\" in the same JSON line (each with its own roofline figures and spot check); 'auto' = "
                         + ",".join(ALSO_DEFAULT) + " for the default run (c2, float, int32, optimised kernels), none "
                         "otherwise; 'none' switches it off")
    ap.add_argument("--also-steps", type=int, default=10, help="timed steps of each extra workload (2 warm-up steps)")
    ap.add_argument("--dtype", default="f32", choices=["f32", "f64"],
                    help="f64 runs the double-precision library (the reference's -DDREAL build)")
    ap.add_argument("--index-bits", type=int, default=32, choices=[32, 64],
                    help="64 runs the int64 library (the reference's default INDEXTYPE) on the same graph")
    ap.add_argument("--general", action="store_true",
                    help="switch the optimised-tuple match off (fusedMM_amd_set_opt(0)): the same tuple goes through "
                         "the general five-stage pipeline, which accumulates into Z")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-check", action="store_true", help="skip the spot check against the oracle")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch a plain 1 GiB copy kernel (yardstick for rocprofv3 --pmc FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--kernel-events-every", type=int, default=4,
                    help="record per-kernel HIP events on every n-th timed step (0: none).  An event record between "
                         "two kernels keeps them from being dispatched back to back, about 20 us per step, so the "
                         "timed region samples rather than instruments every step")
    ap.add_argument("--read-probe", action="store_true",
                    help="also time a read-only stream over 4 GiB (what the memory system delivers to reads alone) and report it")
    ap.add_argument("--ldz", type=int, default=0,
                    help="leading dimension of Z in elements (default K): rows of Z further apart in memory")
    ap.add_argument("--gather-probe", action="store_true",
                    help="time a read-only gather of uniformly random rows of the workload's row size from a buffer "
                         "the size of its Y (what the memory system delivers to such gathers alone) and report it; "
                         "always on for the default run and its extra workloads")
    return ap.parse_args(argv)


# Launch shapes of the gather probe: (workgroups per CU, gathers in flight per wavefront).  4 x 8 is the shape of
# the fused kernel itself; 8 x 4, twice the waves each with half the queue, is the best of a sweep over 2-16 x 4-16 at
# every row size from 128 bytes to 1 KiB.  The yardstick is the better of the two.
GATHER_PROBE_SHAPES = ((4, 8), (8, 4))


def run_gather_probe(torch, probes, n, row_bytes, stream):
    """Read-only gather of 4 GiB of uniformly random rows of row_bytes out of a buffer of n rows: the best rate over
    GATHER_PROBE_SHAPES for plain and for non-temporal loads, and every shape's own figures under "shapes"."""
    dev = torch.device("cuda:0")
    nbytes = n * row_bytes
    src = torch.empty(nbytes // 4, dtype=torch.float32, device=dev).uniform_(-1, 1)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    n_ids = (4 << 30) // row_bytes
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)
    ids = torch.randint(0, n, (n_ids,), device=dev, dtype=torch.int64, generator=gen).to(torch.int32)
    out = {"row_bytes": row_bytes, "buffer_bytes": nbytes, "gathered_bytes": n_ids * row_bytes, "shapes": {}}
    for per_cu, in_flight in GATHER_PROBE_SHAPES:
        shape = out["shapes"].setdefault("%dx%d" % (per_cu, in_flight), {})
        for label, nt in (("plain_loads", 0), ("nontemporal_loads", 1)):
            launch = lambda: probes.fusedMM_amd_gather_probe(src.data_ptr(), row_bytes, ids.data_ptr(), n_ids, per_cu,
                                                             in_flight, nt, sink.data_ptr(), stream)
            for _ in range(2):
                assert launch() == 0
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                launch()
            e1.record()
            torch.cuda.synchronize()
            shape[label + "_GBps"] = n_ids * row_bytes / (e0.elapsed_time(e1) / 10 * 1e-3) / 1e9
            out[label + "_GBps"] = max(out.get(label + "_GBps", 0.0), shape[label + "_GBps"])
    del src, sink, ids
    return out


def run_read_probe(torch, probes, stream):
    dev = torch.device("cuda:0")
    nbytes = 4 << 30
    src = torch.empty(nbytes // 4, dtype=torch.float32, device=dev).uniform_(-1, 1)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    out = {"bytes": nbytes}
    for label, nt in (("plain_loads", 0), ("nontemporal_loads", 1)):
        for _ in range(2):
            assert probes.fusedMM_amd_read_probe(src.data_ptr(), nbytes, 16, 8, nt, sink.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            probes.fusedMM_amd_read_probe(src.data_ptr(), nbytes, 16, 8, nt, sink.data_ptr(), stream)
        e1.record()
        torch.cuda.synchronize()
        out[label + "_GBps"] = nbytes / (e0.elapsed_time(e1) / 10 * 1e-3) / 1e9
    del src, sink
    return out


_graphs = {}


def workload_data(name):
    """make_workload(), the graph shared by workloads that differ in the op tuple only (c3/c3g, c4/c4g)."""
    key = {"c3g": "c3", "c4g": "c4"}.get(name, name)
    if name[0] == "g" and name.endswith("er"):
        key = "k" + name[1:]
    if key not in _graphs:
        _graphs.clear()                     # one graph at a time: the large ones take several GB of host memory
        _graphs[key] = cached_workload(key)
    return _graphs[key]


def cached_workload(key):
    """make_workload(), or its result from a directory named by BENCH_WORKLOAD_CACHE (for repeated runs of the
    same workload on one box, e.g. one per hardware-counter group; the default run never sets it)."""
    cache = os.environ.get("BENCH_WORKLOAD_CACHE")
    path = os.path.join(cache, key + ".npz") if cache else None
    if path and os.path.exists(path):
        d = np.load(path)
        g = {k[2:]: (int(d[k]) if d[k].ndim == 0 else d[k]) for k in d.files if k.startswith("g_")}
        g["pntrb"], g["pntre"] = g["rowptr"][:-1], g["rowptr"][1:]
        X = d["X"] if "X" in d.files else None
        Y = X if "Y" not in d.files else d["Y"]
        return g, X, Y
    g, X, Y = make_workload(key)
    if path:
        os.makedirs(cache, exist_ok=True)
        arrs = {"g_" + k: v for k, v in g.items() if k not in ("pntrb", "pntre")}
        if X is not None:
            arrs["X"] = X
        if Y is not X:
            arrs["Y"] = Y
        np.savez(path, **arrs)
    return g, X, Y


def spot_check(torch, name, g, X, Y, d_Z, k, ldz, tkern, kind_id, vbits, general, step):
    """A window of rows from the middle of the matrix plus the longest row, against the oracle (checker only):
    bit for bit for the optimised kernels, to the parity tests' tolerance for the general pipeline."""
    m = g["rows"]
    np_v = np.float32 if vbits == 32 else np.float64
    if general:
        # the general rule folded every step into Z; one more step on a cleared Z is
        # what the oracle (Z0 = 0) is compared with
        d_Z.zero_()
        step()
        torch.cuda.synchronize()
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from oracle_api import Oracle
    from gpu_api import oracle_mirror, default_split, packed_rows
    orc = Oracle(vbits=vbits)
    heavy_deg, seg_len = default_split(k, vbits)
    # which rows were walked one per sub-wave: decided on groups of rows of the whole matrix (FUSEDMM_PACK_ROWS=off: none)
    packed_all = packed_rows(g, m, k, vbits, heavy_deg, pack=os.environ.get("FUSEDMM_PACK_ROWS", "auto") != "off")
    deg = np.diff(g["rowptr"])
    windows = [(m // 2, min(m, m // 2 + 1024))]
    hub = int(np.argmax(deg))
    # (the general pipeline's tolerance check holds a row's terms in double precision: rows to 10^5 edges)
    if deg[hub] <= (100000 if general else 1200000):
        windows.append((hub, hub + 1))
    ok = True
    for lo, hi in windows:
        sub = dict(g)
        sub.update(rows=hi - lo, pntrb=g["pntrb"][lo:hi], pntre=g["pntre"][lo:hi])
        Xs = None if X is None else X[lo:hi]
        want = oracle_mirror(orc, tkern, sub, Xs, Y, np.zeros((hi - lo, k), np_v), 0.0, kind_id, k, heavy_deg, seg_len,
                             packed=packed_all[lo:hi])
        got = np.ascontiguousarray(d_Z[lo:hi, :k].cpu().numpy())
        if not general:
            ok = ok and bool(np.array_equal(got.view(np.uint8), want.view(np.uint8)))
            continue
        # The general pipeline multiplies and adds where the optimised kernels fuse, so
        # its bits differ from the mirror's: it is held to the tolerance of the parity
        # tests against the oracle's double-precision evaluation instead.
        import checks
        ot = "t" if tkern == "f" else tkern
        z64 = np.zeros((hi - lo, k), np_v)
        es = np.zeros(int(sub["pntre"].max()) if hi > lo else 0, np_v)
        orc.opt(ot, sub, Xs, Y, z64, beta=0.0, sop_kind=kind_id, mode=1, edge_s=es if kind_id else None)
        _, slots = checks.edge_rows(sub)
        d_abs = (np.ones(slots.size) if tkern == "g" else np.abs(g["val"][slots]).astype(np.float64) if tkern == "m"
                 else np.abs(orc.sop(kind_id, es[slots])).astype(np.float64))
        sdeg = (sub["pntre"] - sub["pntrb"]).astype(np.int64)
        extra = 4 * checks.EPS32 * np.sqrt(np.maximum(sdeg, 1))[:, None] * checks.abs_term_sum(tkern, sub, Xs, Y, d_abs)
        if tkern == "s":
            extra = extra + checks.sigmoid_flip_slack(orc.table(), sub, Xs, Y)[0]
        rtol = 1e-5 if tkern in ("g", "m") else 1e-4
        try:
            checks.assert_close(got, z64, rtol, 1e-6, extra, "general pipeline, rows %d..%d" % (lo, hi))
        except AssertionError as e:
            print("bench.py: %s: %s" % (name, e), file=sys.stderr)
            ok = False
    return ok


def measure(torch, fa, probes, name, steps, warmup, args, gather_probe, read_probe=False, copy_probe=False):
    """Time `steps` calls of fusedMM_csr_stream on workload `name`, operands resident.  Returns the figures of the
    JSON line for that workload and what the CPU leg needs (graph, embeddings)."""
    from fusedmm_amd import synth
    desc, tkern, k, kind = WORKLOADS[name]
    bits = args.index_bits
    vbits = 32 if args.dtype == "f32" else 64
    np_v = np.float32 if vbits == 32 else np.float64
    lib = fa.load(bits, vbits)
    kind_id = {None: 0, "sigmoid": 1, "tdist": 2, "fr": 3}[kind]
    lib.fusedMM_amd_set_sop_kind(kind_id)
    lib.fusedMM_amd_set_opt(0 if args.general else 1)
    imsg = {"s": fa.MSG_SIGMOID, "t": fa.MSG_TDIST, "f": fa.MSG_FR, "m": fa.MSG_SPMM, "g": fa.MSG_GCN}[tkern]

    t_gen = time.time()
    g, X, Y = workload_data(name)
    if vbits == 64:
        same = Y is X
        X = None if X is None else X.astype(np_v)
        Y = X if same else Y.astype(np_v)
        g = dict(g, val=g["val"].astype(np_v))
    if bits == 64:
        g = dict(g)
        for key in ("indx", "pntrb", "pntre", "rowptr"):
            g[key] = g[key].astype(np.int64)
    t_gen = time.time() - t_gen
    m, n, nnz = g["rows"], g["cols"], g["nnz"]

    dev = torch.device("cuda:0")
    up = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    d_val, d_indx, d_pb, d_pe = up(g["val"]), up(g["indx"]), up(g["pntrb"]), up(g["pntre"])
    d_X = up(X)
    d_Y = d_X if Y is X else up(Y)
    ldz = max(k, args.ldz)
    d_Z = torch.zeros((m, ldz), dtype=torch.float32 if vbits == 32 else torch.float64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        rc = fa.fusedMM_csr(imsg, m, n, k, 1.0, nnz, m, n, d_val, d_indx, d_pb, d_pe, d_X, k, d_Y, k, 0.0, d_Z, ldz,
                            index_bits=bits, stream=stream, value_bits=vbits)
        if rc != 0:
            raise SystemExit("fusedMM_csr returned %d" % rc)

    if copy_probe:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            assert probes.fusedMM_amd_copy_probe(dst.data_ptr(), src.data_ptr(), 1 << 30, stream) == 0
        torch.cuda.synchronize()
        del src, dst

    rp = run_read_probe(torch, probes, stream) if read_probe else None
    gp = None
    row_bytes = k * (vbits // 8)
    if gather_probe and 16 <= row_bytes <= 2048 and (row_bytes & (row_bytes - 1)) == 0:
        gp = run_gather_probe(torch, probes, n, row_bytes, stream)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    lib.fusedMM_amd_timing(max(0, args.kernel_events_every))
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    r_ms, s_ms, g_ms = C.c_double(), C.c_double(), C.c_double()
    ncalls = lib.fusedMM_amd_timing_summary(C.byref(r_ms), C.byref(s_ms), C.byref(g_ms))
    per_call = []
    for i in range(max(0, ncalls)):
        c_, f_, m_ = C.c_double(), C.c_double(), C.c_double()
        if lib.fusedMM_amd_timing_call(i, C.byref(c_), C.byref(f_), C.byref(m_)) == 0:
            per_call.append(c_.value + f_.value + m_.value)
    lib.fusedMM_amd_timing(0)
    ms_per_step = wall / steps * 1e3

    flops = synth.algorithmic_flops(tkern, k, nnz)
    # the general rule reads Z before it writes it
    b_alg = synth.algorithmic_bytes(tkern, m, k, nnz, bits // 8, beta_nonzero=args.general, value_bytes=vbits // 8)
    value = flops / (ms_per_step * 1e-3) / 1e9

    kern_ms = {"classify_kernel": r_ms.value / max(1, ncalls), "fused_kernel": s_ms.value / max(1, ncalls),
               "merge_kernel": g_ms.value / max(1, ncalls)}
    # dominant kernel: fused_kernel does all the gathering.  When rows were split, the
    # partial results it writes are folded by merge_kernel, so the call's algorithmic
    # bytes are quoted on the three together (classify_kernel only reads row pointers).
    hs = (C.c_uint(), C.c_uint(), C.c_uint())
    lib.fusedMM_amd_last_split(C.byref(hs[0]), C.byref(hs[1]), C.byref(hs[2]))
    ro = (C.c_int(), C.c_uint(), C.c_uint())
    lib.fusedMM_amd_last_row_order(C.byref(ro[0]), C.byref(ro[1]), C.byref(ro[2]))
    row_order = {"scattered": bool(ro[0].value), "sampled_edges_lower_half": ro[1].value, "sampled_edges_upper_half": ro[2].value}
    split = hs[1].value > 0
    dom_ms = kern_ms["fused_kernel"] + (kern_ms["merge_kernel"] + kern_ms["classify_kernel"] if split else 0.0)
    if ncalls <= 0:
        dom_ms = ms_per_step      # no step carried events: whole-step wall time stands in (an upper bound)
    achieved = b_alg / (dom_ms * 1e-3) / 1e9 if dom_ms > 0 else 0.0
    as_profiled = vbits == 32 and bits == 32 and not args.general
    traffic, traffic_from = measured_traffic_bytes(name) if as_profiled else (None, None)
    roofline = {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                "frac": achieved / PEAK_HBM_GBPS, "traffic": traffic, "traffic_from": traffic_from,
                "traffic_is": TRAFFIC_IS if traffic else None,
                "kernel": "classify_kernel+fused_kernel+merge_kernel" if split else "fused_kernel",
                "kernel_ms": dom_ms, "algorithmic_bytes": b_alg}
    if rp:
        roofline["read_stream_probe"] = rp
        roofline["frac_of_read_stream"] = achieved / rp["plain_loads_GBps"]
    if gp:
        roofline["gather_probe"] = gp
        roofline["frac_of_gather_probe"] = achieved / gp["plain_loads_GBps"]

    checked = None
    if not args.no_check:
        checked = spot_check(torch, name, g, X, Y, d_Z, k, ldz, tkern, kind_id, vbits, args.general, step)

    out = {
        "value": value, "unit": "GFLOP/s", "steps": steps, "warmup": warmup, "ms_per_step": ms_per_step,
        "config": {"workload": "%s: %s" % (name, desc), "op": tkern, "K": k, "rows": m, "nnz": nnz,
                   "index_bits": bits, "beta": 0.0, "graph_gen_s": round(t_gen, 2),
                   "pipeline": "general" if args.general else "optimised", "ldz": ldz,
                   # when finished Z rows are written (fusedMM_amd_set_store_tick): "auto" holds them for a common
                   # 82 us clock tick where Y is 1 GiB or more, and writes them as they finish otherwise
                   "store_tick": os.environ.get("FUSEDMM_STORE_TICK", "auto"),
                   "y_bytes": int(Y.shape[0]) * int(Y.shape[1]) * int(Y.itemsize)},
        "edges_per_s": nnz / (ms_per_step * 1e-3),
        "hbm_GBps_algorithmic": b_alg / (ms_per_step * 1e-3) / 1e9,
        "pct_peak_hbm": 100.0 * b_alg / (ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBPS,
        "kernel_ms": kern_ms,
        "kernel_events": {"every_nth_step": args.kernel_events_every, "steps_recorded": max(0, ncalls)},
        "kernels_ms_per_call": {"min": float(np.min(per_call)), "median": float(np.median(per_call)),
                                "max": float(np.max(per_call))} if per_call else None,
        "split": {"heavy_rows": hs[0].value, "segments": hs[1].value, "overflow": hs[2].value},
        "row_order": row_order,
        "spot_check_vs_oracle": checked,
        "roofline": roofline,
    }
    del d_val, d_indx, d_pb, d_pe, d_X, d_Y, d_Z
    torch.cuda.empty_cache()
    return out, (g, X, Y, tkern, kind_id, k, as_profiled)


def compact(name, r):
    """What the "also" list keeps of an extra workload's figures."""
    rl = r["roofline"]
    return {"workload": r["config"]["workload"], "op": r["config"]["op"], "K": r["config"]["K"], "rows": r["config"]["rows"],
            "nnz": r["config"]["nnz"], "steps": r["steps"], "warmup": r["warmup"], "ms_per_step": r["ms_per_step"],
            "value": r["value"], "unit": r["unit"], "edges_per_s": r["edges_per_s"], "kernel_ms": rl["kernel_ms"],
            "kernels": rl["kernel"], "algorithmic_bytes": rl["algorithmic_bytes"],
            "roofline": {"bound": "hbm", "achieved": rl["achieved"], "peak": rl["peak"], "unit": rl["unit"],
                         "frac": rl["frac"], "traffic": rl["traffic"], "traffic_from": rl["traffic_from"],
                         "frac_of_gather_probe": rl.get("frac_of_gather_probe"),
                         "gather_probe_GBps": (rl.get("gather_probe") or {}).get("plain_loads_GBps")},
            "split": r["split"], "row_order_scattered": r["row_order"]["scattered"], "store_tick": r["config"]["store_tick"],
            "y_bytes": r["config"]["y_bytes"],
            "graph_gen_s": r["config"]["graph_gen_s"], "spot_check_vs_oracle": r["spot_check_vs_oracle"]}


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus %d is not supported "
              "(rows are independent: a sharded run would split the rows of A, X and Z across GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import fusedmm_amd as fa
    probes = fa.load_probes()

    default_run = (args.workload == "c2" and args.dtype == "f32" and args.index_bits == 32 and not args.general)
    also_names = []
    if args.also == "auto":
        also_names = list(ALSO_DEFAULT) if default_run else []
    elif args.also not in ("none", ""):
        also_names = [w for w in args.also.split(",") if w]
        for w in also_names:
            if w not in WORKLOADS:
                raise SystemExit("unknown workload %s in --also" % w)

    r, (g, X, Y, tkern, kind_id, k, as_profiled) = measure(
        torch, fa, probes, args.workload, args.steps, args.warmup, args,
        gather_probe=args.gather_probe or default_run, read_probe=args.read_probe, copy_probe=args.copy_probe)
    out = {"metric": "GFLOP/s + HBM GB/s (% of peak), sigmoid K=128, 1 MI355X vs CPU OpenMP",
           "value": r["value"], "unit": r["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": args.dtype, "data": "synthetic"}
    for key in ("config", "edges_per_s", "hbm_GBps_algorithmic", "pct_peak_hbm", "kernel_ms", "kernel_events",
                "kernels_ms_per_call", "split", "row_order", "spot_check_vs_oracle", "roofline"):
        out[key] = r[key]
    failed = [args.workload] if r["spot_check_vs_oracle"] is False else []
    if not args.no_cpu and as_profiled:
        out["cpu_baseline"] = cpu_baseline(args.workload, g, X, Y, tkern, kind_id, k)
    del g, X, Y

    if also_names:
        out["also"] = []
        for w in also_names:
            print("bench.py: extra workload %s ..." % w, file=sys.stderr, flush=True)
            ra, _ = measure(torch, fa, probes, w, args.also_steps, 2, args, gather_probe=True)
            out["also"].append(compact(w, ra))
            if ra["spot_check_vs_oracle"] is False:
                failed.append(w)
    if failed:
        # a run whose output differs from the oracle's is not a measurement
        out["value"] = None
        out["error"] = "spot check against the oracle failed on %s: results differ" % ", ".join(failed)
        print(json.dumps(out))
        sys.exit(3)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
