"""Writes the golden fixtures of tests/golden/ by running the REAL reference
(oracle/_ref/libref_*.so, built by `make -C oracle ref` from /root/reference).

    python tests/golden/make_golden.py

Fixtures are data only: inputs (small seeded graphs and embeddings, stored in
full so nothing has to be regenerated bit-for-bit) and the reference's outputs:
  sop.npz             the harness's 2048-entry sigmoid table and its
                      SOP_UDEF_FUNC bodies evaluated on a fixed probe vector,
                      single precision and (keys ending in _d) double precision
  ops_d_i<bits>.npz   as ops_i<bits>.npz for the reference's -DDREAL build
  ops_i<bits>.npz     Z of the harness's trusted kernels and of the reference's
                      fusedMM_csr (general pipeline) for the five op kinds
  tuples_i32.npz      Z of the reference's fusedMM_csr for a sweep of op tuples
  mtx.npz             CSR the reference's loader builds from hand-written .mtx
                      texts (stored alongside as strings)
  partition.npz       which thread the reference's fusedMM_csr (built with its
                      nnz-balanced row partition on 2, 3, 5, 8 and 16 threads)
                      evaluated each row on, for the degree sets of
                      graphs.partition_cases() (-1: a row without edges, whose
                      holder the reference never shows)
  special_values.npz  Z of the reference's fusedMM_csr (general pipeline) for the MAX / MIN
                      tuples on operands salted with NaN, infinities and zeros of both signs
                      (graphs.special_values_case), float and (keys ending in _d) double
  udef_stages.npz     Z of the reference's fusedMM_csr built with VOP/ROP/VSC/
                      AOP_UDEF_IMPL switched on and linked with the caller-side
                      stage functions of oracle/udef_stage_bodies.inc, for op
                      tuples in which one or more stages are those functions
                      (float and, keys ending in _d, double; int32 and int64
                      builds agree and one copy is kept)
"""
import os
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import graphs  # noqa: E402
from oracle_api import MSG, PARTITION_THREADS, Ref, RefPartition, RefUdef  # noqa: E402

KINDS = {"s": "sigmoid", "t": "tdist", "f": "fr", "m": "spmm", "g": "gcn"}

MTX_TEXTS = {
    # symmetric pattern with a diagonal entry (dropped by the loader) and comments
    "sym_pattern": "%%MatrixMarket matrix coordinate pattern symmetric\n% a comment\n5 5 6\n2 1\n3 1\n3 3\n4 2\n5 4\n5 1\n",
    # general with values, a duplicate entry, a self loop, unsorted
    "general_real": "%%MatrixMarket matrix coordinate real general\n4 6 7\n3 2 5\n1 6 2\n1 1 7\n3 2 4\n2 5 1\n4 4 3\n1 3 9\n",
    # symmetric with integer weights
    "sym_int": "%%MatrixMarket matrix coordinate integer symmetric\n4 4 4\n2 1 3\n4 1 2\n4 3 8\n2 2 5\n",
}


def probe_vector():
    rng = np.random.Generator(np.random.Philox(key=[99, 0]))
    edges = (np.arange(0, 2049, 64) * 10.0 / 2048 - 5.0).astype(np.float32)
    v = np.concatenate([rng.uniform(-6, 6, 400).astype(np.float32), edges,
                        np.nextafter(edges, np.float32(9)), np.nextafter(edges, np.float32(-9)),
                        np.array([0.0, 4.9999995, -4.9999995, 5.000001, -5.000001, 1e-3, 1e3], np.float32)])
    return v[v != np.float32(5.0)]


def main():
    out = {}
    v = probe_vector()
    out["probe"] = v
    out["table"] = Ref("sigmoid", 32).table()
    for kind in ("sigmoid", "tdist", "fr", "ll", "fa"):
        arg = v if kind == "sigmoid" else np.abs(v) + np.float32(1e-3)
        out["sop_" + kind] = Ref(kind, 32).sop(arg)
    vd = v.astype(np.float64)
    vd = vd[vd < 4.99999]          # next to +5 the double build rounds v + 5 to 10 and reads past its table
    out["probe_d"] = vd
    out["table_d"] = Ref("sigmoid", 32, 64).table()
    for kind in ("sigmoid", "tdist", "fr", "ll", "fa"):
        arg = vd if kind == "sigmoid" else np.abs(vd) + 1e-3
        out["sop_%s_d" % kind] = Ref(kind, 32, 64).sop(arg)
    np.savez_compressed(os.path.join(HERE, "sop.npz"), **out)

    for bits in (32, 64):
        out = {}
        g = graphs.ragged(bits)
        out["ragged_pntrb"], out["ragged_pntre"] = g["pntrb"], g["pntre"]
        out["ragged_indx"], out["ragged_val"] = g["indx"], g["val"]
        out["ragged_shape"] = np.array([g["rows"], g["cols"]])
        k = 24
        X = graphs.features(g["rows"], k, 1, -1, 1, 1).astype(np.float64)
        Y = graphs.features(g["cols"], k, 1, -1, 1, 2).astype(np.float64)
        out["ragged_X%d" % k], out["ragged_Y%d" % k] = X, Y
        for t, kind in KINDS.items():
            r = Ref(kind, bits, 64)
            Zt = np.zeros((g["rows"], k))
            r.trusted(t, g, X, Y, Zt)
            Zf = np.zeros((g["rows"], k))
            r.test(t, g, X, Y, Zf)
            out["ragged_%s_k%d_trusted" % (t, k)] = Zt
            out["ragged_%s_k%d_fusedmm" % (t, k)] = Zf
        np.savez_compressed(os.path.join(HERE, "ops_d_i%d.npz" % bits), **out)

    for bits in (32, 64):
        out = {}
        for gname, g in (("ragged", graphs.ragged(bits)), ("er", graphs.with_values(graphs.tiny_er(150, 600, 11, bits)))):
            out[gname + "_pntrb"], out[gname + "_pntre"] = g["pntrb"], g["pntre"]
            out[gname + "_indx"], out[gname + "_val"] = g["indx"], g["val"]
            out[gname + "_shape"] = np.array([g["rows"], g["cols"]])
            for k in (16, 40):
                X = graphs.features(g["rows"], k, 1, -1, 1, 1)
                Y = graphs.features(g["cols"], k, 1, -1, 1, 2)
                out["%s_X%d" % (gname, k)], out["%s_Y%d" % (gname, k)] = X, Y
                for t, kind in KINDS.items():
                    r = Ref(kind, bits)
                    Zt = np.zeros((g["rows"], k), np.float32)
                    r.trusted(t, g, X, Y, Zt)
                    Zf = np.zeros((g["rows"], k), np.float32)
                    r.test(t, g, X, Y, Zf)
                    out["%s_%s_k%d_trusted" % (gname, t, k)] = Zt
                    out["%s_%s_k%d_fusedmm" % (gname, t, k)] = Zf
        np.savez_compressed(os.path.join(HERE, "ops_i%d.npz" % bits), **out)

    # op-tuple sweep through the reference's general pipeline (accumulates into a non-zero Z)
    g = graphs.ragged(32, rows=23, cols=31, hub_deg=40)
    k = 8
    X = graphs.features(g["rows"], k, 1, -1, 1, 1)
    Y = graphs.features(g["cols"], k, 1, -1, 1, 2)
    Z0 = graphs.features(g["rows"], k, 1, -1, 1, 3)
    out = {"pntrb": g["pntrb"], "pntre": g["pntre"], "indx": g["indx"], "val": g["val"],
           "shape": np.array([g["rows"], g["cols"]]), "X": X, "Y": Y, "Z0": Z0}
    r = Ref("tdist", 32)
    msgs = []
    for vop in range(1, 8):
        for rop in (0x00, 0x10, 0x20, 0x30, 0x40, 0x50):
            for sop, vsc in ((0x100, 0x1000), (0x100, 0x2000), (0xF00, 0x1000), (0x000, 0x0000)):
                for aop in (0x10000, 0x20000, 0x30000):
                    if (vop + (rop >> 4) + (sop >> 8) + (vsc >> 12) + (aop >> 16)) % 3:
                        continue   # a third of the 504 combinations
                    msgs.append(vop | rop | sop | vsc | aop)
    msgs = np.array(msgs, np.int32)
    Zs = np.zeros((len(msgs),) + Z0.shape, np.float32)
    for n, imsg in enumerate(msgs):
        Z = Z0.copy()
        assert r.fusedMM_csr(int(imsg), g, X, Y, Z) == 0
        Zs[n] = Z
    out["msgs"], out["Z"] = msgs, Zs
    np.savez_compressed(os.path.join(HERE, "tuples_i32.npz"), **out)

    out = {}
    r = Ref("gcn", 32)
    for name, text in MTX_TEXTS.items():
        with tempfile.NamedTemporaryFile("w", suffix=".mtx", delete=False) as f:
            f.write(text)
        rows, cols, rowptr, colids, values = r.load_mtx(f.name)
        os.unlink(f.name)
        out[name + "_text"] = np.array(text)
        out[name + "_shape"] = np.array([rows, cols])
        out[name + "_rowptr"], out[name + "_colids"], out[name + "_values"] = rowptr, colids, values
    np.savez_compressed(os.path.join(HERE, "mtx.npz"), **out)
    out = {}
    names = []
    for name, pb, pe, m in graphs.partition_cases():
        names.append(name)
        out[name + "_pntrb"], out[name + "_pntre"], out[name + "_m"] = pb, pe, np.array(m)
        for t in PARTITION_THREADS:
            own32, _ = RefPartition(t, 32).owners(pb, pe, m)
            own64, _ = RefPartition(t, 64).owners(pb, pe, m)
            assert np.array_equal(own32, own64)
            out["%s_owner_t%d" % (name, t)] = own32.astype(np.int8)
    out["names"] = np.array(names)
    np.savez_compressed(os.path.join(HERE, "partition.npz"), **out)

    # MAX / MIN stages on NaN, infinities and signed zeros
    multi, single, X, Y, Z0, msgs = graphs.special_values_case(32)
    out = {"msgs": msgs}
    for sfx, vbits, npv in (("", 32, np.float32), ("_d", 64, np.float64)):
        r = Ref("tdist", 32, vbits)
        for gname, g in (("multi", multi), ("single", single)):
            Zs = np.zeros((len(msgs),) + Z0.shape, npv)
            for n, imsg in enumerate(msgs):
                Z = Z0.astype(npv)
                assert r.fusedMM_csr(int(imsg), g, X.astype(npv), Y.astype(npv), Z) == 0
                Zs[n] = Z
            out["Z_%s%s" % (gname, sfx)] = Zs
    np.savez_compressed(os.path.join(HERE, "special_values.npz"), **out)

    # tuples with user stages through the reference built with those stages switched on
    g = graphs.with_values(graphs.ragged(32, rows=37, cols=53, hub_deg=90))
    k = 12
    X = graphs.features(g["rows"], k, 9, -1, 1, 1)
    Y = graphs.features(g["cols"], k, 9, -1, 1, 2)
    Z0 = graphs.features(g["rows"], k, 9, -1, 1, 3)
    out = {"pntrb": g["pntrb"], "pntre": g["pntre"], "indx": g["indx"], "val": g["val"],
           "shape": np.array([g["rows"], g["cols"]]), "X": X, "Y": Y, "Z0": Z0}
    msgs = graphs.udef_stage_tuples()
    for sfx, vbits, npv in (("", 32, np.float32), ("_d", 64, np.float64)):
        Zs = np.zeros((len(msgs),) + Z0.shape, npv)
        g64 = dict(g, indx=g["indx"].astype(np.int64), pntrb=g["pntrb"].astype(np.int64), pntre=g["pntre"].astype(np.int64))
        for n, imsg in enumerate(msgs):
            Z, Zw = Z0.astype(npv), Z0.astype(npv)
            assert RefUdef(32, vbits).fusedMM_csr(int(imsg), g, X.astype(npv), Y.astype(npv), Z) == 0
            assert RefUdef(64, vbits).fusedMM_csr(int(imsg), g64, X.astype(npv), Y.astype(npv), Zw) == 0
            assert np.array_equal(Z.view(np.uint8), Zw.view(np.uint8))
            Zs[n] = Z
        out["Z" + sfx] = Zs
    out["msgs"] = msgs
    np.savez_compressed(os.path.join(HERE, "udef_stages.npz"), **out)
    print("golden fixtures written to", HERE)


if __name__ == "__main__":
    main()
