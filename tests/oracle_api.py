"""ctypes doors into the CPU oracle (oracle/libfusedmm_oracle*.so) and, when it
has been built, the real reference (oracle/_ref/libref_<kind>_i<bits>.so).

Test infrastructure only: nothing under fusedmm_amd/ imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

SOP_IDENTITY, SOP_SIGMOID, SOP_TDIST, SOP_FR, SOP_LL, SOP_FA, SOP_TDIST_PLAIN = range(7)
SOP_NAMES = {"identity": 0, "sigmoid": 1, "tdist": 2, "fr": 3, "ll": 4, "fa": 5, "tdist_plain": 6}

# op tuples the reference harness sends (test/fusedMMtime.cpp:731-753)
MSG = {
    "t": 0x11F55,  # VOP_SUBR | ROP_NORMR | SOP_UDEF | VSC_MUL | AOP_ADD
    "f": 0x11F55,
    "s": 0x11F12,  # VOP_COPY_RHS | ROP_DOT | SOP_UDEF | VSC_MUL | AOP_ADD
    "m": 0x11102,  # VOP_COPY_RHS | ROP_NOOP | SOP_COPY | VSC_MUL | AOP_ADD
    "g": 0x10002,  # VOP_COPY_RHS | ROP_NOOP | SOP_NOOP | VSC_NOOP | AOP_ADD
}

_f32p = C.POINTER(C.c_float)


def _vtype(vbits):
    return (np.float32, C.c_float) if vbits == 32 else (np.float64, C.c_double)


def _ptr(a, ctype):
    if a is None:
        return None
    return a.ctypes.data_as(C.POINTER(ctype))


def _itype(bits):
    return (np.int32, C.c_int32) if bits == 32 else (np.int64, C.c_int64)


def build_oracle():
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR, "all"])


def _load(name):
    path = os.path.join(ORACLE_DIR, name)
    if not os.path.exists(path):
        build_oracle()
    return C.CDLL(path)


def host_has_avx512():
    """Does this host's CPU offer what -march=x86-64-v4 code needs?"""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("flags"):
                have = set(line.split(":", 1)[1].split())
                return {"avx512f", "avx512bw", "avx512cd", "avx512dq", "avx512vl"} <= have
    except OSError:
        pass
    return False


class Oracle:
    """The CPU restatement.  fast=True loads the -O3 build (baseline timing), the AVX-512 one
    where the host has it; vbits=64 selects the double-precision instance (the reference's -DDREAL)."""

    def __init__(self, fast=False, vbits=32):
        self.isa = "strict"
        if fast:
            self.isa = "x86-64-v3 (AVX2+FMA)"
            name = "libfusedmm_oracle_fast.so"
            if host_has_avx512() and os.path.exists(os.path.join(ORACLE_DIR, "libfusedmm_oracle_fast_v4.so")):
                name, self.isa = "libfusedmm_oracle_fast_v4.so", "x86-64-v4 (AVX-512)"
        self.lib = _load(name if fast else "libfusedmm_oracle.so")
        self.vbits = vbits
        self.np_v, self.cv = _vtype(vbits)
        self.sfx = "" if vbits == 32 else "_d"
        L = self.lib
        vp = C.POINTER(self.cv)
        self._table = getattr(L, "orc_sigmoid_table" + self.sfx)
        self._table.argtypes = [vp]
        self._bin = getattr(L, "orc_sigmoid_bin" + self.sfx)
        self._bin.argtypes = [self.cv]
        self._bin.restype = C.c_int
        self._sop_array = getattr(L, "orc_sop_array" + self.sfx)
        self._sop_array.argtypes = [C.c_int, vp, vp, C.c_int64]
        self._gpu_dot = getattr(L, "orc_gpu_dot" + self.sfx)
        self._gpu_dot.argtypes = [vp, vp, C.c_int64, C.c_int, C.c_int, C.c_int]
        self._gpu_dot.restype = self.cv
        L.orc_max_threads.restype = C.c_int

    def table(self):
        t = np.empty(2048, self.np_v)
        self._table(_ptr(t, self.cv))
        return t

    def bin(self, v):
        return self._bin(self.cv(v))

    def sop(self, kind, arr):
        a = np.ascontiguousarray(arr, self.np_v)
        out = np.empty_like(a)
        self._sop_array(kind, _ptr(a, self.cv), _ptr(out, self.cv), a.size)
        return out

    def gpu_dot(self, x, y, V, L, diff=0):
        x = np.ascontiguousarray(x, self.np_v)
        y = np.ascontiguousarray(y, self.np_v)
        return self._gpu_dot(_ptr(x, self.cv), _ptr(y, self.cv), x.size, V, L, diff)

    def max_threads(self):
        return self.lib.orc_max_threads()

    def _val(self, g):
        """Edge values in this instance's precision (graphs carry float32 values)."""
        v = g["val"]
        return v if v is None or v.dtype == self.np_v else v.astype(self.np_v)

    def partition(self, pntrb, pntre, nthreads, m=None):
        bits = pntrb.dtype.itemsize * 8
        _, ct = _itype(bits)
        m = len(pntrb) if m is None else m
        rb = np.empty(nthreads, np.int64)
        re = np.empty(nthreads, np.int64)
        fn = getattr(self.lib, "orc_partition_rows_i%d" % bits)   # value-type independent
        fn.argtypes = [ct, C.POINTER(ct), C.POINTER(ct), C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        fn.restype = C.c_int
        rc = fn(m, _ptr(pntrb, ct), _ptr(pntre, ct), nthreads, _ptr(rb, C.c_int64), _ptr(re, C.c_int64))
        return rc, rb, re

    @staticmethod
    def _csr_args(ct, m, n, k, nnz, rows, cols, val, indx, pntrb, pntre, x, ldx, y, ldy, beta, z, ldz, cv=C.c_float):
        np_v = np.float32 if cv is C.c_float else np.float64
        for a in (val, x, y, z):
            assert a is None or a.dtype == np_v, "operand dtype does not match the library's VALUETYPE"
        return [ct(m), ct(n), ct(k), cv(1.0), ct(nnz), ct(rows), ct(cols),
                _ptr(val, cv), _ptr(indx, ct), _ptr(pntrb, ct), _ptr(pntre, ct),
                _ptr(x, cv), ct(ldx), _ptr(y, cv), ct(ldy), cv(beta),
                _ptr(z, cv), ct(ldz)]

    def generic(self, imsg, g, x, y, z, beta=0.0, sop_kind=0, m=None, k=None, ldx=None, ldy=None, ldz=None):
        """orc_fusedmm_generic; g is a graph dict (see tests/graphs.py). z is updated in place."""
        bits = g["indx"].dtype.itemsize * 8
        _, ct = _itype(bits)
        m = g["rows"] if m is None else m
        k = y.shape[1] if k is None else k
        ldx = (x.shape[1] if x is not None else k) if ldx is None else ldx
        ldy = y.shape[1] if ldy is None else ldy
        ldz = z.shape[1] if ldz is None else ldz
        fn = getattr(self.lib, "orc_fusedmm_generic%s_i%d" % (self.sfx, bits))
        fn.restype = C.c_int
        args = [C.c_int32(imsg)] + self._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"],
                                                  self._val(g), g["indx"], g["pntrb"], g["pntre"],
                                                  x, ldx, y, ldy, beta, z, ldz, self.cv) + [C.c_int(sop_kind)]
        return fn(*args)

    def stage_fn(self, stage, bits):
        """Address of the tests' caller-side stage function (VOP, ROP, SOP, VSC, AOP) for this
        precision and index width (oracle/udef_stage_bodies.inc)."""
        return C.cast(getattr(self.lib, "orc_test_%s%s_i%d" % (stage, self.sfx, bits)), C.c_void_p)

    def generic_udef(self, imsg, g, x, y, z, sop_kind=0, host_sop=False, m=None, k=None, ldx=None, ldy=None, ldz=None):
        """orc_fusedmm_generic_udef with the tests' stage functions bound to every *_UDEF
        nibble (host_sop: also to SOP_UDEF, instead of the numbered body sop_kind)."""
        bits = g["indx"].dtype.itemsize * 8
        _, ct = _itype(bits)
        m = g["rows"] if m is None else m
        k = y.shape[1] if k is None else k
        ldx = (x.shape[1] if x is not None else k) if ldx is None else ldx
        ldy = y.shape[1] if ldy is None else ldy
        ldz = z.shape[1] if ldz is None else ldz
        fn = getattr(self.lib, "orc_fusedmm_generic_udef%s_i%d" % (self.sfx, bits))
        fn.restype = C.c_int
        args = [C.c_int32(imsg)] + self._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"],
                                                  self._val(g), g["indx"], g["pntrb"], g["pntre"],
                                                  x, ldx, y, ldy, 0.0, z, ldz, self.cv) + [C.c_int(sop_kind)]
        args += [self.stage_fn("VOP", bits), self.stage_fn("ROP", bits),
                 self.stage_fn("SOP", bits) if host_sop else C.c_void_p(None),
                 self.stage_fn("VSC", bits), self.stage_fn("AOP", bits)]
        return fn(*args)

    def opt(self, tkern, g, x, y, z, beta=0.0, sop_kind=0, mode=0, V=4, L=32, S=1, m=None, k=None,
            ldx=None, ldy=None, ldz=None, edge_s=None):
        bits = g["indx"].dtype.itemsize * 8
        _, ct = _itype(bits)
        m = g["rows"] if m is None else m
        k = y.shape[1] if k is None else k
        ldx = (x.shape[1] if x is not None else k) if ldx is None else ldx
        ldy = y.shape[1] if ldy is None else ldy
        ldz = z.shape[1] if ldz is None else ldz
        fn = getattr(self.lib, "orc_fusedmm_opt%s_i%d" % (self.sfx, bits))
        fn.restype = C.c_int
        args = [C.c_char(tkern.encode())] + self._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"],
                                                           self._val(g), g["indx"], g["pntrb"], g["pntre"],
                                                           x, ldx, y, ldy, beta, z, ldz, self.cv)
        args += [C.c_int(sop_kind), C.c_int(mode), C.c_int(V), C.c_int(L), C.c_int(S), _ptr(edge_s, self.cv)]
        return fn(*args)

    def baseline(self, tkern, g, x, y, z, beta=0.0, sop_kind=0, nthreads=1, m=None):
        bits = g["indx"].dtype.itemsize * 8
        _, ct = _itype(bits)
        m = g["rows"] if m is None else m
        k = y.shape[1]
        fn = getattr(self.lib, "orc_fusedmm_baseline%s_i%d" % (self.sfx, bits))
        fn.restype = C.c_int
        args = [C.c_char(tkern.encode())] + self._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"],
                                                           self._val(g), g["indx"], g["pntrb"], g["pntre"],
                                                           x, x.shape[1] if x is not None else k, y, k, beta, z, k,
                                                           self.cv)
        args += [C.c_int(sop_kind), C.c_int(nthreads)]
        return fn(*args)


def _ref_name(kind, bits, vbits, threads=None):
    if threads:    # timing variant: the reference's OpenMP team fixed at `threads` (float, int32 only)
        return "libref_%s_t%d_i%d.so" % (kind, threads, bits)
    return "libref_%s_%si%d.so" % (kind, "d_" if vbits == 64 else "", bits)


def ref_available(kind="sigmoid", bits=32, vbits=32, threads=None):
    return os.path.exists(os.path.join(ORACLE_DIR, "_ref", _ref_name(kind, bits, vbits, threads)))


REF_TIME_THREADS = (8, 16, 32, 64, 96, 128)    # TIME_THREADS of oracle/Makefile


def ref_threads_for(cores):
    """The largest thread count the reference's general path was built for that does not exceed `cores`."""
    fit = [t for t in REF_TIME_THREADS if t <= max(cores, REF_TIME_THREADS[0])]
    return fit[-1]


class Ref:
    """The real reference (harness + generic fusedMM_csr), one library per SOP body."""

    def __init__(self, kind, bits=32, vbits=32, threads=None):
        self.bits = bits
        self.np_i, self.ct = _itype(bits)
        self.np_v, self.cv = _vtype(vbits)
        self.lib = C.CDLL(os.path.join(ORACLE_DIR, "_ref", _ref_name(kind, bits, vbits, threads)))
        assert self.lib.ref_index_bytes() * 8 == bits and self.lib.ref_value_bytes() * 8 == vbits

    def table(self):
        t = np.empty(2048, self.np_v)
        self.lib.ref_sm_table(_ptr(t, self.cv))
        return t

    def sop(self, arr):
        a = np.ascontiguousarray(arr, self.np_v)
        out = np.empty_like(a)
        vp = C.POINTER(self.cv)
        self.lib.ref_sop_array.argtypes = [vp, vp, C.c_int64]
        self.lib.ref_sop_array(_ptr(a, self.cv), _ptr(out, self.cv), a.size)
        return out

    def _call(self, fn, head, g, x, y, z, beta, m):
        ct = self.ct
        m = g["rows"] if m is None else m
        k = y.shape[1]
        val = g["val"] if g["val"] is None or g["val"].dtype == self.np_v else g["val"].astype(self.np_v)
        args = head + Oracle._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"], val, g["indx"],
                                       g["pntrb"], g["pntre"], x, k, y, k, beta, z, k, self.cv)
        return fn(*args)

    def trusted(self, tkern, g, x, y, z, beta=0.0, m=None):
        self.lib.ref_trusted_csr.restype = None
        return self._call(self.lib.ref_trusted_csr, [C.c_char(tkern.encode())], g, x, y, z, beta, m)

    def test(self, tkern, g, x, y, z, beta=0.0, m=None):
        self.lib.ref_test_csr.restype = None
        return self._call(self.lib.ref_test_csr, [C.c_char(tkern.encode())], g, x, y, z, beta, m)

    def fusedMM_csr(self, imsg, g, x, y, z, beta=0.0, m=None):
        self.lib.ref_fusedMM_csr.restype = C.c_int
        return self._call(self.lib.ref_fusedMM_csr, [C.c_int32(imsg)], g, x, y, z, beta, m)

    def load_mtx(self, path):
        r, c, n = C.c_int64(), C.c_int64(), C.c_int64()
        self.lib.ref_load_mtx(path.encode(), C.byref(r), C.byref(c), C.byref(n))
        rowptr = np.empty(r.value + 1, self.np_i)
        colids = np.empty(n.value, self.np_i)
        values = np.empty(n.value, self.np_v)
        self.lib.ref_get_csr(_ptr(rowptr, self.ct), _ptr(colids, self.ct), _ptr(values, self.cv))
        return r.value, c.value, rowptr, colids, values


def ref_udef_available(bits=32, vbits=32):
    return os.path.exists(os.path.join(ORACLE_DIR, "_ref", _ref_name("udefstages", bits, vbits)))


class RefUdef:
    """The real reference's general fusedMM_csr built with VOP/ROP/VSC/AOP_UDEF_IMPL switched
    on and linked with the tests' caller-side stage functions (oracle/ref_udef_stages.c)."""

    def __init__(self, bits=32, vbits=32):
        self.np_i, self.ct = _itype(bits)
        self.np_v, self.cv = _vtype(vbits)
        self.lib = C.CDLL(os.path.join(ORACLE_DIR, "_ref", _ref_name("udefstages", bits, vbits)))
        assert self.lib.ref_udef_index_bytes() * 8 == bits and self.lib.ref_udef_value_bytes() * 8 == vbits

    def fusedMM_csr(self, imsg, g, x, y, z, m=None):
        m = g["rows"] if m is None else m
        k = y.shape[1]
        val = g["val"] if g["val"] is None or g["val"].dtype == self.np_v else g["val"].astype(self.np_v)
        self.lib.fusedMM_csr.restype = C.c_int
        args = [C.c_int32(imsg)] + Oracle._csr_args(self.ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"], val, g["indx"],
                                                    g["pntrb"], g["pntre"], x, x.shape[1], y, k, 0.0, z, k, self.cv)
        return self.lib.fusedMM_csr(*args)


PARTITION_THREADS = (2, 3, 5, 8, 16)   # PART_THREADS of oracle/Makefile


def ref_partition_available(nthreads=8, bits=32):
    return os.path.exists(os.path.join(ORACLE_DIR, "_ref", "libref_partition_t%d_i%d.so" % (nthreads, bits)))


class RefPartition:
    """The real reference's fusedMM.c built with its nnz-balanced row partition
    (fusedMM.c:633-676) on `nthreads` threads, plus oracle/ref_partition_probe.c,
    whose SOP_UDEF_FUNC records which thread evaluates each row."""

    def __init__(self, nthreads, bits=32):
        self.np_i, self.ct = _itype(bits)
        self.nthreads = nthreads
        self.lib = C.CDLL(os.path.join(ORACLE_DIR, "_ref", "libref_partition_t%d_i%d.so" % (nthreads, bits)))
        assert self.lib.ref_probe_index_bytes() * 8 == bits and self.lib.ref_probe_threads() == nthreads

    def owners(self, pntrb, pntre, m=None):
        """(owner, calls): thread that evaluated each of the first m rows (-1 for
        a row with no edge: the reference never shows who holds it) and the
        number of edges it evaluated there."""
        pntrb = np.ascontiguousarray(pntrb, self.np_i)
        pntre = np.ascontiguousarray(pntre, self.np_i)
        m = len(pntrb) if m is None else m
        slots = int(pntre[:m].max()) if m else 0
        val = np.zeros(max(slots, 1), np.float32)
        for i in range(m):
            val[int(pntrb[i]):int(pntre[i])] = i
        indx = np.zeros(max(slots, 1), self.np_i)
        x = np.zeros(max(m, 1), np.float32)
        y = np.ones(1, np.float32)
        z = np.zeros(max(m, 1), np.float32)
        owner = np.full(max(m, 1), -1, np.int32)
        calls = np.zeros(max(m, 1), np.int32)
        fp, ip = C.POINTER(C.c_float), C.POINTER(self.ct)
        fn = self.lib.ref_partition_probe
        fn.restype = C.c_int
        rc = fn(self.ct(m), self.ct(slots), _ptr(val, C.c_float), _ptr(indx, self.ct), _ptr(pntrb, self.ct),
                _ptr(pntre, self.ct), _ptr(x, C.c_float), _ptr(y, C.c_float), _ptr(z, C.c_float),
                _ptr(owner, C.c_int32), _ptr(calls, C.c_int32))
        assert rc == 0, "reference fusedMM_csr returned %d" % rc
        # the tuple adds val[j] * y[0] = row id once per edge: a second check that every edge ran once
        deg = (pntre[:m].astype(np.int64) - pntrb[:m].astype(np.int64))
        assert np.array_equal(calls[:m], deg), "the reference evaluated some edge zero or several times"
        return owner[:m], calls[:m]


def owners_from_ranges(rowb, rowe, m):
    """Row -> thread id from the oracle's ranges [rowb[id], rowe[id]); -2 for a row in no range,
    -3 for a row in two."""
    own = np.full(m, -2, np.int64)
    for t in range(len(rowb)):
        b, e = int(rowb[t]), int(rowe[t])
        if e > b:
            own[b:e] = np.where(own[b:e] == -2, t, -3)
    return own
