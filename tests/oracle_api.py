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

SOP_IDENTITY, SOP_SIGMOID, SOP_TDIST, SOP_FR, SOP_LL, SOP_FA = range(6)
SOP_NAMES = {"identity": 0, "sigmoid": 1, "tdist": 2, "fr": 3, "ll": 4, "fa": 5}

# op tuples the reference harness sends (test/fusedMMtime.cpp:731-753)
MSG = {
    "t": 0x11F55,  # VOP_SUBR | ROP_NORMR | SOP_UDEF | VSC_MUL | AOP_ADD
    "f": 0x11F55,
    "s": 0x11F12,  # VOP_COPY_RHS | ROP_DOT | SOP_UDEF | VSC_MUL | AOP_ADD
    "m": 0x11102,  # VOP_COPY_RHS | ROP_NOOP | SOP_COPY | VSC_MUL | AOP_ADD
    "g": 0x10002,  # VOP_COPY_RHS | ROP_NOOP | SOP_NOOP | VSC_NOOP | AOP_ADD
}

_f32p = C.POINTER(C.c_float)


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


class Oracle:
    """The CPU restatement.  fast=True loads the -O3 build (baseline timing)."""

    def __init__(self, fast=False):
        self.lib = _load("libfusedmm_oracle_fast.so" if fast else "libfusedmm_oracle.so")
        L = self.lib
        L.orc_sigmoid_table.argtypes = [_f32p]
        L.orc_sigmoid_bin.argtypes = [C.c_float]
        L.orc_sigmoid_bin.restype = C.c_int
        L.orc_sop.argtypes = [C.c_int, C.c_float]
        L.orc_sop.restype = C.c_float
        L.orc_sop_array.argtypes = [C.c_int, _f32p, _f32p, C.c_int64]
        L.orc_gpu_dot.argtypes = [_f32p, _f32p, C.c_int64, C.c_int, C.c_int, C.c_int]
        L.orc_gpu_dot.restype = C.c_float
        L.orc_max_threads.restype = C.c_int

    def table(self):
        t = np.empty(2048, np.float32)
        self.lib.orc_sigmoid_table(_ptr(t, C.c_float))
        return t

    def bin(self, v):
        return self.lib.orc_sigmoid_bin(C.c_float(v))

    def sop(self, kind, arr):
        a = np.ascontiguousarray(arr, np.float32)
        out = np.empty_like(a)
        self.lib.orc_sop_array(kind, _ptr(a, C.c_float), _ptr(out, C.c_float), a.size)
        return out

    def gpu_dot(self, x, y, V, L, diff=0):
        x = np.ascontiguousarray(x, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        return self.lib.orc_gpu_dot(_ptr(x, C.c_float), _ptr(y, C.c_float), x.size, V, L, diff)

    def max_threads(self):
        return self.lib.orc_max_threads()

    def partition(self, pntrb, pntre, nthreads, m=None):
        bits = pntrb.dtype.itemsize * 8
        _, ct = _itype(bits)
        m = len(pntrb) if m is None else m
        rb = np.empty(nthreads, np.int64)
        re = np.empty(nthreads, np.int64)
        fn = getattr(self.lib, "orc_partition_rows_i%d" % bits)
        fn.argtypes = [ct, C.POINTER(ct), C.POINTER(ct), C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        fn.restype = C.c_int
        rc = fn(m, _ptr(pntrb, ct), _ptr(pntre, ct), nthreads, _ptr(rb, C.c_int64), _ptr(re, C.c_int64))
        return rc, rb, re

    @staticmethod
    def _csr_args(ct, m, n, k, nnz, rows, cols, val, indx, pntrb, pntre, x, ldx, y, ldy, beta, z, ldz):
        return [ct(m), ct(n), ct(k), C.c_float(1.0), ct(nnz), ct(rows), ct(cols),
                _ptr(val, C.c_float), _ptr(indx, ct), _ptr(pntrb, ct), _ptr(pntre, ct),
                _ptr(x, C.c_float), ct(ldx), _ptr(y, C.c_float), ct(ldy), C.c_float(beta),
                _ptr(z, C.c_float), ct(ldz)]

    def generic(self, imsg, g, x, y, z, beta=0.0, sop_kind=0, m=None, k=None, ldx=None, ldy=None, ldz=None):
        """orc_fusedmm_generic; g is a graph dict (see tests/graphs.py). z is updated in place."""
        bits = g["indx"].dtype.itemsize * 8
        _, ct = _itype(bits)
        m = g["rows"] if m is None else m
        k = y.shape[1] if k is None else k
        ldx = (x.shape[1] if x is not None else k) if ldx is None else ldx
        ldy = y.shape[1] if ldy is None else ldy
        ldz = z.shape[1] if ldz is None else ldz
        fn = getattr(self.lib, "orc_fusedmm_generic_i%d" % bits)
        fn.restype = C.c_int
        args = [C.c_int32(imsg)] + self._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"],
                                                  g["val"], g["indx"], g["pntrb"], g["pntre"],
                                                  x, ldx, y, ldy, beta, z, ldz) + [C.c_int(sop_kind)]
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
        fn = getattr(self.lib, "orc_fusedmm_opt_i%d" % bits)
        fn.restype = C.c_int
        args = [C.c_char(tkern.encode())] + self._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"],
                                                           g["val"], g["indx"], g["pntrb"], g["pntre"],
                                                           x, ldx, y, ldy, beta, z, ldz)
        args += [C.c_int(sop_kind), C.c_int(mode), C.c_int(V), C.c_int(L), C.c_int(S), _ptr(edge_s, C.c_float)]
        return fn(*args)

    def baseline(self, tkern, g, x, y, z, beta=0.0, sop_kind=0, nthreads=1, m=None):
        bits = g["indx"].dtype.itemsize * 8
        _, ct = _itype(bits)
        m = g["rows"] if m is None else m
        k = y.shape[1]
        fn = getattr(self.lib, "orc_fusedmm_baseline_i%d" % bits)
        fn.restype = C.c_int
        args = [C.c_char(tkern.encode())] + self._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"],
                                                           g["val"], g["indx"], g["pntrb"], g["pntre"],
                                                           x, x.shape[1] if x is not None else k, y, k, beta, z, k)
        args += [C.c_int(sop_kind), C.c_int(nthreads)]
        return fn(*args)


def ref_available(kind="sigmoid", bits=32):
    return os.path.exists(os.path.join(ORACLE_DIR, "_ref", "libref_%s_i%d.so" % (kind, bits)))


class Ref:
    """The real reference (harness + generic fusedMM_csr), one library per SOP body."""

    def __init__(self, kind, bits=32):
        self.bits = bits
        self.np_i, self.ct = _itype(bits)
        self.lib = C.CDLL(os.path.join(ORACLE_DIR, "_ref", "libref_%s_i%d.so" % (kind, bits)))
        assert self.lib.ref_index_bytes() * 8 == bits

    def table(self):
        t = np.empty(2048, np.float32)
        self.lib.ref_sm_table(_ptr(t, C.c_float))
        return t

    def sop(self, arr):
        a = np.ascontiguousarray(arr, np.float32)
        out = np.empty_like(a)
        self.lib.ref_sop_array.argtypes = [_f32p, _f32p, C.c_int64]
        self.lib.ref_sop_array(_ptr(a, C.c_float), _ptr(out, C.c_float), a.size)
        return out

    def _call(self, fn, head, g, x, y, z, beta, m):
        ct = self.ct
        m = g["rows"] if m is None else m
        k = y.shape[1]
        args = head + Oracle._csr_args(ct, m, g["cols"], k, g["nnz"], g["rows"], g["cols"], g["val"], g["indx"],
                                       g["pntrb"], g["pntre"], x, k, y, k, beta, z, k)
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
        values = np.empty(n.value, np.float32)
        self.lib.ref_get_csr(_ptr(rowptr, self.ct), _ptr(colids, self.ct), _ptr(values, C.c_float))
        return r.value, c.value, rowptr, colids, values
