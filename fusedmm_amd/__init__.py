"""Python door to the C ABI of libfusedmm_amd_i{32,64}.so.

The libraries are the product; this module only loads them with ctypes, mirrors
the op-tuple constants of include/fusedMM.h and passes raw addresses through.
There is no CPU fallback: a missing library is an ImportError-like failure at
load time, a failing call returns the library's status code.
"""
import ctypes as C
import os

from .build import lib_path, probes_path

# op-tuple nibbles (include/fusedMM.h; reference fusedMM.h:18-73)
VOP_NOOP, VOP_COPY_LHS, VOP_COPY_RHS, VOP_ADD, VOP_SUBL, VOP_SUBR, VOP_MAX, VOP_MIN, VOP_UDEF = \
    0x0, 0x1, 0x2, 0x3, 0x4, 0x5, 0x6, 0x7, 0xF
ROP_NOOP, ROP_DOT, ROP_ADD_LHS, ROP_ADD_RHS, ROP_NORML, ROP_NORMR, ROP_UDEF = \
    0x00, 0x10, 0x20, 0x30, 0x40, 0x50, 0xF0
SOP_NOOP, SOP_COPY, SOP_UDEF = 0x000, 0x100, 0xF00
VSC_NOOP, VSC_MUL, VSC_ADD, VSC_UDEF = 0x0000, 0x1000, 0x2000, 0xF000
AOP_NOOP, AOP_ADD, AOP_MAX, AOP_MIN, AOP_UDEF = 0x00000, 0x10000, 0x20000, 0x30000, 0xF0000

# tuples the reference's tester sends (test/fusedMMtime.cpp:731-753)
MSG_TDIST = VOP_SUBR | ROP_NORMR | SOP_UDEF | VSC_MUL | AOP_ADD
MSG_FR = MSG_TDIST
MSG_SIGMOID = VOP_COPY_RHS | ROP_DOT | SOP_UDEF | VSC_MUL | AOP_ADD
MSG_SPMM = VOP_COPY_RHS | ROP_NOOP | SOP_COPY | VSC_MUL | AOP_ADD
MSG_GCN = VOP_COPY_RHS | ROP_NOOP | SOP_NOOP | VSC_NOOP | AOP_ADD

SOP_KIND_HOST, SOP_KIND_IDENTITY, SOP_KIND_SIGMOID, SOP_KIND_TDIST, SOP_KIND_FR, SOP_KIND_LL, SOP_KIND_FA, \
    SOP_KIND_TDIST_PLAIN = -1, 0, 1, 2, 3, 4, 5, 6

SUCCESS, FAIL, VOP_FAIL, ROP_FAIL, AOP_FAIL, SOP_FAIL, VSC_FAIL = 0, 1, 2, 4, 8, 16, 32
NOT_ENOUGH_MEM, UNDEFINED_USER_FUNCTION, NO_OPT_IMPL = -1, 64, 128

# every symbol include/fusedMM.h and include/fusedmm_amd.h declare (sgfusedMM_csr / dgfusedMM_csr by precision)
EXPORTS = ("fusedMM_csr", "fusedMM_csr_stream", "fusedMM_csr_stream_noalloc", "fusedMM_amd_init",
           "fusedMM_amd_init_noalloc", "fusedMM_amd_noalloc_capacity", "fusedMM_amd_index_bytes",
           "fusedMM_amd_value_bytes", "fusedMM_amd_set_sop_kind", "fusedMM_amd_get_sop_kind",
           "fusedMM_amd_set_sop_callback", "fusedMM_amd_set_stage_callbacks", "fusedMM_amd_set_opt",
           "fusedMM_amd_set_validate", "fusedMM_amd_set_cache", "fusedMM_amd_invalidate",
           "fusedMM_amd_last_host_phases", "fusedMM_amd_set_split", "fusedMM_amd_get_split", "fusedMM_amd_set_pack_rows", "fusedMM_amd_set_store_tick", "fusedMM_amd_timing",
           "fusedMM_amd_timing_summary", "fusedMM_amd_timing_call", "fusedMM_amd_last_split",
           "fusedMM_amd_last_row_order", "fusedMM_amd_finalize")
# the measuring aids of libfusedmm_amd_probes.so (csrc/fusedmm_probes.h): not part of the product's ABI
PROBE_EXPORTS = ("fusedMM_amd_copy_probe", "fusedMM_amd_read_probe", "fusedMM_amd_gather_probe")

_libs = {}


def load(index_bits=32, value_bits=32):
    """dlopen the library for INDEXTYPE = int<index_bits>_t and VALUETYPE = float
    (value_bits 32) or double (64), and declare its signatures."""
    key = (index_bits, value_bits)
    if key in _libs:
        return _libs[key]
    # One HIP runtime per process: when PyTorch is present its bundled
    # libamdhip64 (same SONAME as ROCm's) must be mapped first, so that this
    # library binds to it and device addresses and streams can be shared.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    path = lib_path(index_bits, value_bits)
    if not os.path.exists(path):
        raise OSError("%s is not built; run `python -m fusedmm_amd.build`" % path)
    lib = C.CDLL(path)
    it = C.c_int32 if index_bits == 32 else C.c_int64
    vt = C.c_float if value_bits == 32 else C.c_double
    vp = C.c_void_p
    csr = [C.c_int32, it, it, it, vt, it, it, it, vp, vp, vp, vp, vp, it, vp, it, vt, vp, it]
    lib.fusedMM_csr.argtypes = csr
    lib.fusedMM_csr.restype = C.c_int
    lib.fusedMM_csr_stream.argtypes = csr + [vp]
    lib.fusedMM_csr_stream.restype = C.c_int
    lib.fusedMM_csr_stream_noalloc.argtypes = csr + [vp]
    lib.fusedMM_csr_stream_noalloc.restype = C.c_int
    lib.fusedMM_amd_init.restype = C.c_int
    lib.fusedMM_amd_init_noalloc.restype = C.c_int
    lib.fusedMM_amd_noalloc_capacity.restype = C.c_int64
    gf = lib.sgfusedMM_csr if value_bits == 32 else lib.dgfusedMM_csr   # kernels.h:17-37 of the reference
    gf.argtypes = [C.c_char] + csr[1:]
    gf.restype = None
    lib.fusedMM_amd_index_bytes.restype = C.c_int
    lib.fusedMM_amd_value_bytes.restype = C.c_int
    lib.fusedMM_amd_set_sop_kind.argtypes = [C.c_int]
    lib.fusedMM_amd_set_sop_kind.restype = C.c_int
    lib.fusedMM_amd_get_sop_kind.restype = C.c_int
    lib.fusedMM_amd_set_sop_callback.argtypes = [vp]
    lib.fusedMM_amd_set_opt.argtypes = [C.c_int]
    lib.fusedMM_amd_set_opt.restype = C.c_int
    lib.fusedMM_amd_set_validate.argtypes = [C.c_int]
    lib.fusedMM_amd_set_validate.restype = C.c_int
    lib.fusedMM_amd_set_split.argtypes = [C.c_int64, C.c_int]
    lib.fusedMM_amd_timing.argtypes = [C.c_int]
    lib.fusedMM_amd_timing_summary.argtypes = [C.POINTER(C.c_double)] * 3
    lib.fusedMM_amd_timing_summary.restype = C.c_int
    lib.fusedMM_amd_timing_call.argtypes = [C.c_int] + [C.POINTER(C.c_double)] * 3
    lib.fusedMM_amd_timing_call.restype = C.c_int
    lib.fusedMM_amd_last_split.argtypes = [C.POINTER(C.c_uint)] * 3
    lib.fusedMM_amd_last_split.restype = C.c_int
    lib.fusedMM_amd_get_split.argtypes = [C.POINTER(C.c_int64), C.POINTER(C.c_int)]
    lib.fusedMM_amd_get_split.restype = None
    lib.fusedMM_amd_set_pack_rows.argtypes = [C.c_int]
    lib.fusedMM_amd_set_pack_rows.restype = C.c_int
    lib.fusedMM_amd_set_store_tick.argtypes = [C.c_int]
    lib.fusedMM_amd_set_store_tick.restype = C.c_int
    lib.fusedMM_amd_last_row_order.argtypes = [vp, vp, vp]
    lib.fusedMM_amd_last_row_order.restype = C.c_int
    lib.fusedMM_amd_set_stage_callbacks.argtypes = [vp, vp, vp, vp]
    lib.fusedMM_amd_set_stage_callbacks.restype = None
    lib.fusedMM_amd_set_cache.argtypes = [C.c_int]
    lib.fusedMM_amd_set_cache.restype = C.c_int
    lib.fusedMM_amd_invalidate.restype = None
    lib.fusedMM_amd_last_host_phases.argtypes = [C.POINTER(C.c_double)] * 3
    lib.fusedMM_amd_last_host_phases.restype = C.c_int
    assert lib.fusedMM_amd_index_bytes() * 8 == index_bits
    assert lib.fusedMM_amd_value_bytes() * 8 == value_bits
    _libs[key] = lib
    return lib


_probes = None


def load_probes():
    """dlopen libfusedmm_amd_probes.so, the measuring aids of the benchmark (copy, read-stream and
    gather probes; csrc/fusedmm_probes.h): bench.py's yardsticks, not part of the product ABI."""
    global _probes
    if _probes is not None:
        return _probes
    try:
        import torch  # noqa: F401  (one HIP runtime per process, as in load())
    except ImportError:
        pass
    path = probes_path()
    if not os.path.exists(path):
        raise OSError("%s is not built; run `python -m fusedmm_amd.build`" % path)
    lib = C.CDLL(path)
    vp = C.c_void_p
    lib.fusedMM_amd_copy_probe.argtypes = [vp, vp, C.c_int64, vp]
    lib.fusedMM_amd_copy_probe.restype = C.c_int
    lib.fusedMM_amd_read_probe.argtypes = [vp, C.c_int64, C.c_int, C.c_int, C.c_int, vp, vp]
    lib.fusedMM_amd_read_probe.restype = C.c_int
    lib.fusedMM_amd_gather_probe.argtypes = [vp, C.c_int, vp, C.c_int64, C.c_int, C.c_int, C.c_int, vp, vp]
    lib.fusedMM_amd_gather_probe.restype = C.c_int
    _probes = lib
    return lib


def _addr(a):
    """Raw address of a numpy array, a torch tensor, an int, or None."""
    if a is None:
        return None
    if isinstance(a, int):
        return a
    if hasattr(a, "data_ptr"):
        return a.data_ptr()
    return a.ctypes.data


def fusedMM_csr(imessage, m, n, k, alpha, nnz, rows, cols, val, indx, pntrb, pntre, x, ldx, y, ldy, beta, z, ldz,
                index_bits=32, stream=None, value_bits=32, noalloc=False):
    """Same argument list as the C entry point (include/fusedMM.h).  Operands
    are numpy arrays (host memory) or torch tensors / integer addresses (device
    memory).  With `stream` (an integer hipStream_t) the call is asynchronous;
    noalloc=True takes the entry point that allocates nothing."""
    lib = load(index_bits, value_bits)
    args = [imessage, m, n, k, alpha, nnz, rows, cols, _addr(val), _addr(indx), _addr(pntrb), _addr(pntre),
            _addr(x), ldx, _addr(y), ldy, beta, _addr(z), ldz]
    if noalloc:
        return lib.fusedMM_csr_stream_noalloc(*args, stream)
    if stream is None:
        return lib.fusedMM_csr(*args)
    return lib.fusedMM_csr_stream(*args, stream)
