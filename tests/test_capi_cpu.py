"""Host-side checks of the C ABI that need no GPU: the libraries load, export
every entry point the headers declare, and reject malformed op tuples with the
reference's status codes before touching the device."""
import os
import re

import numpy as np
import pytest

import fusedmm_amd as fa

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_entry_points():
    names = set()
    for h in ("fusedMM.h", "fusedmm_amd.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b((?:fusedMM_|sgfusedMM_|dgfusedMM_)\w+)\s*\(", text))
    names.discard("fusedMM_amd_sop_fn")
    return sorted(names)


@pytest.mark.parametrize("vbits", [32, 64])
@pytest.mark.parametrize("bits", [32, 64])
def test_library_exports_declared_symbols(bits, vbits):
    lib = fa.load(bits, vbits)
    names = declared_entry_points()
    assert "fusedMM_csr" in names and "fusedMM_csr_stream" in names and len(names) >= 14
    # the second-level entry is named after the precision, as in the reference (kernels.h:17-37)
    own, other = ("sgfusedMM_csr", "dgfusedMM_csr") if vbits == 32 else ("dgfusedMM_csr", "sgfusedMM_csr")
    for n in names:
        if n != other:
            assert hasattr(lib, n), n
    assert set(names) == set(fa.EXPORTS) | {own, other}
    assert lib.fusedMM_amd_index_bytes() * 8 == bits and lib.fusedMM_amd_value_bytes() * 8 == vbits


def test_header_constants_match_python_mirror():
    text = open(os.path.join(ROOT, "include", "fusedMM.h")).read()
    for name in ("VOP_COPY_RHS", "VOP_SUBR", "ROP_DOT", "ROP_NORMR", "SOP_UDEF", "VSC_MUL", "AOP_ADD", "AOP_MIN"):
        m = re.search(r"#define\s+%s\s+(0x[0-9A-Fa-f]+)" % name, text)
        assert m and int(m.group(1), 16) == getattr(fa, name), name
    assert fa.MSG_SIGMOID == 0x11F12 and fa.MSG_TDIST == 0x11F55 and fa.MSG_SPMM == 0x11102 and fa.MSG_GCN == 0x10002


@pytest.mark.parametrize("bits", [32, 64])
def test_bad_tuples_rejected_like_the_reference(bits):
    """Order and codes of reference fusedMM.c:610-628; no operand is read."""
    it = np.int32 if bits == 32 else np.int64
    p = np.zeros(4, it)
    f = np.zeros(16, np.float32)
    call = lambda imsg: fa.fusedMM_csr(imsg, 2, 2, 4, 1.0, 0, 2, 2, f, p, p, p, f, 4, f, 4, 0.0, f, 4, index_bits=bits)
    assert call(0x11100) == fa.VOP_FAIL              # VOP_NOOP is not accepted
    assert call(0x11108) == fa.VOP_FAIL
    assert call(0x11162) == fa.ROP_FAIL
    assert call(0x11202) == fa.SOP_FAIL
    assert call(0x13102) == fa.VSC_FAIL
    assert call(0x41102) == fa.AOP_FAIL
    assert call(0x1110F) == fa.UNDEFINED_USER_FUNCTION   # VOP_UDEF: no user function on the device
    assert call(0x111F2) == fa.UNDEFINED_USER_FUNCTION
    assert call(0x1F102) == fa.UNDEFINED_USER_FUNCTION
    assert call(0xF1102) == fa.UNDEFINED_USER_FUNCTION
    # first failing stage wins
    assert call(0x43208) == fa.VOP_FAIL


def test_sop_kind_selection():
    lib = fa.load(32)
    prev = lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_FR)
    assert lib.fusedMM_amd_get_sop_kind() == fa.SOP_KIND_FR
    assert lib.fusedMM_amd_set_sop_kind(99) == -2
    assert lib.fusedMM_amd_get_sop_kind() == fa.SOP_KIND_FR
    lib.fusedMM_amd_set_sop_kind(prev)
    assert lib.fusedMM_amd_set_opt(1) in (0, 1)


@pytest.mark.parametrize("idx,val", [("int32_t", "float"), ("int64_t", "float"), ("int64_t", "double")])
@pytest.mark.parametrize("compiler,std", [("gcc", "-std=c99"), ("g++", "-std=c++11")])
def test_headers_compile_as_plain_c_and_cpp(tmp_path, compiler, std, idx, val):
    """The boundary is a C ABI: both headers must compile as C99 and as C++11 with
    nothing but INDEXTYPE / VALUETYPE defined, as the reference's header does."""
    import subprocess
    src = tmp_path / ("t.c" if compiler == "gcc" else "t.cpp")
    src.write_text('#include <stdint.h>\n#include "fusedMM.h"\n#include "fusedmm_amd.h"\n'
                   'int probe(void) { return VOP_COPY_RHS | ROP_DOT | SOP_UDEF | VSC_MUL | AOP_ADD; }\n')
    r = subprocess.run([compiler, std, "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only",
                        "-DINDEXTYPE=" + idx, "-DVALUETYPE=" + val, "-I", os.path.join(ROOT, "include"), str(src)],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout


def test_must_opt_mode_refuses_unmatched_tuples():
    """fusedMM_amd_set_opt(2) is the reference built with MUST_OPT_FUSEDMM (fusedMM.c:599-604):
    a tuple that matches none of the optimised kernels returns FUSEDMM_NO_OPT_IMPL.  Decided
    from the op tuple alone, before any operand is looked at."""
    lib = fa.load(32)
    p = np.zeros(4, np.int32)
    f = np.zeros(16, np.float32)
    call = lambda imsg: fa.fusedMM_csr(imsg, 0, 2, 4, 1.0, 0, 2, 2, f, p, p, p, f, 4, f, 4, 0.0, f, 4)
    prev = lib.fusedMM_amd_set_opt(2)
    try:
        assert lib.fusedMM_amd_set_opt(2) == 2
        for matched in (fa.MSG_GCN, fa.MSG_SPMM, fa.MSG_SIGMOID, fa.MSG_TDIST):
            assert call(matched) != fa.NO_OPT_IMPL
        assert call(fa.VOP_ADD | fa.ROP_DOT | fa.SOP_COPY | fa.VSC_MUL | fa.AOP_ADD) == fa.NO_OPT_IMPL
        assert call(fa.VOP_COPY_RHS | fa.ROP_NOOP | fa.SOP_COPY | fa.VSC_MUL | fa.AOP_MAX) == fa.NO_OPT_IMPL
        assert call(0x11100) == fa.VOP_FAIL            # a malformed tuple keeps its own code
        lib.fusedMM_amd_set_opt(1)
        assert call(fa.VOP_ADD | fa.ROP_DOT | fa.SOP_COPY | fa.VSC_MUL | fa.AOP_ADD) != fa.NO_OPT_IMPL
    finally:
        lib.fusedMM_amd_set_opt(prev)


def test_cmake_target_of_the_reference_configures(tmp_path):
    """The consumer project (add_subdirectory + target_link_libraries(... fusedmm), as the
    reference's CMakeLists.txt:1-14 is used) configures; where the in-tree build exists,
    its executable really links the library the target names."""
    import shutil
    import subprocess
    if not shutil.which("cmake"):
        pytest.skip("cmake not installed")
    src = os.path.join(ROOT, "fusedmm_amd", "consumer")
    r = subprocess.run(["cmake", "-S", src, "-B", str(tmp_path / "b"), "-DFUSEDMM_INDEX_BITS=32"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0, r.stdout
    r = subprocess.run(["cmake", "--build", str(tmp_path / "b"), "--target", "help"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert "xconsumer" in r.stdout and "fusedmm_build" in r.stdout
    exe = os.path.join(ROOT, "fusedmm_amd", "cmake_build", "xconsumer")
    if os.path.exists(exe):
        r = subprocess.run(["readelf", "-d", exe], stdout=subprocess.PIPE, text=True)
        assert "libfusedmm.so" in r.stdout


def test_measuring_aids_are_not_in_the_product_libraries():
    """The copy, read-stream and gather probes are the benchmark's yardsticks: they live in a library of
    their own, and the libraries a consumer links export nothing of the kind."""
    import subprocess
    from fusedmm_amd import build
    for bits in (32, 64):
        for vbits in (32, 64):
            syms = subprocess.run(["nm", "-D", "--defined-only", build.lib_path(bits, vbits)], stdout=subprocess.PIPE, text=True).stdout
            assert "probe" not in syms
            c_names = set(re.findall(r" T (\w+)$", syms, flags=re.M))
            own = "sgfusedMM_csr" if vbits == 32 else "dgfusedMM_csr"
            # what the library exports by a C name is exactly what the headers declare (kernel stubs aside)
            assert {n for n in c_names if not n.startswith("_")} == set(fa.EXPORTS) | {own}
    syms = subprocess.run(["nm", "-D", "--defined-only", build.probes_path()], stdout=subprocess.PIPE, text=True).stdout
    assert set(re.findall(r" T (\w+)$", syms, flags=re.M)) == set(fa.PROBE_EXPORTS)
    probes = fa.load_probes()
    for n in fa.PROBE_EXPORTS:
        assert hasattr(probes, n)
    text = open(os.path.join(ROOT, "include", "fusedmm_amd.h")).read()
    assert "probe" not in text


_CHILD = r"""
import ctypes as C, sys
import numpy as np
sys.path.insert(0, %r)
import fusedmm_amd as fa
lib = fa.load(32)
%s
"""


def _child(body, **env):
    import subprocess
    import sys
    e = dict(os.environ, **env)
    return subprocess.run([sys.executable, "-c", _CHILD % (ROOT, body)], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          text=True, timeout=120, env=e)


def test_no_usable_gpu_is_a_status_code_not_an_abort():
    """A well-formed call (valid tuple, m > 0, host operands) in a process that sees no GPU: the HIP runtime's
    error becomes FUSEDMM_FAIL_RETURN (reference fusedMM.h:103-112) with a message on stderr; the process goes on.
    The condition is forced from the host (the devices are hidden from the child), so it holds on a GPU box too."""
    body = (
        "p = np.array([0, 2, 4], np.int32); ix = np.array([0, 1, 1, 0], np.int32)\n"
        "v = np.ones(4, np.float32); X = np.ones((2, 8), np.float32); Z = np.zeros((2, 8), np.float32)\n"
        "lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_SIGMOID)\n"
        "for msg in (fa.MSG_SIGMOID, fa.MSG_GCN, fa.VOP_ADD | fa.ROP_DOT | fa.SOP_COPY | fa.VSC_MUL | fa.AOP_MAX):\n"
        "    rc = fa.fusedMM_csr(msg, 2, 2, 8, 1.0, 4, 2, 2, v, ix, p[:-1], p[1:], X, 8, X, 8, 0.0, Z, 8)\n"
        "    print('rc', rc)\n"
        "print('init', lib.fusedMM_amd_init(), lib.fusedMM_amd_init_noalloc())\n"
        "print('m0', fa.fusedMM_csr(fa.MSG_GCN, 0, 2, 8, 1.0, 4, 2, 2, v, ix, p[:-1], p[1:], X, 8, X, 8, 0.0, Z, 8))\n"
        "print('alive', float(Z.sum()))\n")
    r = _child(body, HIP_VISIBLE_DEVICES="", ROCR_VISIBLE_DEVICES="", CUDA_VISIBLE_DEVICES="")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = r.stdout.split()
    assert r.stdout.count("rc %d" % fa.FAIL) == 3, r.stdout
    assert "init %d %d" % (fa.FAIL, fa.FAIL) in r.stdout
    assert "m0 0" in r.stdout                          # nothing to do: success without touching any device
    assert "alive 0.0" in r.stdout                     # Z untouched, process alive
    assert "fusedmm_amd:" in r.stderr and "failed" in r.stderr


def test_a_setter_overrides_the_environment_whenever_it_is_called():
    """FUSEDMM_SPLIT / FUSEDMM_SOP_KIND are read once, by the first call into the library, whichever it is; a value
    set through the API afterwards (also as the very first call) stays in force."""
    body = (
        "h, s = C.c_int64(), C.c_int()\n"
        "%s"
        "lib.fusedMM_amd_get_split(C.byref(h), C.byref(s)); print('split', h.value, s.value)\n"
        "print('kind', lib.fusedMM_amd_get_sop_kind())\n")
    env = dict(FUSEDMM_SPLIT="300,150", FUSEDMM_SOP_KIND="fr")
    r = _child(body % "", **env)
    assert "split 300 150" in r.stdout and "kind %d" % fa.SOP_KIND_FR in r.stdout, r.stdout + r.stderr
    r = _child(body % "lib.fusedMM_amd_set_split(40, 20); lib.fusedMM_amd_set_sop_kind(fa.SOP_KIND_TDIST_PLAIN)\n", **env)
    assert "split 40 20" in r.stdout and "kind %d" % fa.SOP_KIND_TDIST_PLAIN in r.stdout, r.stdout + r.stderr
    r = _child(body % "lib.fusedMM_amd_set_split(0, 0)\n", **env)      # back to the defaults, not back to the variable
    assert "split 0 0" in r.stdout, r.stdout
    assert lib_rejects_unknown_kind()


def lib_rejects_unknown_kind():
    lib = fa.load(32)
    return lib.fusedMM_amd_set_sop_kind(7) == -2 and lib.fusedMM_amd_set_sop_kind(-2) == -2
