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
