"""Build recipe for libfusedmm_amd_i32.so / libfusedmm_amd_i64.so (gfx950).

    python -m fusedmm_amd.build            # both index widths, in parallel

The libraries are written next to this file so that they travel with the
source tree; nothing is installed.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")

HIPCC = os.environ.get("HIPCC", "hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    # the wavefront summation order is a numerical contract with the tests:
    # fuse only where the source says fmaf
    "-ffp-contract=off",
    # scalar fp32 arithmetic only
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def lib_name(index_bits, value_bits=32):
    """libfusedmm_amd_i<bits>.so for float (the reference's default), libfusedmm_amd_d_i<bits>.so for double."""
    return "libfusedmm_amd_%si%d.so" % ("d_" if value_bits == 64 else "", index_bits)


def lib_path(index_bits, value_bits=32):
    """Where the library for INDEXTYPE = int<index_bits>_t lives; FUSEDMM_AMD_LIB_DIR
    points the loader at another build of it."""
    return os.path.join(os.environ.get("FUSEDMM_AMD_LIB_DIR", HERE), lib_name(index_bits, value_bits))


def build_one(index_bits, value_bits=32, verbose=False):
    out = os.path.join(HERE, lib_name(index_bits, value_bits))
    cmd = [HIPCC] + FLAGS + ["-DINDEXTYPE=int%d_t" % index_bits] + (["-DDREAL"] if value_bits == 64 else []) + \
          [os.path.join(CSRC, "fusedmm_capi.hip"), "-o", out, "-ldl"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout)
        raise RuntimeError("hipcc failed for int%d / %d-bit values" % (index_bits, value_bits))
    return out


def timer_path(index_bits, value_bits=32):
    return os.path.join(HERE, "bin", "xfusedMMtime_%si%d" % ("d_" if value_bits == 64 else "", index_bits))


def dropin_path(index_bits):
    return os.path.join(HERE, "bin", "xdropin_example_i%d" % index_bits)


def harness_lib_path(index_bits):
    return os.path.join(HERE, "libfusedmm_harness_i%d.so" % index_bits)


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout)
        raise RuntimeError("build step failed: " + " ".join(cmd))


def build_timer(index_bits, verbose=False):
    """The tester/timer executable (csrc/fusedMMtime.cpp) and the loader's C doorway."""
    os.makedirs(os.path.join(HERE, "bin"), exist_ok=True)
    for vbits in (32, 64):
        exe_v = timer_path(index_bits, vbits)
        _run([HIPCC, "-O2", "-std=c++17", "-fopenmp", "-DINDEXTYPE=int%d_t" % index_bits] +
             (["-DDREAL"] if vbits == 64 else []) +
             [os.path.join(CSRC, "fusedMMtime.cpp"), "-o", exe_v, "-L" + HERE,
              "-l" + lib_name(index_bits, vbits)[3:-3],
              "-Wl,-rpath,$ORIGIN/..", "-L/opt/rocm/lib", "-lrocprofiler-sdk-roctx", "-Wl,-rpath,/opt/rocm/lib"], verbose)
    exe = timer_path(index_bits)
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-DINDEXTYPE=int%d_t" % index_bits,
          os.path.join(CSRC, "harness_capi.cpp"), "-o", harness_lib_path(index_bits)], verbose)
    # a reference-style caller in plain C (gcc, host pointers, its own SOP_UDEF_FUNC)
    _run(["gcc", "-O2", "-DINDEXTYPE=int%d_t" % index_bits, "-DVALUETYPE=float",
          os.path.join(CSRC, "dropin_example.c"), "-rdynamic", "-o", dropin_path(index_bits), "-L" + HERE,
          "-lfusedmm_amd_i%d" % index_bits, "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath-link,/opt/rocm/lib", "-lm"], verbose)
    return exe


def build_all(verbose=False):
    with ThreadPoolExecutor(4) as ex:
        libs = list(ex.map(lambda a: build_one(a[0], a[1], verbose), ((32, 32), (64, 32), (32, 64), (64, 64))))
        exes = list(ex.map(lambda b: build_timer(b, verbose), (32, 64)))
    return libs + exes


if __name__ == "__main__":
    for p in build_all(verbose=True):
        print("built", p)
