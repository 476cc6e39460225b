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


def lib_path(index_bits):
    return os.path.join(HERE, "libfusedmm_amd_i%d.so" % index_bits)


def build_one(index_bits, verbose=False):
    out = lib_path(index_bits)
    cmd = [HIPCC] + FLAGS + ["-DINDEXTYPE=int%d_t" % index_bits,
                             os.path.join(CSRC, "fusedmm_capi.hip"), "-o", out, "-ldl"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout)
        raise RuntimeError("hipcc failed for int%d" % index_bits)
    return out


def build_all(verbose=False):
    with ThreadPoolExecutor(2) as ex:
        return list(ex.map(lambda b: build_one(b, verbose), (32, 64)))


if __name__ == "__main__":
    for p in build_all(verbose=True):
        print("built", p)
