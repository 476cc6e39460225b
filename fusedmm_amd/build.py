"""Build recipe for the gfx950 libraries of this package.

    python -m fusedmm_amd.build            # every library, objects in parallel, only what changed
    python -m fusedmm_amd.build --force    # recompile everything

libfusedmm_amd_i32.so / _i64.so (float) and libfusedmm_amd_d_i32.so / _d_i64.so (double) are
linked from a dozen objects each (csrc/*.hip; the fused kernel's instances are spread over
eight of them, one per op), libfusedmm_amd_probes.so holds the benchmark's yardsticks.  The
libraries are written next to this file so that they travel with the source tree; nothing is
installed.  Objects go to fusedmm_amd/obj/.
"""
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "obj")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")

HIPCC = os.environ.get("HIPCC", "hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # the wavefront summation order is a numerical contract with the tests:
    # fuse only where the source says fmaf
    "-ffp-contract=off",
    # scalar fp32 arithmetic only.  A device-side feature; hipcc hands -Xclang options to its host pass as
    # well (-Xarch_device takes no option with an argument), which answers with the line filtered below.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# experiments: FUSEDMM_BUILD_EXTRA="-DX=1 ..." adds compiler flags, FUSEDMM_BUILD_OUT=<dir> writes libraries and
# objects there (load them with FUSEDMM_AMD_LIB_DIR=<dir>)
FLAGS += os.environ.get("FUSEDMM_BUILD_EXTRA", "").split()
if os.environ.get("FUSEDMM_BUILD_OUT"):
    OUT = os.path.abspath(os.environ["FUSEDMM_BUILD_OUT"])
    OBJ = os.path.join(OUT, "obj")
else:
    OUT = HERE
HOST_PASS_NOISE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"

# translation units of a product library: (source, extra defines, object tag)
LAUNCH_UNITS = 8
UNITS = [("fusedmm_state.hip", [], "state"), ("fusedmm_dispatch.hip", [], "dispatch"),
         ("fusedmm_staging.hip", [], "staging"), ("fusedmm_host_stages.hip", [], "host_stages"),
         ("fusedmm_exports.hip", [], "exports")] + \
        [("fusedmm_launch.hip", ["-DFMM_LAUNCH_UNIT=%d" % u], "launch%d" % u) for u in range(LAUNCH_UNITS)]
VARIANTS = ((32, 32), (64, 32), (32, 64), (64, 64))     # (index bits, value bits)
JOBS = int(os.environ.get("FUSEDMM_BUILD_JOBS", "0")) or min(16, os.cpu_count() or 4)


def lib_name(index_bits, value_bits=32):
    """libfusedmm_amd_i<bits>.so for float (the reference's default), libfusedmm_amd_d_i<bits>.so for double."""
    return "libfusedmm_amd_%si%d.so" % ("d_" if value_bits == 64 else "", index_bits)


def lib_path(index_bits, value_bits=32):
    """Where the library for INDEXTYPE = int<index_bits>_t lives; FUSEDMM_AMD_LIB_DIR
    points the loader at another build of it."""
    return os.path.join(os.environ.get("FUSEDMM_AMD_LIB_DIR", HERE), lib_name(index_bits, value_bits))


def probes_path():
    p = os.path.join(os.environ.get("FUSEDMM_AMD_LIB_DIR", HERE), "libfusedmm_amd_probes.so")
    return p if os.path.exists(p) else os.path.join(HERE, "libfusedmm_amd_probes.so")


def variant_defines(index_bits, value_bits):
    return ["-DINDEXTYPE=int%d_t" % index_bits] + (["-DDREAL"] if value_bits == 64 else [])


def _headers():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".h", ".hpp"))]
    hs += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE) if f.endswith(".h")]
    return hs


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    said = "\n".join(ln for ln in r.stdout.splitlines() if ln.strip() and HOST_PASS_NOISE not in ln)
    if said:                         # warnings (and errors) of the compiler, minus the one known line
        sys.stderr.write(said + "\n")
    if r.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd))
    return r.stdout


def _compile(src, obj, defines, force, verbose):
    """hipcc -c src -> obj unless obj is newer than the source, every header and this recipe's flags."""
    cmd = [HIPCC] + FLAGS + defines + ["-c", os.path.join(CSRC, src), "-o", obj]
    stamp = obj + ".cmd"
    digest = hashlib.sha1(" ".join(cmd).encode()).hexdigest()
    if not force and os.path.exists(obj) and os.path.exists(stamp) and open(stamp).read() == digest:
        t = os.path.getmtime(obj)
        if all(os.path.getmtime(p) <= t for p in [os.path.join(CSRC, src)] + _headers()):
            return obj
    _run(cmd, verbose)
    with open(stamp, "w") as f:
        f.write(digest)
    return obj


def _objects(index_bits, value_bits):
    tag = "%si%d" % ("d_" if value_bits == 64 else "", index_bits)
    return [(src, os.path.join(OBJ, "%s_%s.o" % (name, tag)), variant_defines(index_bits, value_bits) + defs)
            for src, defs, name in UNITS]


def _link(out, objs, verbose, extra=()):
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs + list(extra), verbose)
    return out


def build_libs(variants=VARIANTS, force=False, verbose=False, probes=True):
    """Compile the objects of the requested libraries side by side, then link each library."""
    os.makedirs(OBJ, exist_ok=True)
    jobs = []
    for ib, vb in variants:
        jobs += _objects(ib, vb)
    if probes:
        jobs.append(("fusedmm_probes.hip", os.path.join(OBJ, "probes.o"), []))
    # the objects with the most kernel instances first, so that they do not end the build alone
    jobs.sort(key=lambda j: 0 if "launch" in j[1] else 1)
    with ThreadPoolExecutor(JOBS) as ex:
        list(ex.map(lambda j: _compile(j[0], j[1], j[2], force, verbose), jobs))
    libs = []
    for ib, vb in variants:
        libs.append(_link(os.path.join(OUT, lib_name(ib, vb)), [o for _, o, _ in _objects(ib, vb)], verbose, ["-ldl"]))
    if probes:
        libs.append(_link(os.path.join(OUT, "libfusedmm_amd_probes.so"), [os.path.join(OBJ, "probes.o")], verbose))
    return libs


def build_one(index_bits, value_bits=32, verbose=False, force=False):
    return build_libs(((index_bits, value_bits),), force, verbose, probes=False)[0]


def timer_path(index_bits, value_bits=32):
    return os.path.join(HERE, "bin", "xfusedMMtime_%si%d" % ("d_" if value_bits == 64 else "", index_bits))


def dropin_path(index_bits):
    return os.path.join(HERE, "bin", "xdropin_example_i%d" % index_bits)


def harness_lib_path(index_bits):
    return os.path.join(HERE, "libfusedmm_harness_i%d.so" % index_bits)


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


def build_all(verbose=False, force=False):
    libs = build_libs(VARIANTS, force, verbose)
    with ThreadPoolExecutor(2) as ex:
        exes = list(ex.map(lambda b: build_timer(b, verbose), (32, 64)))
    return libs + exes


if __name__ == "__main__":
    for p in build_all(verbose=True, force="--force" in sys.argv[1:]):
        print("built", p)
