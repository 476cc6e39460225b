"""The tester/timer executable on a small .mtx: the reference's own workflow
(`x...time -input f.mtx -T 1 -K k`) must pass its tester and print the CSV."""
import os
import subprocess

import pytest

from fusedmm_amd import build as fbuild
from fusedmm_amd import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [32, 64])
@pytest.mark.parametrize("tkern,k", [("f", 32), ("s", 128), ("t", 64), ("m", 256), ("g", 40)])
def test_timer_passes_its_tester(tmp_path, tkern, k, bits):
    g = synth.er_graph(4096, 32768, 1, bits)
    path = str(tmp_path / "er.mtx")
    synth.write_mtx_symmetric(path, g)
    exe = fbuild.timer_path(bits)
    assert os.path.exists(exe)
    r = subprocess.run([exe, "-input", path, "-T", "1", "-K", str(k), "-t", tkern, "-nrep", "3"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    print(r.stdout)
    assert r.returncode == 0, r.stdout
    assert "PASSED TEST" in r.stdout
    lines = [l for l in r.stdout.splitlines() if "," in l]
    assert lines[-2].startswith("Filename,NNZ,M,N,K,Trusted_exe_time,Test_exe_time,Speedup_exe_time")
    f = lines[-1].split(",")
    assert f[1:5] == [str(g["nnz"]), "4096", "4096", str(k)]
    assert float(f[6]) > 0 and float(f[8]) > 0


@pytest.mark.parametrize("tkern,k", [("s", 128), ("f", 32), ("m", 64)])
def test_timer_general_pipeline(tmp_path, tkern, k):
    """-opt 0: what the reference's xsFusedMMtime_* executables (no ENABLE_OPT_FUSEDMM) run,
    the general pipeline for the same tuples; -opt 2 (MUST_OPT_FUSEDMM) still finds the
    optimised kernels of these tuples."""
    g = synth.er_graph(4096, 32768, 5, 32)
    path = str(tmp_path / "er.mtx")
    synth.write_mtx_symmetric(path, g)
    for opt in ("0", "2"):
        r = subprocess.run([fbuild.timer_path(32), "-input", path, "-T", "1", "-K", str(k), "-t", tkern, "-nrep", "2",
                            "-opt", opt], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
        assert r.returncode == 0 and "PASSED TEST" in r.stdout, r.stdout


def test_timer_host_pointer_mode(tmp_path):
    g = synth.er_graph(2048, 16384, 2, 64)
    path = str(tmp_path / "er.mtx")
    synth.write_mtx_symmetric(path, g)
    r = subprocess.run([fbuild.timer_path(64), "-input", path, "-T", "1", "-K", "64", "-t", "s", "-nrep", "2",
                        "-gpu", "0", "-skHd", "1", "-M", "1000"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    assert r.returncode == 0 and "PASSED TEST" in r.stdout, r.stdout
    assert "Filename" not in r.stdout
    assert r.stdout.strip().splitlines()[-1].split(",")[2] == "1000"


@pytest.mark.parametrize("bits", [32, 64])
def test_reference_style_c_caller(bits):
    """Plain-C program that includes only fusedMM.h, defines SOP_UDEF_FUNC itself
    and passes host arrays -- the reference's calling convention, untouched."""
    r = subprocess.run([fbuild.dropin_path(bits)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout


def test_timer_double_precision(tmp_path):
    g = synth.er_graph(2048, 16384, 3, 64)
    path = str(tmp_path / "er.mtx")
    synth.write_mtx_symmetric(path, g)
    for tkern in ("s", "t", "m"):
        r = subprocess.run([fbuild.timer_path(64, 64), "-input", path, "-T", "1", "-K", "96", "-t", tkern, "-nrep", "2"],
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
        assert r.returncode == 0 and "PASSED TEST" in r.stdout, r.stdout


def test_sweep_script(tmp_path):
    """The counterpart of the reference's runtime.sh: one CSV per dataset and kind."""
    g = synth.er_graph(1024, 8192, 4, 32)
    path = str(tmp_path / "tiny.mtx")
    synth.write_mtx_symmetric(path, g)
    script = os.path.join(os.path.dirname(fbuild.timer_path(32)), "..", "runtime_sweep.sh")
    r = subprocess.run(["bash", script, "-i", "32", "-r", str(tmp_path / "res"), path],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=280)
    assert r.returncode == 0, r.stdout
    lines = open(str(tmp_path / "res" / "tiny-s-sreal-gpu.csv")).read().strip().splitlines()
    assert lines[0].startswith("Filename,NNZ") and len(lines) == 9
    assert [l.split(",")[4] for l in lines[1:]] == ["32", "64", "96", "128", "160", "192", "224", "256"]


def test_config1_through_the_timer(tmp_path):
    """Benchmark configuration 1 end to end, the way the reference runs it
    (x..time_fr -input file.mtx -T 1 -K 32): symmetric ER graph with 16 384 nodes
    and 131 072 undirected pairs written as .mtx from seed, loaded by the timer's
    own loader, FR op, tester on, then timed."""
    from bench import make_workload
    g, _, _ = make_workload("c1")
    path = str(tmp_path / "c1.mtx")
    synth.write_mtx_symmetric(path, g)
    exe = os.path.join(str(tmp_path), "xsOptFusedMMtime_fr_pt")     # the reference's executable name selects the kind
    os.symlink(fbuild.timer_path(64), exe)
    r = subprocess.run([exe, "-input", path, "-T", "1", "-K", "32", "-nrep", "5"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=200)
    assert r.returncode == 0 and "PASSED TEST" in r.stdout, r.stdout
    f = r.stdout.strip().splitlines()[-1].split(",")
    assert f[1:5] == ["262144", "16384", "16384", "32"]
