"""The GPU parity tests, as many of them as finish quickly, against the library built for the host.

tests/cpu_sim/build_sim.py links the library's own host objects (the ones inside libophip.so) with its kernel sources
compiled for the host and with a stand-in for the HIP runtime: device memory is host memory between guard pages,
a launch runs the kernel work-item by work-item (MFMA, shuffles, DPP, buffer resources and the transposing LDS read
emulated per wave of 64), a recording stream keeps its launches for replay.  This test starts pytest again on the GPU
tests named in tests/cpu_sim/selection.txt with the environment variable that makes tests/conftest.py load that build,
so the same test code, the same oracle and the same bars apply.  What it shows without a GPU: that the host side plans
launches whose every access stays inside its operands (a stray access stops the run and names the allocation), that the
kernels compute what the oracle computes, including the hand-over between workgroups, and that the C ABI behaves the
same from creation to destruction.  What it cannot show: anything about time, and whatever depends on how the hardware
interleaves waves.  The tests marked `gpu` remain the parity tests proper; on a GPU box they load libophip.so.

selection.txt lists test ids that take a few seconds at most here (the large shapes are left to the GPU); it was made
by running every GPU test this way once and keeping the fast ones (tests/cpu_sim/select_tests.py).
"""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SIM = os.path.join(ROOT, "tests", "cpu_sim")


@pytest.fixture(scope="module")
def sim_library():
    sys.path.insert(0, SIM)
    try:
        import build_sim
    finally:
        sys.path.remove(SIM)
    if build_sim.compiler() is None:
        pytest.skip("no clang++ (the kernel sources use clang's vector extensions)")
    return build_sim.build()


def selection():
    by_file = {}
    for line in open(os.path.join(SIM, "selection.txt")):
        line = line.strip()
        if line and not line.startswith("#"):
            by_file.setdefault(line.split("::")[0], []).append(line)
    return by_file


@pytest.mark.parametrize("test_file", sorted(selection()))
def test_gpu_tests_against_the_host_build(sim_library, test_file):
    ids = selection()[test_file]
    env = dict(os.environ, OPHIP_CPU_SIM_LIBRARY=sim_library)
    cmd = [sys.executable, "-m", "pytest", "-m", "gpu", "-q", "-p", "no:cacheprovider", "--timeout", "300", "-n", "4"] + ids
    r = subprocess.run(cmd, cwd=ROOT, env=env, capture_output=True, text=True, timeout=1500)
    tail = (r.stdout + r.stderr)[-6000:]
    assert r.returncode == 0, tail
    assert ("%d passed" % len(ids)) in tail, tail  # none skipped, none deselected
