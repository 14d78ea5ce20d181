"""The weight-streaming mat_mul kernels, as they are written, on the CPU.

tests/cpu_sim/hip/hip_runtime.h stands in for the HIP headers: every work-item a fiber, workgroups one after
another, MFMA / shuffles / buffer resources emulated.  tests/cpu_sim/gemm_cpu.cpp compiles
operators-rs_amd/csrc/kernels/gemm.hip with it for the host, under AddressSanitizer and UndefinedBehaviorSanitizer,
gives every operand a heap block of exactly its size, launches gemm_stream_m1 (grid from the function the library's
host side uses) or gemm_skinny_m1_q0 over a small product and compares with a double-precision product.  What this
pins without a GPU: that no work-item of any workgroup touches a byte outside an operand, for even and uneven cuts of
K, every alignment class of the weight, partial last strips, few rows, batches; that K ranges meet correctly (the
workgroup that runs last sums the others' partials, over a workspace that held NaNs) and leave their arrival counters
at zero; that a K range past the end of K (a cut the planner never emits) is harmless.  The parity tests proper
(tests/test_gpu_ops.py) run on the GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLANG = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib", "llvm", "bin", "clang++")


@pytest.fixture(scope="module")
def gemm_cpu(tmp_path_factory):
    cxx = CLANG if os.path.exists(CLANG) else shutil.which("clang++")
    if cxx is None:
        pytest.skip("no clang++ (the kernel sources use clang's vector extensions)")
    exe = str(tmp_path_factory.mktemp("cpu_sim") / "gemm_cpu")
    sim = os.path.join(ROOT, "tests", "cpu_sim")
    res = subprocess.run([cxx, "-std=c++20", "-O1", "-g", "-pthread", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                          "-x", "c++", "-I", sim, "-I", os.path.join(ROOT, "operators-rs_amd", "csrc", "kernels"), "-Wno-unused-value",
                          "-o", exe, os.path.join(sim, "gemm_cpu.cpp")], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-4000:]

    def run(*args):
        r = subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=600)
        return r.returncode, (r.stdout + r.stderr).strip()
    return run


# kernel, M, N, K, batch, split_k, slow_mask, split_slow, first granule of Q
CASES = [
    ("stream", 16, 128, 64, 1, 1, 0, 0, 0),
    ("stream", 16, 256, 128, 1, 2, 0, 0, 0),
    ("stream", 16, 1160, 256, 1, 2, 0x22, 4, 0),     # partial last strip, uneven cut
    ("stream", 16, 1160, 256, 1, 2, 0x22, 4, 3),     # the same with the weight three granules further on
    ("stream", 5, 2056, 128, 1, 1, 0x22, 2, 5),
    ("stream", 16, 1024, 64, 1, 1, 0x22, 2, 1),      # ranges of a single K-step
    ("stream", 16, 1024, 32, 1, 1, 0, 0, 0),         # one K-step: three of the four waves have none
    ("stream", 9, 640, 352, 1, 1, 0x22, 11, 3),      # 11 K-steps in 11 ranges
    ("stream", 16, 512, 256, 3, 2, 0x22, 4, 0),      # batched
    ("stream", 1, 384, 4096, 1, 8, 0, 0, 0),         # one row, long K
    ("stream", 16, 8, 32, 1, 1, 0, 0, 0),            # a strip of 8 columns
    ("stream", 16, 136, 96, 2, 3, 0xFF, 1, 0),       # every strip "slow", fewer ranges than the others would get
    ("stream", 16, 1024, 128, 1, 1, 0x22, 3, 0),     # 4 K-steps in 3 ranges of 2: the third starts past K and is empty
    ("skinny", 16, 256, 100, 1, 2, 0, 0, 0),         # the older kernel: ragged last K-step
    ("skinny", 7, 136, 33, 2, 1, 0, 0, 0),
    ("skinny", 16, 384, 1024, 1, 4, 0, 0, 0),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(str(v) for v in c))
def test_kernel_source_on_the_cpu(gemm_cpu, case):
    rc, out = gemm_cpu(*case)
    assert rc == 0 and "0 bad, 0 counters not back at zero, 0 accesses past" in out, out


def test_the_cpu_build_does_catch_an_access_outside_an_operand(gemm_cpu):
    """The check of the checker: a K that the arguments overstate (the kernel is told 96 rows, the operands hold 64)
    makes the kernel read past both operands, and the sanitizer stops it."""
    rc, out = gemm_cpu("stream", 16, 128, 64, 1, 1, 0, 0, 0, 32)
    assert rc != 0 and "AddressSanitizer" in out, out
