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
import shutil
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


def hand_over_tests():
    """The selected tests of kernels in which workgroups or waves hand data to each other (K ranges of a product, key
    ranges of attention, the passes of sampling, rows spread over waves)."""
    words = ("split_k", "stream", "decode", "kv_cached", "one_pass", "sample", "softmax")
    return [t for ids in selection().values() for t in ids if any(w in t for w in words)]


@pytest.mark.parametrize("schedule", ["shuffle:5"])  # ("reverse" is the other order the stand-in knows)
def test_results_do_not_depend_on_the_order_of_workgroups_and_waves(sim_library, schedule):
    """Between barriers the hardware runs workgroups and waves in any order it likes.  The stand-in runs them in a fixed
    one by default; here backwards, and in a pseudo-random order that changes at every point where work-items wait for
    each other.  The same tests must pass (several of them compare bit for bit)."""
    ids = hand_over_tests()
    assert len(ids) > 50
    env = dict(os.environ, OPHIP_CPU_SIM_LIBRARY=sim_library, CPUSIM_SCHEDULE=schedule)
    cmd = [sys.executable, "-m", "pytest", "-m", "gpu", "-q", "-p", "no:cacheprovider", "--timeout", "300", "-n", "4"] + ids
    r = subprocess.run(cmd, cwd=ROOT, env=env, capture_output=True, text=True, timeout=1500)
    tail = (r.stdout + r.stderr)[-6000:]
    assert r.returncode == 0 and ("%d passed" % len(ids)) in tail, tail


def test_smoke_against_the_host_build(sim_library):
    """__graft_entry__.smoke(), the check that runs on the GPU box before the benchmark, line by line on the stand-in."""
    code = ("import sys; sys.path[:0] = [%r, %r]; import ophip; ophip.LIB_PATH = %r; import __graft_entry__; __graft_entry__.smoke()"
            % (ROOT, os.path.join(ROOT, "operators-rs_amd"), sim_library))
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0 and "smoke ok" in r.stdout, r.stdout + r.stderr


WEIGHT_TRAFFIC = """
import ctypes, sys
sys.path[:0] = [%r, %r]
import numpy as np
import ophip
ophip.LIB_PATH = %r
from ophip import TensorLayout, dt
gpu = ophip.Gpu(0)
stream = gpu.stream()
def counters():
    out = (ctypes.c_uint64 * 13)()
    ophip.lib().cpusim_counters(out)
    return np.array(list(out), dtype=np.int64)
for m, n, k in ((16, 4096, 4096), (16, 22016, 4096), (16, 4096, 11008), (7, 12288, 4096)):
    ad, bd, cd = gpu.malloc(m * k * 2), gpu.malloc(k * n * 2), gpu.malloc(m * n * 2)
    lay = lambda r, c: TensorLayout.new_contiguous(dt.F16, [1, r, c])
    op = ophip.MatMul(gpu)
    args = ophip.MatMulArgs(lay(m, n), cd, 0.0, lay(m, k), ad, lay(k, n), bd, 1.0)
    kernel = op.describe(args)
    before = counters()
    op.launch(args, None, stream)
    stream.synchronize()
    d = counters() - before
    print(m, n, k, kernel, "workgroups", d[1], "loads plain / nt / sc1", d[5:8], "stores", d[8:11], flush=True)
    assert kernel.startswith("stream"), kernel
    assert d[0] == 1 and d[2] == 0 and d[3] == 0                  # one launch, nothing past a resource
    assert d[6] == k * n * 2, (d[6], k * n * 2)                   # the weight, through the non-temporal loads: once
    strips = -(-n // 128)
    assert d[5] == strips * 16 * k * 2, (d[5], strips)            # a (16 rows, the ones past m read as zeros) once per strip
    assert d[7] == d[10] and d[8] == 0 and d[9] == 0              # what crosses workgroups is stored once and loaded once
    assert d[10] <= 2 * 16 * n * 4 * 8                            # ... and is small beside the weight
print("ok")
"""


def test_streaming_product_asks_for_every_weight_byte_once(sim_library):
    """The stand-in counts the bytes that kernels move through buffer resources, by cache policy.  For the decode layer's
    weight products on gemm_stream_m1 with the planner's cut (even and uneven): the weight goes through the non-temporal
    loads, each byte exactly once per launch; the activations once per strip of 128 columns (from the caches); the
    partial sums that cross workgroups are written once and read once.  No counter of the machine, but what the kernel
    asks of it: a re-read of the weight would have to come from here."""
    code = WEIGHT_TRAFFIC % (ROOT, os.path.join(ROOT, "operators-rs_amd"), sim_library)
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stdout + r.stderr[-3000:]


NO_ALLOCATION = """
import ctypes, sys
sys.path[:0] = [%r, %r, %r]
import numpy as np
import ophip
ophip.LIB_PATH = %r
from ophip import TensorLayout
from helpers import normal_f16
gpu = ophip.Gpu(0)
stream = gpu.stream()
def counters():
    out = (ctypes.c_uint64 * 13)()
    ophip.lib().cpusim_counters(out)
    return np.array(list(out), dtype=np.int64)
before = counters()
probe = gpu.malloc(64)
assert counters()[11] == before[11] + 1  # (the counters are alive)
probe.free()
assert counters()[12] == before[12] + 1
op = ophip.MatMul(gpu)
rng = np.random.default_rng(0)
kinds = set()
# split K in the streaming kernel (counters and partial sums), in a skinny kernel ([N, K] operand), in the tile kernel
# (partial tiles and a reduce kernel), batched with counters per batch; two products that use no scratch
for m, n, k, batch, b_nk in ((16, 4096, 4096, None, False), (16, 1024, 4096, None, True), (256, 512, 4096, None, True),
                             (16, 128, 2048, 8, False), (40, 2048, 512, None, False), (7, 24, 40, None, False)):
    lead = () if batch is None else (batch,)
    a, c = normal_f16(rng, lead + (m, k)), normal_f16(rng, lead + (m, n))
    b = normal_f16(rng, lead + ((n, k) if b_nk else (k, n)), std=0.05)
    b_view = np.swapaxes(b, -1, -2) if b_nk else b
    ad, bd, c1, c2 = gpu.from_host(a), gpu.from_host(b), gpu.from_host(c), gpu.from_host(c)
    args = lambda cd: ophip.MatMulArgs(TensorLayout.of(c), cd, 0.5, TensorLayout.of(a), ad, TensorLayout.of(b_view), bd, 0.25)
    static_args, kind = args(c2), op.describe(args(c2))
    op.launch(args(c1), None, stream)
    stream.synchronize()
    before = counters()
    op.launch_static(static_args, stream)
    op.launch_static(static_args, stream)
    stream.synchronize()
    d = counters() - before
    print(m, n, k, batch, kind, "launches", d[0], "allocations", d[11], "frees", d[12], flush=True)
    assert d[0] >= 2 and d[11] == 0 and d[12] == 0 and d[4] == 0, d
    kinds.add(kind.split()[0] + (" split" if "split_k=1" not in kind else ""))
    op.launch_static(args(c1), stream)  # (c1 holds one product already: beta = 0.5 makes this the second for both)
    one, two = (gpu.to_host(x, np.float16, c.size, stream=stream).view(np.uint16) for x in (c1, c2))
    assert np.array_equal(one, two), kind
assert {"stream split", "skinny split", "tile128x64 split", "skinny", "tile128x64"} <= kinds, kinds
print("ok")
"""


def test_static_entry_point_reaches_no_allocator(sim_library):
    """ophip_mat_mul_launch_static on the stand-in, whose allocator counts its calls: between the first and the last of
    its launches, for products that split K in each kernel family and for products that do not, no allocation is made
    and none is freed (the ordinary entry point, on a fresh operator and stream, makes several)."""
    code = NO_ALLOCATION % (ROOT, os.path.join(ROOT, "operators-rs_amd"), os.path.join(ROOT, "tests"), sim_library)
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stdout + r.stderr[-3000:]


def test_c_consumer_against_the_host_build(sim_library, tmp_path):
    """tests/c_abi/consumer.c (the ABI used from C11 as a binding of another language would use it: create, scheme,
    launch, compare with plain C) linked against the host build instead of libophip.so."""
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    exe, libdir = str(tmp_path / "consumer"), os.path.dirname(sim_library)
    cmd = [cc, "-std=c11", "-O1", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "c_abi", "consumer.c"), "-o", exe, "-L", libdir, "-lophip_cpusim", "-lm", "-Wl,-rpath," + libdir]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    res = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0 and res.stdout.strip().endswith("ok"), (res.returncode, res.stdout, res.stderr)


def build_threads_driver(library, exe, extra=()):
    sys.path.insert(0, SIM)
    try:
        import build_sim
    finally:
        sys.path.remove(SIM)
    libdir = os.path.dirname(library)
    cmd = [build_sim.compiler(), "-std=c++17", "-O1", "-g", "-pthread", "-I", os.path.join(ROOT, "include"), os.path.join(SIM, "threads_driver.cpp"),
           "-o", exe, "-L", libdir, "-lophip_cpusim", "-Wl,-rpath," + libdir] + list(extra)
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_one_device_and_its_operators_shared_by_several_threads(sim_library, tmp_path):
    """tests/cpu_sim/threads_driver.cpp: four threads launch through one device, one rms_norm and one mat_mul operator,
    each on a stream of its own, while operators and streams come and go; every result equals the single-threaded one."""
    exe = str(tmp_path / "threads_driver")
    build_threads_driver(sim_library, exe)
    res = subprocess.run([exe, "4", "8"], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0 and res.stdout.strip().endswith("ok"), (res.returncode, res.stdout, res.stderr)


@pytest.mark.skipif(not os.environ.get("OPHIP_TEST_SANITIZERS"), reason="three more builds of the stand-in, minutes each: set OPHIP_TEST_SANITIZERS=1")
def test_under_thread_address_and_undefined_behaviour_sanitizers(tmp_path):
    """The same threaded program against a ThreadSanitizer build of the stand-in and of the library's host sources (a
    data race in the host side ends the run), against an AddressSanitizer build with leak detection, and the smoke check
    against an UndefinedBehaviorSanitizer build (which python can load: it needs no preloading).  The builds are kept
    under tests/cpu_sim/_build_*."""
    sys.path.insert(0, SIM)
    try:
        import build_sim
    finally:
        sys.path.remove(SIM)
    tsan = build_sim.build(os.path.join(SIM, "_build_thread"), sanitize="thread")
    exe = str(tmp_path / "threads_driver_tsan")
    runtime = os.path.dirname(subprocess.run([build_sim.compiler(), "-print-file-name=libclang_rt.tsan-x86_64.so"], capture_output=True, text=True).stdout.strip())
    build_threads_driver(tsan, exe, ["-fsanitize=thread", "-shared-libsan", "-Wl,-rpath," + runtime])
    res = subprocess.run([exe, "6", "8"], capture_output=True, text=True, timeout=1200)
    assert res.returncode == 0 and res.stdout.strip().endswith("ok") and "ThreadSanitizer" not in res.stderr, (res.returncode, res.stdout, res.stderr[-4000:])
    # the same program under AddressSanitizer with leak detection: heap errors in the host side, and operators, streams
    # and devices that do not give back what they took
    asan = build_sim.build(os.path.join(SIM, "_build_address"), sanitize="address")
    exe = str(tmp_path / "threads_driver_asan")
    build_threads_driver(asan, exe, ["-fsanitize=address", "-shared-libsan", "-Wl,-rpath," + runtime])
    # ("large": the driver's sweep over mat_mul's kernel families then reaches the 256 x 256 tile as well)
    res = subprocess.run([exe, "3", "4", "large"], capture_output=True, text=True, timeout=2400, env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1"))
    assert res.returncode == 0 and res.stdout.strip().endswith("ok") and "AddressSanitizer" not in res.stderr, (res.returncode, res.stdout, res.stderr[-4000:])
    ubsan = build_sim.build(os.path.join(SIM, "_build_undefined"), sanitize="undefined")
    code = ("import sys; sys.path[:0] = [%r, %r]; import ophip; ophip.LIB_PATH = %r; import __graft_entry__; __graft_entry__.smoke()"
            % (ROOT, os.path.join(ROOT, "operators-rs_amd"), ubsan))
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0 and "smoke ok" in r.stdout, r.stdout + r.stderr
