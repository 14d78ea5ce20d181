"""The weight-streaming mat_mul kernel for up to 16 rows (gemm_stream) numbers its workgroups' (strip, K range) units
with one function that the host and the kernel both compile (operators-rs_amd/csrc/kernels/params.h).  Here it is
compiled for the CPU and every workgroup of a launch is walked through it: for hand-picked cuts, for what the planner
chooses on a list of shapes (read back through ophip_mat_mul_describe), and for cuts that must be refused."""
import os
import re
import shutil
import subprocess

import pytest

import ophip
from ophip import TensorLayout, dt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no C++ compiler")
    exe = str(tmp_path_factory.mktemp("units") / "stream_units")
    res = subprocess.run([cxx, "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-I",
                          os.path.join(ROOT, "operators-rs_amd", "csrc", "kernels"),
                          os.path.join(ROOT, "tests", "c_abi", "stream_units.cpp"), "-o", exe], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr

    def run(n, k, split_k, k_per_split, mask, split_slow):
        r = subprocess.run([exe] + [str(v) for v in (n, k, split_k, k_per_split, mask, split_slow)], capture_output=True, text=True)
        return r.returncode, r.stdout.strip()
    return run


def even_cut(k, split):
    steps = k // 32
    sps = -(-steps // split)
    return -(-steps // sps), sps * 32


@pytest.mark.parametrize("n,k,split,mask,slow", [
    (22016, 4096, 1, 0x22, 2), (12288, 4096, 2, 0, 0), (12288, 4096, 2, 0x22, 3), (12288, 4096, 2, 0x22, 4),
    (4096, 4096, 8, 0, 0), (4096, 11008, 8, 0x22, 11), (2056, 1024, 1, 0x22, 3), (1024, 64, 1, 0x22, 2), (136, 32, 1, 0xAA, 1),
    (8, 32, 1, 0, 0), (128256, 4096, 1, 0x22, 2), (36864, 1024, 2, 0, 0), (640, 11008, 1, 0xFF, 43)])
def test_every_unit_once_and_inside_k(checker, n, k, split, mask, slow):
    split, kps = even_cut(k, split)
    rc, out = checker(n, k, split, kps, mask, slow)
    assert rc == 0 and out.startswith("OK"), out


def test_a_cut_with_empty_ranges_is_caught(checker):
    """128 steps in 24 ranges of 6: ranges 22 and 23 would start past K.  The planner never emits such a cut (it rounds
    the count to ceil(steps / ceil(steps / n))); the kernel treats such a range as empty; this check names it."""
    rc, out = checker(12288, 4096, 2, 2048, 0x22, 24)
    assert rc != 0 and "FAIL" in out, out
    rc, out = checker(12288, 4096, 24, 192, 0, 0)
    assert rc != 0 and "FAIL" in out, out


SHAPES = [(16, 22016, 4096), (16, 12288, 4096), (16, 4096, 4096), (16, 4096, 11008), (1, 32000, 4096), (8, 128256, 4096),
          (16, 36864, 1024), (16, 40960, 5120), (3, 1000 * 8, 2048), (16, 128, 2048), (16, 1024, 32), (16, 1024, 64),
          (5, 2056, 1024), (16, 11008, 4096), (16, 14336, 4096), (16, 28672, 4096), (16, 8192, 8192), (16, 57344, 8192)]


@pytest.mark.parametrize("slow_knob", [None, "0", "2", "3", "5", "64"])
def test_what_the_planner_chooses_numbers_its_units_soundly(checker, monkeypatch, slow_knob):
    if slow_knob is not None:
        monkeypatch.setenv("OPHIP_GEMM_SLOW_SPLIT", slow_knob)
    c = lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    streamed = 0
    for m, n, k in SHAPES:
        args = ophip.MatMulArgs(c(m, n), None, 0.0, c(m, k), None, c(k, n), None, 1.0)
        what = ophip.mat_mul_describe(args)  # no operator: the plan for 256 compute units
        if not what.startswith("stream"):
            continue
        streamed += 1
        g = re.match(r"stream rows<=16 qN split_k=(\d+)(?: \((\d+) on granule classes 0x([0-9a-f]+)\))?$", what)
        assert g, what
        split = int(g.group(1))
        slow, mask = (int(g.group(2)), int(g.group(3), 16)) if g.group(2) else (0, 0)
        cut, kps = even_cut(k, split)
        assert cut == split, (what, cut)
        rc, out = checker(n, k, split, kps, mask, slow)
        assert rc == 0 and out.startswith("OK"), (m, n, k, what, out)
    assert streamed >= 10


def test_the_planner_on_the_decode_layers_products():
    """What launch() picks for the six GEMMs of the benchmark's decode layer (16 tokens, Llama-7B shapes) and their
    32- / 48-row siblings, on a device of 256 compute units: the 16-row products against N-contiguous weights on the
    low-register streaming kernel, about one workgroup per CU, gate/up with its slow strips in two K ranges."""
    import numpy as np

    f16 = np.float16
    want = {("qkv", 1, 16, 12288, 4096, False): "stream rows<=16 qN split_k=2",
            ("o_proj", 1, 16, 4096, 4096, False): "stream rows<=16 qN split_k=8",
            ("gate_up", 1, 16, 22016, 4096, False): "stream rows<=16 qN split_k=1 (2 on granule classes 0x22)",
            ("down", 1, 16, 4096, 11008, False): "stream rows<=16 qN split_k=8",
            ("qk_t", 32, 16, 2048, 128, True): "skinny rows<=16 qK split_k=1",
            ("pv", 32, 16, 128, 2048, False): "stream rows<=16 qN split_k=4",
            ("qkv_32_rows", 1, 32, 12288, 4096, False): "skinny rows<=32 qN paired split_k=2",
            ("gate_up_48_rows", 1, 48, 22016, 4096, False): "skinny rows<=64 qN paired split_k=1",
            ("ragged_k", 1, 7, 24, 40, False): "skinny rows<=16 qN split_k=1"}
    for (name, bt, m, n, k, b_transposed), text in want.items():
        shape = lambda *s: (bt,) + s if bt > 1 else s
        a, c = np.zeros(shape(m, k), f16), np.zeros(shape(m, n), f16)
        bfull = np.zeros(shape(n, k) if b_transposed else shape(k, n), f16)
        b = bfull.swapaxes(-1, -2) if b_transposed else bfull
        args = ophip.MatMulArgs(TensorLayout.of(c), None, 0.0, TensorLayout.of(a), None, TensorLayout.of(b), None, 1.0)
        assert ophip.mat_mul_describe(args) == text, (name, ophip.mat_mul_describe(args))


def test_the_uneven_cut_needs_strips_that_stay_in_their_granule_class():
    """The slow strips are cut finer only where a strip does stay in one class (or alternates c, c + 4): a weight whose
    first strip starts on a 256-byte boundary and whose rows are whole KiB apart.  Anything else gets the even cut."""
    import numpy as np

    f16 = np.float16
    m, n, k = 16, 22016, 4096

    def what(b_base, row_elems):
        c, a = np.zeros((m, n), f16), np.zeros((m, k), f16)
        b_layout = TensorLayout(dt.F16, [k, n], [row_elems * 2, 2])
        return ophip.mat_mul_describe(ophip.MatMulArgs(TensorLayout.of(c), None, 0.0, TensorLayout.of(a), None, b_layout, b_base, 1.0))

    cut = "stream rows<=16 qN split_k=1 (2 on granule classes 0x22)"
    even = "stream rows<=16 qN split_k=1"
    assert what(0x7f0000000000, n) == cut
    assert what(0x7f0000000000 + 5 * 256, n) == cut          # any granule, as long as it is a whole one
    assert what(0x7f0000000000 + 128, n) == even             # strips straddle two granules: one odd, one even, always
    assert what(0x7f0000000000, n + 128) == even             # rows of 172.5 KiB quarters: classes rotate from row to row
    assert what(0x7f0000000000, n + 512) == cut              # rows of 44 KiB
    assert what(0x7f0000000000, n + 8) == even
