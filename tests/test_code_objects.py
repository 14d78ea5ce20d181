"""What the compiler made of the kernels, read from the library's own code objects (operators-rs_amd/csrc/build/*.hsaco):
the properties the design counts on and that a change of source or of compiler flags can lose without any test of
results noticing.

  * No kernel touches scratch memory (register spills) except the few listed here, and those not beyond what they use
    today; the MFMA kernels that do spill (the 256 x 256 tile, at the limit of 512 registers) do so outside their main
    loops: no scratch instruction between the first and the last v_mfma of their code.
  * gemm_stream_m1 fits four waves per SIMD (at most 128 registers): its design is residency.
  * Every kernel's static LDS fits a CU (160 KiB), and what is launched with 256 work-items was compiled for 256.
Needs the code objects (make -C operators-rs_amd/csrc) and LLVM's readelf / objdump from the ROCm tree; skipped without.
"""
import glob
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "operators-rs_amd", "csrc", "build")
LLVM = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib", "llvm", "bin")

# kernel name (f16 or f32 build; `_bf16` names follow their f16 twin) -> bytes of scratch per work-item it may use
MAY_SPILL = {
    "softmax_f16_v8_p8_g1024": 128, "softmax_bf16_v8_p8_g1024": 128,           # 1024 work-items share 128 registers each
    "gemm_tile_256x256r_p1_q1": 16, "gemm_tile_256x256_p1_q0": 400, "gemm_tile_256x256r_p1_q0": 400,
    "gemm_tile_256x256_p0_q0": 400, "gemm_tile_256x256r_p0_q0": 400,           # epilogue addresses of a kernel at 512 registers
    "sample_topk_k64_f16": 16, "sample_topk_k64_f32": 48, "sample_topk_f16": 16, "sample_topk_f32": 80,
    "sample_topk_list_f16": 16, "sample_topk_list_f32": 16,
}


def modules():
    text = open(os.path.join(ROOT, "operators-rs_amd", "csrc", "Makefile")).read().replace("\\\n", " ")
    return re.search(r"^KERNELS\s*:=\s*(.*)$", text, re.M).group(1).split()


@pytest.fixture(scope="module")
def kernels():
    readelf = os.path.join(LLVM, "llvm-readelf")
    files = [os.path.join(BUILD, m + ".hsaco") for m in modules()]
    if not os.path.exists(readelf) or not all(os.path.exists(f) for f in files):
        pytest.skip("code objects or llvm-readelf not here")
    out = {}
    for f in files:
        notes = subprocess.run([readelf, "--notes", f], capture_output=True, text=True, check=True).stdout
        rec = {}
        for line in notes.splitlines():
            m = re.match(r"\s+(-\s+)?\.(\w+):\s+(\S+)", line)
            if not m:
                continue
            if m.group(2) == "agpr_count" and m.group(1):  # the first key of a kernel's record
                rec = {"module": os.path.basename(f)[:-6]}
            rec[m.group(2)] = m.group(3)
            if m.group(2) == "name" and "vgpr_count" not in rec:
                out[m.group(3)] = rec
    assert len(out) > 300, len(out)
    return out


def test_scratch_memory_is_used_only_where_listed(kernels):
    bad = []
    for name, k in kernels.items():
        allowed = MAY_SPILL.get(name[:-5] if name.endswith("_bf16") and name not in MAY_SPILL else name, 0)
        if int(k["private_segment_fixed_size"]) > allowed:
            bad.append((name, k["private_segment_fixed_size"], allowed))
    assert not bad, bad


def test_stream_kernel_keeps_four_waves_per_simd(kernels):
    for name in ("gemm_stream_m1", "gemm_stream_m1_bf16"):
        k = kernels[name]
        assert int(k["vgpr_count"]) <= 128 and int(k["agpr_count"]) == 0 and int(k["private_segment_fixed_size"]) == 0, (name, k)
        assert int(k["group_segment_fixed_size"]) <= 40 << 10, (name, k)  # four workgroups' LDS fit a CU


def test_lds_and_workgroup_sizes(kernels):
    for name, k in kernels.items():
        assert int(k["group_segment_fixed_size"]) <= 160 << 10, (name, k["group_segment_fixed_size"])
        assert int(k["max_flat_workgroup_size"]) in (64, 128, 256, 512, 1024), (name, k["max_flat_workgroup_size"])
        assert int(k["wavefront_size"]) == 64, name


def test_mfma_kernels_do_not_spill_inside_their_main_loops():
    objdump = os.path.join(LLVM, "llvm-objdump")
    files = sorted(glob.glob(os.path.join(BUILD, "gemm*.hsaco")) + glob.glob(os.path.join(BUILD, "attention*.hsaco")))
    if not os.path.exists(objdump) or not files:
        pytest.skip("code objects or llvm-objdump not here")
    seen = 0
    for f in files:
        text = subprocess.run([objdump, "-d", "--mcpu=gfx950", f], capture_output=True, text=True, check=True).stdout
        for body in re.split(r"\n(?=[0-9a-f]{16} <)", text):
            m = re.match(r"[0-9a-f]{16} <(\w+)>", body)
            if not m:
                continue
            lines = body.splitlines()
            mfma = [i for i, l in enumerate(lines) if "v_mfma" in l]
            if not mfma:
                continue
            seen += 1
            inside = [l for l in lines[mfma[0]:mfma[-1]] if "scratch_" in l]
            assert not inside, (m.group(1), len(inside), inside[:3])
    assert seen > 60, seen
