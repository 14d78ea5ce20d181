"""The C ABI used from C: tests/c_abi/consumer.c includes include/ophip.h as C11, links against libophip.so and goes
through create / scheme / launch for rms_norm and mat_mul the way a binding of another language would (the reference's
side of the boundary is Rust FFI over the same header, operators-rs_amd/rust_shim).  Without a GPU the program has to
build, load the library and report that there is no device; on a GPU it checks the results against plain C."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "operators-rs_amd", "ophip")


def build(tmp_path):
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    exe = str(tmp_path / "consumer")
    rocm_lib = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")
    cmd = [cc, "-std=c11", "-O1", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "c_abi", "consumer.c"), "-o", exe, "-L", LIBDIR, "-lophip", "-lm",
           "-Wl,-rpath," + LIBDIR, "-Wl,-rpath-link," + rocm_lib, "-Wl,-rpath," + rocm_lib]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    return exe


def test_c_consumer_builds_links_and_reports_a_missing_device(tmp_path):
    exe = build(tmp_path)
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="-1")
    res = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=120)
    assert res.returncode == 2 and "no device" in res.stdout, (res.returncode, res.stdout, res.stderr)


@pytest.mark.gpu
def test_c_consumer_runs_rms_norm_and_mat_mul(tmp_path):
    exe = build(tmp_path)
    print("running the C consumer", flush=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0 and res.stdout.strip().endswith("ok"), (res.returncode, res.stdout, res.stderr)
