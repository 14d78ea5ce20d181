"""bench_probe: the measurement kernels behind `bench.py --ceilings`, `--floors` and `--granules` (a library of their
own, bench_probes/libbenchprobe.so; no counterpart in the reference and no part of the operator library).
What they compute is checked where they compute something (write, copy, the clock ticks of granules); the read probes
and the MFMA loop only have to run; bad arguments are refused on the host, before any launch."""
import numpy as np
import pytest

import bench
import ophip

pytestmark = pytest.mark.gpu


def probe(gpu, stream, kind, dst, src, nbytes, iters=0, seed=1, blocks=64):
    bench.bench_probe(kind, dst, src, nbytes, iters, seed, blocks, stream)


def test_probe_write_and_copy_move_what_they_say(gpu, stream):
    n = 1 << 20
    rng = np.random.default_rng(0)
    host = rng.integers(0, 2 ** 32, n // 4, dtype=np.uint32)
    src, dst = gpu.from_host(host), gpu.malloc(n)
    print("probe write", flush=True)
    probe(gpu, stream, "write", dst, None, n, seed=0xA5A5A5A5)
    assert (gpu.to_host(dst, np.uint32, n // 4, stream=stream) == 0xA5A5A5A5).all()
    print("probe copy", flush=True)
    probe(gpu, stream, "copy", dst, src, n)
    assert np.array_equal(gpu.to_host(dst, np.uint32, n // 4, stream=stream), host)
    # a size that is no multiple of what a grid step covers: the tails of the loops
    odd = 16 * 100003
    big = gpu.from_host(rng.integers(0, 2 ** 32, odd // 4, dtype=np.uint32))
    out = gpu.malloc(odd)
    probe(gpu, stream, "copy", out, big, odd, blocks=7)
    assert np.array_equal(gpu.to_host(out, np.uint32, odd // 4, stream=stream), gpu.to_host(big, np.uint32, odd // 4, stream=stream))


@pytest.mark.parametrize("kind", ["read", "read_nt", "read16", "read_nt16"])
def test_read_probes_run_and_leave_memory_alone(gpu, stream, kind):
    n = 16 * 70001
    host = np.arange(n // 4, dtype=np.uint32)
    src, dst = gpu.from_host(host), gpu.from_host(np.zeros(4, np.uint32))
    print("probe", kind, flush=True)
    for blocks in (1, 5, 300):
        probe(gpu, stream, kind, dst, src, n, blocks=blocks)
    assert np.array_equal(gpu.to_host(src, np.uint32, n // 4, stream=stream), host)
    assert (gpu.to_host(dst, np.uint32, 4, stream=stream) == 0).all()


def test_strips_and_mfma_probes_run(gpu, stream):
    rows, cols = 512, 1000  # a last strip of 104 columns
    src = gpu.from_host(np.ones((rows, cols), np.float16))
    dst = gpu.malloc(4096)
    print("probe strips", flush=True)
    for ranges in (1, 2, 4, 16):
        probe(gpu, stream, "strips", dst, src, rows * cols * 2, iters=cols, seed=rows, blocks=ranges)
    print("probe granules", flush=True)
    ticks = gpu.from_host(np.zeros(9, np.uint32))
    probe(gpu, stream, "granules", ticks, src, rows * cols * 2, iters=cols, seed=rows, blocks=1)
    t = gpu.to_host(ticks, np.uint32, 9, stream=stream)
    assert (t[:8] > 0).all() and (t[:8] < 100000).all() and t[8] == 0, t  # 8 strips, each well under a millisecond
    print("probe mfma", flush=True)
    scratch = gpu.malloc(8 * 1024)
    probe(gpu, stream, "mfma", scratch, None, 0, iters=2, seed=12345, blocks=8)
    stream.synchronize()


def test_probe_refuses_bad_arguments(gpu, stream):
    buf = gpu.malloc(4096)
    cases = [("nonsense", buf, buf, 4096, 0, 1, 8), ("read", buf, None, 4096, 0, 1, 8), ("copy", None, buf, 4096, 0, 1, 8),
             ("write", buf, None, 4090, 0, 1, 8), ("read", buf, buf, 4096, 0, 1, 0),
             ("strips", buf, buf, 4096, 64, 64, 1),      # 64 x 64 f16 = 8192 bytes, more than the buffer
             ("strips", buf, buf, 4096, 32, 64, 4),      # 64 rows do not split into 4 ranges of whole 32-row groups
             ("strips", buf, buf, 4096, 4, 32, 1)]       # fewer than 8 columns
    for kind, dst, src, nbytes, iters, seed, blocks in cases:
        with pytest.raises(RuntimeError):
            probe(gpu, stream, kind, dst, src, nbytes, iters, seed, blocks)
