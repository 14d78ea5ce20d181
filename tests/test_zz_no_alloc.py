"""ophip_mat_mul_launch_static: the mat_mul entry point that allocates nothing (its split-K scratch is a device
array inside the library) gives the bits of ophip_mat_mul_launch, call after call on the shared array."""
import numpy as np
import pytest

import ophip
from ophip import TensorLayout
from helpers import normal_f16

pytestmark = pytest.mark.gpu
f16 = np.float16


def say(msg):
    print(msg, flush=True)


def both_ways(gpu, stream, op, m, n, k, batch=None, b_k_contiguous=False, seed=0):
    """One product through ophip_mat_mul_launch (workspace from the stream's allocator) and through
    ophip_mat_mul_launch_static, from the same device operands into two C buffers that start as the same NaNs-free
    random values (beta = 0.5, so both read C)."""
    rng = np.random.default_rng(seed)
    lead = () if batch is None else (batch,)
    a = normal_f16(rng, lead + (m, k))
    b = normal_f16(rng, lead + ((n, k) if b_k_contiguous else (k, n)), std=0.05)
    b_view = np.swapaxes(b, -1, -2) if b_k_contiguous else b
    c = normal_f16(rng, lead + (m, n))
    ad, bd = gpu.from_host(a), gpu.from_host(b)
    outs = []
    what = None
    for static in (False, True):
        cd = gpu.from_host(c)
        args = ophip.MatMulArgs(TensorLayout.of(c), cd, 0.5, TensorLayout.of(a), ad, TensorLayout.of(b_view), bd, 0.25)
        what = op.describe(args)
        if static:
            op.launch_static(args, stream)
        else:
            op.launch(args, None, stream)
        outs.append(gpu.to_host(cd, f16, c.size, stream=stream).reshape(c.shape))
    return outs[0], outs[1], what


def test_static_scratch_entry_point_matches_the_ordinary_one(gpu, stream):
    op = ophip.MatMul(gpu)
    # (m, n, k, batch, B stored [N, K]): the decode products that split K inside the streaming kernel (arrival
    # counters), each followed by a smaller one on the same array; a tile product that splits K (separate reduce
    # kernel); products without any scratch
    cases = [
        (16, 12288, 4096, None, False),  # split 2
        (16, 4096, 4096, None, False),   # split 8, smaller: partials and counters the call before left behind
        (16, 1024, 4096, None, False),
        (48, 4096, 11008, None, False),
        (16, 128, 2048, 32, False),      # PV of the decode layer: batched, counters per (strip, batch)
        (16, 4096, 4096, None, True),
        (512, 4096, 11008, None, False),  # tile kernel, split K
        (256, 512, 4096, None, True),
        (16, 22016, 4096, None, False),  # the strips on slow granule classes in two K ranges, the others whole
        (40, 22016, 4096, None, False),  # no split: no scratch used
        (16, 49152, 1024, None, False),  # more strips than CUs: the streaming kernel for 16 rows without any cut
        (7, 24, 40, None, False),        # generic kernel
    ]
    kinds = set()
    for i, (m, n, k, batch, bk) in enumerate(cases):
        say("static scratch case %d: %s x %s x %s batch %s B[N,K]=%s" % (i, m, n, k, batch, bk))
        plain, static, what = both_ways(gpu, stream, op, m, n, k, batch, bk, seed=i)
        say("  -> %s" % what)
        kinds.add(what.split()[0] + (" split" if "split_k=1" not in what.replace("split_k=1 (", "") and "split_k" in what else ""))
        assert not np.isnan(plain).any()
        assert np.array_equal(plain.view(np.uint16), static.view(np.uint16)), (i, what)
    assert {"stream split", "stream", "skinny split", "skinny"} <= kinds and any(w.startswith("tile") and w.endswith("split") for w in kinds), kinds


def test_static_scratch_entry_point_refuses_what_does_not_fit(gpu, stream, monkeypatch):
    """On a 256-CU device the planner's own splits stay within the array (split x tiles never exceeds what fills the
    CUs); a split forced through the sweep knob asks for more, and the entry point says no before anything runs."""
    monkeypatch.setenv("OPHIP_GEMM_TILE_SPLITK", "8")
    op = ophip.MatMul(gpu)  # the knob is read when an operator is created
    monkeypatch.delenv("OPHIP_GEMM_TILE_SPLITK")
    m, n, k = 512, 4096, 11008
    L = TensorLayout.new_contiguous
    args = ophip.MatMulArgs(L(ophip.dt.F16, [m, n]), None, 0.0, L(ophip.dt.F16, [m, k]), None,
                            L(ophip.dt.F16, [k, n]), None, 1.0)
    need = op.scheme(args, 2 ** 40)
    say("static scratch refusal: %d x %d x %d, %s, needs %d bytes" % (m, n, k, op.describe(args), need))
    assert need == 8 * m * n * 4 > 32 << 20
    with pytest.raises(ophip.LaunchError) as e:
        op.launch_static(args, stream)
    assert e.value.kind == "ArgsNotSupport" and "static" in str(e.value)


def test_static_scratch_entry_point_runs_while_a_stream_records(gpu, stream):
    """What defines the entry point: it allocates nothing.  A stream that is being recorded into a graph refuses
    allocations, so the split-K products that need scratch (streaming kernel with arrival counters, tile kernel with
    the separate sum, and a product without scratch) are recorded through the static entry point, replayed twice and
    compared with the ordinary entry point's bits."""
    rng = np.random.default_rng(5)
    op = ophip.MatMul(gpu)
    cases = [(16, 4096, 4096), (16, 12288, 4096), (512, 4096, 11008), (7, 24, 40)]
    prepared = []
    for m, n, k in cases:
        a, b, c = normal_f16(rng, (m, k)), normal_f16(rng, (k, n), std=0.05), normal_f16(rng, (m, n))
        ad, bd, cd = gpu.from_host(a), gpu.from_host(b), gpu.from_host(c)
        args = ophip.MatMulArgs(TensorLayout.of(c), cd, 0.5, TensorLayout.of(a), ad, TensorLayout.of(b), bd, 0.25)
        op.launch(args, None, stream)  # warms the operator; its result is what the replays must give
        want = gpu.to_host(cd, f16, c.size, stream=stream).copy()
        prepared.append((args, cd, c, want, op.describe(args)))
    say("static scratch under recording: " + "; ".join(p[4] for p in prepared))
    stream.begin_capture()
    for args, cd, c, want, what in prepared:
        op.launch_static(args, stream)
    graph = stream.end_capture()
    for rep in range(2):
        for args, cd, c, want, what in prepared:  # beta = 0.5 reads C: the original C goes back before every replay
            gpu.upload(cd, c, stream=stream)
        stream.synchronize()
        graph.launch(stream)
        for args, cd, c, want, what in prepared:
            got = gpu.to_host(cd, f16, c.size, stream=stream)
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), "replay %d: %s" % (rep, what)
    graph.destroy()
