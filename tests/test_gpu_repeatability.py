"""Launch after launch, the same inputs give the same bits, whatever the workspace held before.

Kernels whose workgroups or waves hand data to each other (split-K partial sums, the attention composite's
score matrix, the sampling kernels' candidate lists and flags) are launched repeatedly over a workspace filled
with 0xFF bytes (f16 / f32 NaNs): a handover that can be overtaken shows up as a launch that differs from the first.
The first launch of every case is covered by the parity tests of its operator."""
import numpy as np
import pytest

import ophip
from helpers import normal_f16
from ophip import TensorLayout, dt

pytestmark = pytest.mark.gpu

f16 = np.float16
LAUNCHES = 150


def repeat(gpu, stream, launch, out_mem, nbytes, ws, what):
    first = None
    for it in range(LAUNCHES):
        if ws is not None:
            gpu.memset(ws, 0xFF, stream=stream)
        launch()
        out = gpu.to_host(out_mem, np.uint8, nbytes, stream=stream)
        if first is None:
            first = out
        else:
            assert np.array_equal(out, first), "%s: launch %d differs from the first" % (what, it)
    return first


@pytest.mark.parametrize("bt,m,n,k,b_transposed", [
    (1, 512, 4096, 4096, False),   # tile kernel, split K, separate reduce kernel
    (1, 64, 4096, 4096, False),    # ragged tile build, split K 8
    (32, 16, 128, 2048, False),    # decode PV: the splits of one strip sit on different XCDs
    (1, 16, 1160, 2048, False),    # ragged last strip, splits on different XCDs
    (2, 40, 512, 1024, True),      # 64-row build, weight stored [N, K]
    (1, 16, 12288, 4096, False),   # low-register streaming kernel: two K ranges per strip, three on the slow granule classes
])
def test_mat_mul_repeats_bit_for_bit(gpu, stream, bt, m, n, k, b_transposed):
    rng = np.random.default_rng(bt + m + n + k)
    shape = lambda *s: (bt,) + s if bt > 1 else s
    a = normal_f16(rng, shape(m, k))
    bfull = normal_f16(rng, shape(n, k) if b_transposed else shape(k, n), std=0.05)
    b = bfull.swapaxes(-1, -2) if b_transposed else bfull
    c = np.zeros(shape(m, n), f16)
    ad, bd, cd = gpu.from_host(a), gpu.from_host(bfull), gpu.from_host(c)
    op = ophip.MatMul(gpu)
    args = ophip.MatMulArgs(TensorLayout.of(c), cd, 0.0, TensorLayout.of(a), ad, TensorLayout.of(b), bd, 1.0)
    need = op.scheme(args, 2 ** 40)
    ws = gpu.malloc(need) if need else None
    what = "mat_mul %s (%s)" % ((bt, m, n, k), op.describe(args))
    print(what, flush=True)
    out = repeat(gpu, stream, lambda: op.launch(args, ws, stream), cd, c.nbytes, ws, what)
    assert not np.isnan(out.view(f16)).any(), what


@pytest.mark.parametrize("nh,nkvh,seq,att,dh", [(32, 32, 16, 2048, 128), (8, 2, 200, 333, 64)])
def test_attention_repeats_bit_for_bit(gpu, stream, nh, nkvh, seq, att, dh):
    rng = np.random.default_rng(nh + seq + att)
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, att, dh)), normal_f16(rng, (nkvh, att, dh))
    o = np.zeros((nh, seq, dh), f16)
    qd, kd, vd, od = (gpu.from_host(x) for x in (q, k, v, o))
    lay = TensorLayout.of
    op = ophip.Attention(gpu)
    args = ophip.AttentionArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(o), od, 1)
    ws = gpu.malloc(op.scheme(args, 2 ** 40))
    what = "attention %s" % ((nh, nkvh, seq, att, dh),)
    print(what, flush=True)

    def launch():
        gpu.upload(qd, q, stream=stream)  # the operator leaves its result in q as well
        stream.synchronize()
        op.launch(args, ws, stream)

    out = repeat(gpu, stream, launch, od, o.nbytes, ws, what)
    assert not np.isnan(out.view(f16)).any(), what


@pytest.mark.parametrize("nh,nkvh,seq,dh,buf,pos", [(32, 32, 16, 128, 2048, 2032), (32, 4, 7, 64, 1500, 1017),
                                                    (64, 8, 1, 128, 8192, 8000)])
def test_attention_kv_cached_one_pass_repeats_bit_for_bit(gpu, stream, nh, nkvh, seq, dh, buf, pos):
    """The one-pass kernel hands every chunk's maximum, sum and partial output to a second launch through the
    workspace (8, 4 and 63 chunks here; the last case takes 128 keys per workgroup): the same bits every time, o and
    both caches, over a workspace of NaNs."""
    rng = np.random.default_rng(nh + buf + pos)
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, seq, dh)), normal_f16(rng, (nkvh, seq, dh))
    kc, vc = normal_f16(rng, (nkvh, buf, dh)), normal_f16(rng, (nkvh, buf, dh))
    o = np.zeros((nh, seq, dh), f16)
    qd, kd, vd, od, kcd, vcd = (gpu.from_host(x) for x in (q, k, v, o, kc, vc))
    lay = TensorLayout.of
    op = ophip.AttnKVCached(gpu)
    args = ophip.AttnKVCachedArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(o), od, lay(kc), kcd, lay(vc), vcd, 1, pos)
    ws = gpu.malloc(max(op.scheme(args, 2 ** 40), 16))
    what = "attention_kv_cached one pass %s" % ((nh, nkvh, seq, dh, buf, pos),)
    print(what, flush=True)

    def launch():
        gpu.upload(qd, q, stream=stream)  # the operator leaves its result in q as well
        stream.synchronize()
        op.launch(args, ws, stream)

    out = repeat(gpu, stream, launch, od, o.nbytes, ws, what)
    assert not np.isnan(out.view(f16)).any(), what
    k_after = gpu.to_host(kcd, f16, kc.size, stream=stream).reshape(kc.shape)
    assert np.array_equal(k_after[:, pos:pos + seq], k) and np.array_equal(k_after[:, :pos], kc[:, :pos])


@pytest.mark.parametrize("rows,n,top_k,top_p", [(16, 32000, 50, 0.9), (4, 128256, 50, 0.9), (4, 32000, 2000, 0.95),
                                                (2, 50000, 2 ** 62, 0.9)])
def test_random_sample_repeats_bit_for_bit(gpu, stream, rows, n, top_k, top_p):
    rng = np.random.default_rng(rows + n)
    x = normal_f16(rng, (rows, n), std=2.0)
    xd = gpu.from_host(x)
    kv = gpu.malloc(rows * 8)
    L = TensorLayout
    op = ophip.RandomSample(gpu)
    args = ophip.RandomSampleArgs(L(dt.KVPAIR, [], []), kv, L(dt.F16, [n], [2]), xd, L(dt.U32, [n], [4]), None,
                                  ophip.SampleArgs(0.8, top_p, top_k), 0.37)
    ws = gpu.malloc(max(op.scheme(args, 2 ** 40), 16) * rows + 4096)
    what = "random_sample %s" % ((rows, n, top_k, top_p),)
    print(what, flush=True)
    out = repeat(gpu, stream, lambda: op.launch_batch(args, rows, n * 2, None, ws, stream), kv, rows * 8, ws, what)
    idx = out.view(np.uint32).reshape(rows, 2)[:, 0]
    assert (idx < n).all(), what
