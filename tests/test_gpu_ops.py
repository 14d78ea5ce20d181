"""Parity of the HIP backend with the CPU oracle, through the C ABI, on a real MI355X.

Shapes follow the reference's own device tests (cited per test) and the
benchmark configurations.  Bars: rearrange bytes and sampled indices are exact;
f16 outputs are within max-abs 2e-3 / rel 1e-2 of the oracle AND satisfy the
reference's ErrorCollector rule; mat_mul is within rel 1e-2 at K = 4096."""
import numpy as np
import pytest

import ophip
import oracle
from helpers import assert_close_f16, normal_f16
from ophip import TensorLayout, dt

pytestmark = pytest.mark.gpu

f16, f32 = np.float16, np.float32


def say(msg):
    print(msg, flush=True)


class DevBuf:
    """A host byte buffer mirrored on the device; numpy views with byte strides on the host side."""

    def __init__(self, gpu, host):
        self.gpu = gpu
        self.host = np.ascontiguousarray(host).view(np.uint8).reshape(-1).copy()
        self.mem = gpu.from_host(self.host)

    @property
    def ptr(self):
        return self.mem.ptr

    def download(self, stream):
        return self.gpu.to_host(self.mem, np.uint8, self.host.size, stream=stream)


def view_of(buf_u8, dtype, shape, strides, offset=0):
    base = np.frombuffer(buf_u8, dtype=np.uint8)
    return np.lib.stride_tricks.as_strided(base[offset:].view(dtype), shape=shape, strides=strides, writeable=True)


# ------------------------------------------------------------- rms_norm ----

def run_rms_norm(gpu, stream, x, w, eps, y_strides=None):
    n, d = x.shape
    xd, wd = gpu.from_host(x), gpu.from_host(w)
    y = np.zeros_like(x)
    yd = gpu.from_host(y)
    op = ophip.RmsNorm(gpu)
    args = ophip.RmsNormArgs(TensorLayout.of(y), yd, TensorLayout.of(x), xd, TensorLayout.of(w), wd, eps)
    op.scheme(args, 0)
    op.launch(args, None, stream)
    return gpu.to_host(yd, x.dtype, n * d, stream=stream).reshape(n, d)


def test_rms_norm_benchmark_shape(gpu, stream):
    rng = np.random.default_rng(0)
    x = normal_f16(rng, (64, 4096))
    w = rng.uniform(0.5, 1.5, 4096).astype(f32).astype(f16)
    say("rms_norm f16 [64,4096] seed 0")
    y = run_rms_norm(gpu, stream, x, w, 1e-5)
    ref = oracle.rms_norm(np.empty_like(x), x, w, 1e-5)
    assert_close_f16(y, ref, "rms_norm 64x4096")


@pytest.mark.parametrize("k", range(8, 14))
def test_rms_norm_reference_sweep_f32_weights(gpu, stream, k):
    """rms_norm/cuda/mod.rs:286-377: n = 4, d = 2^8 .. 2^13, w f32, a f16, inputs U[0,1)."""
    rng = np.random.default_rng(k)
    d = 1 << k
    x = rng.random((4, d)).astype(f16)
    w = rng.random(d).astype(f32)
    say("rms_norm sweep d=%d" % d)
    y = run_rms_norm(gpu, stream, x, w, 1e-5)
    ref = oracle.rms_norm(np.empty_like(x), x, w, 1e-5)
    assert_close_f16(y, ref, "rms_norm d=%d" % d)
    ref64 = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(1, keepdims=True) + 1e-5) * w
    assert_close_f16(y, ref64, "rms_norm vs f64 d=%d" % d)


@pytest.mark.parametrize("n,d,dta,dtw", [(4096, 4096, f16, f16), (3, 16384, f16, f16), (5, 80000, f16, f32),
                                          (7, 1000, f16, f16), (9, 4095, f16, f32), (300, 4096, f32, f32),
                                          (2, 130, f32, f32), (1, 8, f16, f16), (33, 2048, f16, f16),
                                          (20001, 1024, f16, f16), (17000, 1024, f16, f32),  # these two: one wave streaming many rows
                                          (16500, 512, f16, f16), (16499, 768, f16, f32), (16387, 1600, f16, f16), (16390, 2048, f16, f16),  # 8 / 4 / 2 / 2 rows per trip
                                          (8200, 5120, f16, f16), (8193, 8192, f16, f16), (8200, 4104, f16, f16),  # the same, 16 vectors a lane
                                          (8200, 5120, f16, f32),  # (f32 weights: a workgroup per row)
                                          (5, 4096, np.float64, np.float64), (64, 333, np.float64, np.float64)])
def test_rms_norm_shapes_and_types(gpu, stream, n, d, dta, dtw):
    rng = np.random.default_rng(n * 131 + d)
    x = rng.standard_normal((n, d)).astype(f32).astype(dta)
    w = rng.uniform(0.5, 1.5, d).astype(dtw)
    say("rms_norm n=%d d=%d %s/%s" % (n, d, dta.__name__, dtw.__name__))
    y = run_rms_norm(gpu, stream, x, w, 1e-5)
    ref = oracle.rms_norm(np.empty_like(x), x, w, 1e-5)
    if dta is f16:
        assert_close_f16(y, ref, "rms_norm")
    elif dta is f32:
        np.testing.assert_allclose(y, ref, rtol=2e-5, atol=1e-6)
    else:  # f64: the row sum is a parallel f64 sum here and a sequential one in the reference
        np.testing.assert_allclose(y, ref, rtol=1e-13, atol=0)


def test_rms_norm_strided_rows(gpu, stream):
    rng = np.random.default_rng(5)
    n, d, ld = 16, 4096, 12288
    xbuf = DevBuf(gpu, normal_f16(rng, (n, ld)))
    ybuf = DevBuf(gpu, np.zeros((n, ld + 64), f16))
    w = rng.uniform(0.5, 1.5, d).astype(f16)
    wd = gpu.from_host(w)
    xv = view_of(xbuf.host, f16, (n, d), (ld * 2, 2), offset=4096 * 2)
    op = ophip.RmsNorm(gpu)
    args = ophip.RmsNormArgs(TensorLayout(dt.F16, [n, d], [(ld + 64) * 2, 2]), ybuf.ptr + 64,
                             TensorLayout(dt.F16, [n, d], [ld * 2, 2]), xbuf.ptr + 4096 * 2,
                             TensorLayout.of(w), wd, 1e-5)
    say("rms_norm strided rows")
    op.launch(args, None, stream)
    out = ybuf.download(stream)
    yv = view_of(out, f16, (n, d), ((ld + 64) * 2, 2), offset=64)
    ref = oracle.rms_norm(np.empty((n, d), f16), xv, w, 1e-5)
    assert_close_f16(yv, ref, "rms_norm strided")
    mask = np.ones(out.size, bool)
    idx = (np.arange(n)[:, None] * (ld + 64) * 2 + 64 + np.arange(d * 2)[None, :]).ravel()
    mask[idx] = False
    assert (out[mask] == 0).all()  # nothing outside the view was written


def test_rms_norm_errors(gpu, stream):
    op = ophip.RmsNorm(gpu)
    L = TensorLayout
    mk = lambda y, x, w, **kw: ophip.RmsNormArgs(y, None, x, None, w, None, 1e-5)
    good = L(dt.F16, [4, 256], [512, 2])
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(mk(L(dt.F16, [4, 256, 1], [512, 2, 2]), good, L(dt.F16, [256], [2])), 0)
    assert e.value.kind == "RankNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(mk(good, L(dt.F32, [4, 256], [1024, 4]), L(dt.F16, [256], [2])), 0)
    assert e.value.kind == "TypeMismatch"
    # f64 mixed with a narrower type and non-floating types (every pairing of f16 / bf16 / f32 has a kernel, tests/test_gpu_bf16.py):
    # refused by scheme and launch alike
    for dta, dtw in [(dt.F16, dt.F64), (dt.F64, dt.F32), (dt.F64, dt.BF16), (dt.U32, dt.U32), (dt.F16, dt.I32)]:
        na, nw = ophip.dtype_nbytes(dta), ophip.dtype_nbytes(dtw)
        a = mk(L(dta, [4, 256], [256 * na, na]), L(dta, [4, 256], [256 * na, na]), L(dtw, [256], [nw]))
        with pytest.raises(ophip.SchemeError) as e:
            op.scheme(a, 0)
        assert e.value.kind == "TypeNotSupport"
        with pytest.raises(ophip.LaunchError) as e:
            op.launch(a, None, stream)
        assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(mk(good, good, L(dt.F16, [128], [2])), 0)
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(mk(L(dt.F16, [None, None], [None, None]), L(dt.F16, [None, None], [None, None]),
                     L(dt.F16, [None], [None])), 0)
    assert e.value.kind == "DynamicNotSupport"
    # dynamic n and strides are fine at scheme time (rms_norm/cuda/mod.rs:229-241), not at launch
    dyn = mk(L(dt.F16, [None, 256], [None, None]), L(dt.F16, [None, 256], [None, None]), L(dt.F32, [256], [None]))
    assert op.scheme(dyn, 0) == 0
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(dyn, None, stream)
    assert e.value.kind == "DynamicNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(mk(good, L(dt.F16, [4, 256], [1024, 4]), L(dt.F16, [256], [2])), None, stream)
    assert e.value.kind == "StridesNotSupport"


# ----------------------------------------------------------------- rope ----

def rope_args(t_layout, t_base, p_layout, p_base, dh, theta):
    empty = TensorLayout(dt.F16, [0, dh], [2 * dh, 2])  # the reference tests pass shape [0, dh] and null bases
    return ophip.RopeArgs(t_layout, t_base, p_layout, p_base, empty, None, empty, None, theta)


def run_rope(gpu, stream, t, pos, theta=1e4):
    td, pd = gpu.from_host(t), gpu.from_host(pos)
    op = ophip.Rope(gpu)
    args = rope_args(TensorLayout.of(t), td, TensorLayout.of(pos), pd, t.shape[2], theta)
    op.scheme(args, 0)
    op.launch(args, None, stream)
    return gpu.to_host(td, t.dtype, t.size, stream=stream).reshape(t.shape)


def test_rope_benchmark_shape(gpu, stream):
    rng = np.random.default_rng(0)
    t = normal_f16(rng, (512, 32, 128))
    pos = np.arange(512, dtype=np.uint32)
    say("rope f16 [512,32,128]")
    out = run_rope(gpu, stream, t, pos)
    ref = oracle.rope(t.copy(), pos, 1e4)
    assert_close_f16(out, ref, "rope 512x32x128")
    assert np.array_equal(out[0].view(np.uint16), t[0].view(np.uint16))  # pos 0 leaves the token untouched


@pytest.mark.parametrize("pdt", [np.uint32, np.uint64])
def test_rope_reference_shape(gpu, stream, pdt):
    """rope/cuda/mod.rs:257-346: nt = 7, nh = 32, dh = 64, pos = [0,1,2,3,7,8,1], inputs U[0,1)."""
    rng = np.random.default_rng(1)
    t = rng.random((7, 32, 64)).astype(f16)
    pos = np.array([0, 1, 2, 3, 7, 8, 1], pdt)
    say("rope reference shape %s" % pdt.__name__)
    out = run_rope(gpu, stream, t, pos)
    assert_close_f16(out, oracle.rope(t.copy(), pos, 1e4), "rope ref shape")


@pytest.mark.parametrize("shape,dtype", [((16, 32, 128), f16), ((3, 5, 20), f16), ((2, 1, 2), f16),
                                         ((5, 7, 64), f32), ((1, 40, 256), f16), ((100, 8, 96), f16),
                                         ((4099, 8, 128), f16), ((4101, 16, 128), f16), ((4097, 16, 64), f16)])  # several tokens per workgroup
def test_rope_shapes(gpu, stream, shape, dtype):
    rng = np.random.default_rng(sum(shape))
    t = rng.standard_normal(shape).astype(f32).astype(dtype)
    pos = rng.integers(0, 4096, shape[0]).astype(np.uint32)
    say("rope %s %s" % (shape, dtype.__name__))
    out = run_rope(gpu, stream, t, pos)
    ref = oracle.rope(t.copy(), pos, 1e4)
    if dtype is f16:
        assert_close_f16(out, ref, "rope %s" % (shape,))
    else:
        np.testing.assert_allclose(out, ref, rtol=0, atol=5e-3)  # f32 angles near 4096 rad carry ~ang * 2^-23 of error


def test_rope_gives_a_token_the_same_bits_whatever_the_call_holds(gpu, stream):
    """The host picks another kernel from 4096 tokens on (several tokens per workgroup, one sine / cosine table each):
    the same tokens at the same positions must come out bit for bit the same on either side of that line, or a
    prefill cut into chunks would differ from one that is not."""
    rng = np.random.default_rng(77)
    for nh, dh in ((8, 128), (16, 64)):
        t = normal_f16(rng, (4200, nh, dh))
        pos = rng.integers(0, 100000, 4200).astype(np.uint32)
        say("rope: 4095 / 4096 / 4200 tokens of %d heads x %d" % (nh, dh))
        outs = [run_rope(gpu, stream, t[:n].copy(), pos[:n].copy()) for n in (4095, 4096, 4200)]
        single = run_rope(gpu, stream, t[:7].copy(), pos[:7].copy())
        assert np.array_equal(outs[0].view(np.uint16), outs[1][:4095].view(np.uint16))
        assert np.array_equal(outs[1].view(np.uint16), outs[2][:4096].view(np.uint16))
        assert np.array_equal(single.view(np.uint16), outs[2][:7].view(np.uint16))


def test_rope_q_and_k_views_inside_qkv(gpu, stream):
    """Decode layer: q and k are [16, 32, 128] views of one [16, 12288] QKV buffer."""
    rng = np.random.default_rng(2)
    nt, nh, dh = 16, 32, 128
    qkv = DevBuf(gpu, normal_f16(rng, (nt, 3 * nh * dh)))
    pos = (np.arange(nt) + 2032).astype(np.uint32)
    pd = gpu.from_host(pos)
    op = ophip.Rope(gpu)
    lay = TensorLayout(dt.F16, [nt, nh, dh], [3 * nh * dh * 2, dh * 2, 2])
    say("rope q/k views")
    for part in (0, 1):
        op.launch(rope_args(lay, qkv.ptr + part * nh * dh * 2, TensorLayout.of(pos), pd, dh, 1e4), None, stream)
    out = qkv.download(stream).view(f16).reshape(nt, 3 * nh * dh)
    ref = qkv.host.view(f16).reshape(nt, 3 * nh * dh).copy()
    for part in (0, 1):
        v = view_of(ref.view(np.uint8).reshape(-1), f16, (nt, nh, dh), (3 * nh * dh * 2, dh * 2, 2),
                    offset=part * nh * dh * 2)
        oracle.rope(v, pos, 1e4)
    assert_close_f16(out, ref, "rope qkv views")
    assert np.array_equal(out[:, 2 * nh * dh:], ref[:, 2 * nh * dh:])  # v untouched


def test_rope_build_pos_and_errors(gpu, stream):
    ptr = ophip.Rope.build_pos(dt.U32, 7, [(3, 4), (10, 2), (0, 5)], stream)
    got = gpu.to_host(ptr, np.uint32, 7, stream=stream)
    assert got.tolist() == [3, 4, 5, 6, 10, 11, 0]
    ptr64 = ophip.Rope.build_pos(dt.U64, 3, [(2 ** 33, 3)], stream)
    assert gpu.to_host(ptr64, np.uint64, 3, stream=stream).tolist() == [2 ** 33, 2 ** 33 + 1, 2 ** 33 + 2]
    nctx, _ = ophip.Rope.build_sincos(dt.F16, 4096, 128, stream)
    assert nctx == 0
    op = ophip.Rope(gpu)
    L = TensorLayout
    t = L(dt.F16, [4, 2, 16], [64, 32, 2])
    p = L(dt.U32, [4], [4])
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(rope_args(L(dt.U16, [4, 2, 16], [64, 32, 2]), None, p, None, 16, 1e4), 0)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(rope_args(t, None, L(dt.I32, [4], [4]), None, 16, 1e4), 0)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(rope_args(t, None, L(dt.U32, [5], [4]), None, 16, 1e4), 0)
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(rope_args(t, None, p, None, 32, 1e4), 0)  # sin/cos last dim must equal dh
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(rope_args(L(dt.F16, [4, 32], [64, 2]), None, p, None, 16, 1e4), 0)
    assert e.value.kind == "RankNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(rope_args(L(dt.F16, [4, 2, 16], [128, 64, 4]), None, p, None, 16, 1e4), None, stream)
    assert e.value.kind == "StridesNotSupport"


# -------------------------------------------------------- fused softmax ----

def run_softmax(gpu, stream, att, causal=True):
    ad = gpu.from_host(att)
    op = ophip.FusedSoftmax(gpu)
    args = ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL if causal else ophip.AttnMask.NONE, TensorLayout.of(att), ad)
    op.scheme(args, 0)
    op.launch(args, None, stream)
    return gpu.to_host(ad, att.dtype, att.size, stream=stream).reshape(att.shape)


def check_softmax(out, att, causal, what):
    ref = oracle.fused_softmax(att.copy(), causal=causal)
    assert_close_f16(out, ref, what)
    nh, seq, al = att.shape
    if causal:
        bits = out.view(np.uint16)
        for r in range(seq):
            assert (bits[:, r, al - seq + r + 1:] == 0).all(), "masked tail must be +0"


@pytest.mark.parametrize("shape", [(32, 512, 512), (32, 1, 2048), (32, 16, 2048)])
def test_softmax_benchmark_shapes(gpu, stream, shape):
    rng = np.random.default_rng(0)
    att = normal_f16(rng, shape, std=2.0)  # N(0, 4): variance 4
    say("softmax %s" % (shape,))
    oracle.set_threads(8)
    try:
        check_softmax(run_softmax(gpu, stream, att), att, True, "softmax %s" % (shape,))
    finally:
        oracle.set_threads(1)


@pytest.mark.parametrize("seq,al", [(1, 511), (1, 2048), (7, 511), (7, 2048)])
def test_softmax_reference_shapes(gpu, stream, seq, al):
    """fuesd_softmax/cuda/mod.rs:233-296: nh = 32, inputs U[0,1)."""
    rng = np.random.default_rng(seq * 10000 + al)
    att = rng.random((32, seq, al)).astype(f16)
    say("softmax reference shape seq=%d att=%d" % (seq, al))
    check_softmax(run_softmax(gpu, stream, att), att, True, "softmax ref")


@pytest.mark.parametrize("shape,causal", [((2, 3, 8), True), ((1, 1, 1), True), ((3, 5, 5), True),
                                          ((2, 4, 1000), False), ((2, 4, 4096), True), ((1, 3, 9000), True),
                                          ((1, 2, 16384), True), ((1, 2, 40000), True), ((1, 2, 70001), True),
                                          ((4, 300, 300), True), ((2, 2, 1023), False), ((1, 2, 5000), True),
                                          # many short rows, four to a wave: a row count that is no multiple of four, two
                                          # vectors per lane, more columns than rows, no mask, a single vector per row
                                          ((32, 257, 264), True), ((16, 514, 1024), True), ((16, 512, 1000), True),
                                          ((32, 256, 512), False), ((64, 130, 136), True), ((1100, 8, 8), True), ((33, 250, 256), True)])
def test_softmax_shapes(gpu, stream, shape, causal):
    rng = np.random.default_rng(sum(shape))
    att = normal_f16(rng, shape, std=2.0)
    say("softmax %s causal=%s" % (shape, causal))
    check_softmax(run_softmax(gpu, stream, att, causal), att, causal, "softmax %s" % (shape,))


def test_softmax_strided_heads(gpu, stream):
    rng = np.random.default_rng(9)
    nh, seq, al, ld = 4, 6, 256, 320
    buf = DevBuf(gpu, normal_f16(rng, (seq, nh, ld), std=2.0))  # heads interleaved: [seq, nh, ld]
    lay = TensorLayout(dt.F16, [nh, seq, al], [ld * 2, nh * ld * 2, 2])
    op = ophip.FusedSoftmax(gpu)
    say("softmax strided")
    op.launch(ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL, lay, buf.ptr), None, stream)
    out = buf.download(stream)
    ref = buf.host.copy()
    oracle.fused_softmax(view_of(ref, f16, (nh, seq, al), (ld * 2, nh * ld * 2, 2)), causal=True)
    assert_close_f16(out.view(f16), ref.view(f16), "softmax strided")


def test_softmax_errors(gpu, stream):
    op = ophip.FusedSoftmax(gpu)
    L = TensorLayout
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.FusedSoftmaxArgs(1, L(dt.F16, [4, 4], [8, 2]), None), 0)
    assert e.value.kind == "RankNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.FusedSoftmaxArgs(1, L(dt.U16, [1, 4, 4], [32, 8, 2]), None), 0)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.FusedSoftmaxArgs(1, L(dt.F16, [1, 4, 4], [64, 16, 4]), None), None, stream)
    assert e.value.kind == "StridesNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.FusedSoftmaxArgs(1, L(dt.F16, [1, None, 4], [32, 8, 2]), None), None, stream)
    assert e.value.kind == "DynamicNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.FusedSoftmaxArgs(1, L(dt.F16, [1, 8, 4], [64, 8, 2]), None), None, stream)
    assert e.value.kind == "ShapeNotSupport"


# ------------------------------------------------------------ rearrange ----

def run_rearrange(gpu, stream, dst_host, dst_view, src_host, src_view):
    """dst_view / src_view are numpy views into dst_host / src_host (uint8 buffers)."""
    sd, dd = gpu.from_host(src_host), gpu.from_host(dst_host)
    doff = dst_view.__array_interface__["data"][0] - dst_host.__array_interface__["data"][0]
    soff = src_view.__array_interface__["data"][0] - src_host.__array_interface__["data"][0]
    op = ophip.Rearrange(gpu)
    args = ophip.RearrangeArgs(TensorLayout.of(dst_view), dd.ptr + doff, TensorLayout.of(src_view), sd.ptr + soff)
    op.scheme(args, 0)
    op.launch(args, None, stream)
    return gpu.to_host(dd, np.uint8, dst_host.size, stream=stream)


def test_rearrange_benchmark_shape_is_bit_exact(gpu, stream):
    rng = np.random.default_rng(0)
    src = rng.integers(0, 65536, (32, 512, 128)).astype(np.uint16).view(f16)  # any bit pattern, NaNs included
    src_host = src.view(np.uint8).reshape(-1)
    dst_host = np.zeros(src_host.size, np.uint8)
    # destination: contiguous [512, 32, 128] viewed with the dims in the source's order
    dst_view = view_of(dst_host, f16, (32, 512, 128), (256, 8192, 2))
    say("rearrange [32,512,128] -> [512,32,128]")
    out = run_rearrange(gpu, stream, dst_host, dst_view, src_host, src)
    want = np.ascontiguousarray(src.transpose(1, 0, 2)).view(np.uint8).reshape(-1)
    assert np.array_equal(out, want)
    ref = np.zeros_like(dst_host)
    oracle.rearrange(view_of(ref, f16, (32, 512, 128), (256, 8192, 2)), src)
    assert np.array_equal(out, ref)


def test_rearrange_reference_shape(gpu, stream):
    """rearrange/cuda/mod.rs:252-325: u32 [32, 7, 128] into a transposed-contiguous [7, 32, 128]."""
    nh, seq, dh = 32, 7, 128
    src = np.arange(nh * seq * dh, dtype=np.uint32).reshape(nh, seq, dh)
    src_host = src.view(np.uint8).reshape(-1)
    dst_host = np.zeros(src_host.size, np.uint8)
    dst_view = view_of(dst_host, np.uint32, (nh, seq, dh), (dh * 4, nh * dh * 4, 4))
    say("rearrange reference shape")
    out = run_rearrange(gpu, stream, dst_host, dst_view, src_host, src)
    assert np.array_equal(out.view(np.uint32).reshape(seq, nh, dh), src.transpose(1, 0, 2))


def test_rearrange_random_layouts_bit_exact(gpu, stream):
    rng = np.random.default_rng(1)
    done = 0
    for trial in range(60):
        nd = int(rng.integers(1, 6))
        shape = [int(rng.integers(1, 9)) for _ in range(nd)]
        dtype = [np.uint8, np.uint16, np.uint32, np.uint64][int(rng.integers(0, 4))]
        es = np.dtype(dtype).itemsize

        def make(full_fill):
            full_shape = [2 * s + 1 for s in shape]
            full = (rng.integers(0, 256, int(np.prod(full_shape)) * es).astype(np.uint8) if full_fill
                    else np.zeros(int(np.prod(full_shape)) * es, np.uint8))
            arr = full.view(dtype).reshape(full_shape)
            idx = []
            for s in shape:
                step = int(rng.choice([1, 2, -1, -2]))
                start = int(rng.integers(0, 2))
                if step > 0:
                    idx.append(slice(start, start + step * s, step))
                else:
                    hi = start + (-step) * (s - 1)
                    stop = hi + step * s
                    idx.append(slice(hi, None if stop < 0 else stop, step))
            v = arr[tuple(idx)]
            assert list(v.shape) == shape
            perm = rng.permutation(nd)
            return full, v.transpose(perm), perm

        src_full, sv, sperm = make(True)
        dst_full, dv, dperm = make(False)
        # bring both views to the same logical dim order
        sv = sv.transpose(np.argsort(sperm))
        dv = dv.transpose(np.argsort(dperm))
        if rng.random() < 0.2 and nd >= 1:  # broadcast one source dim
            ax = int(rng.integers(0, nd))
            st = list(sv.strides)
            st[ax] = 0
            sv = np.lib.stride_tricks.as_strided(sv, sv.shape, st)
        say("rearrange trial %d shape %s %s dst %s src %s" % (trial, shape, np.dtype(dtype).name, dv.strides, sv.strides))
        out = run_rearrange(gpu, stream, dst_full, dv, src_full, sv)
        ref = dst_full.copy()
        rv = np.lib.stride_tricks.as_strided(
            ref[dv.__array_interface__["data"][0] - dst_full.__array_interface__["data"][0]:].view(dtype),
            dv.shape, dv.strides)
        oracle.rearrange(rv, sv)
        assert np.array_equal(out, ref)
        done += 1
    assert done == 60


@pytest.mark.parametrize("shape,perm,dtype", [((1000, 37), (1, 0), np.uint16), ((64, 64, 64), (2, 1, 0), np.uint8),
                                              ((7, 2048, 128), (1, 0, 2), np.uint16), ((5, 3, 7, 11, 13), (4, 2, 0, 3, 1), np.uint32),
                                              ((4096, 4096), (0, 1), np.uint16), ((3,), (0,), np.uint64),
                                              ((64, 8200, 64), (1, 0, 2), np.uint16)])  # the last: > 64 MiB
def test_rearrange_permutations(gpu, stream, shape, perm, dtype):
    rng = np.random.default_rng(7)
    src = rng.integers(0, 256, int(np.prod(shape)) * np.dtype(dtype).itemsize).astype(np.uint8).view(dtype).reshape(shape)
    src_host = src.view(np.uint8).reshape(-1)
    dst_host = np.zeros(src_host.size, np.uint8)
    dst_contig = dst_host.view(dtype).reshape([shape[p] for p in perm])
    dst_view = dst_contig.transpose(np.argsort(perm))  # same logical order as src
    say("rearrange perm %s %s" % (shape, perm))
    out = run_rearrange(gpu, stream, dst_host, dst_view, src_host, src)
    assert np.array_equal(out.view(dtype).reshape(dst_contig.shape), src.transpose(perm))


def test_rearrange_errors(gpu, stream):
    op = ophip.Rearrange(gpu)
    L = TensorLayout
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.RearrangeArgs(L(dt.F16, [2, 3], [0, 2]), None, L(dt.F16, [2, 3], [6, 2]), None), None, stream)
    assert e.value.kind == "ShapeNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.RearrangeArgs(L(dt.F16, [2, 3], [6, 2]), None, L(dt.F16, [6], [2]), None), None, stream)
    assert e.value.kind == "RankMismatch"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.RearrangeArgs(L(dt.F16, [2, None], [6, 2]), None, L(dt.F16, [2, None], [6, 2]), None), None,
                  stream)
    assert e.value.kind == "DynamicNotSupport"
    # null bases with something to copy are refused before anything is launched: a scalar (one contiguous run), a
    # contiguous matrix, a transposition; with nothing to copy they are not looked at
    buf = gpu.malloc(64)
    for shape, dst_strides, src_strides in (([], [], []), ([2, 3], [6, 2], [6, 2]), ([64, 64], [2, 128], [128, 2])):
        for dst, src in ((None, buf), (buf, None), (None, None)):
            with pytest.raises(ophip.LaunchError) as e:
                op.launch(ophip.RearrangeArgs(L(dt.F16, shape, dst_strides), dst, L(dt.F16, shape, src_strides), src), None, stream)
            assert e.value.kind == "ArgsNotSupport", (shape, dst, src)
    op.launch(ophip.RearrangeArgs(L(dt.F16, [0, 3], [6, 2]), None, L(dt.F16, [0, 3], [6, 2]), None), None, stream)


# --------------------------------------------------------------- swiglu ----

def test_swiglu_reference_shape(gpu, stream):
    """swiglu/cuda/mod.rs:174-241: n = 5632, d = 2048, inputs U[0,1)."""
    rng = np.random.default_rng(0)
    n, d = 5632, 2048
    g, u = rng.random((n, d)).astype(f16), rng.random((n, d)).astype(f16)
    gd, ud = gpu.from_host(g), gpu.from_host(u)
    op = ophip.Swiglu(gpu)
    args = ophip.SwigluArgs(TensorLayout.of(g), gd, TensorLayout.of(u), ud)
    op.scheme(args, 0)
    say("swiglu reference shape")
    op.launch(args, None, stream)
    out = gpu.to_host(gd, f16, n * d, stream=stream).reshape(n, d)
    assert_close_f16(out, oracle.swiglu(g.copy(), u), "swiglu ref shape")


@pytest.mark.parametrize("n,d,ld", [(16, 11008, 22016), (3, 1001, 2002), (1, 8, 16), (70000, 16, 40), (8195, 512, 1032),
                                     (16400, 2048, 4096), (3100, 11008, 22016)])  # the last two: > 64 MiB (one vector per thread
                                                                                   # over the whole tensor; 1376 vectors a row: workgroups straddle rows)
def test_swiglu_gate_up_halves(gpu, stream, n, d, ld):
    """gate and up are the two halves of one [n, 2*d] GEMM output (independent row strides)."""
    rng = np.random.default_rng(n + d)
    buf = DevBuf(gpu, normal_f16(rng, (n, ld), std=2.0))
    lay = TensorLayout(dt.F16, [n, d], [ld * 2, 2])
    op = ophip.Swiglu(gpu)
    say("swiglu halves n=%d d=%d" % (n, d))
    op.launch(ophip.SwigluArgs(lay, buf.ptr, lay, buf.ptr + d * 2), None, stream)
    out = buf.download(stream).view(f16).reshape(n, ld)
    ref = buf.host.view(f16).reshape(n, ld).copy()
    oracle.swiglu(ref[:, :d], ref[:, d:2 * d])
    assert_close_f16(out, ref, "swiglu halves")
    assert np.array_equal(out[:, d:], ref[:, d:])


def test_swiglu_errors(gpu, stream):
    op = ophip.Swiglu(gpu)
    L = TensorLayout
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.SwigluArgs(L(dt.F16, [4, 8], [16, 2]), None, L(dt.F16, [4, 9], [18, 2]), None), 0)
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.SwigluArgs(L(dt.F16, [4, 8], [16, 2]), None, L(dt.F32, [4, 8], [32, 4]), None), 0)
    assert e.value.kind == "TypeMismatch"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.SwigluArgs(L(dt.F16, [4, 8], [32, 4]), None, L(dt.F16, [4, 8], [16, 2]), None), None, stream)
    assert e.value.kind == "StridesNotSupport"


# -------------------------------------------------------- random_sample ----

def run_sample(gpu, stream, logits, config=None, seed=0.0, op=None, workspace=None):
    n = logits.shape[0]
    ld = gpu.from_host(logits)
    kvd = gpu.from_host(np.array([0xFFFFFFFF, 0xFFFFFFFF], np.uint32))
    op = op or ophip.RandomSample(gpu)
    args = ophip.RandomSampleArgs.layout(ophip.NP_DT[logits.dtype], n)
    args.kv_pair_base, args.logits_base = kvd, ld
    if config is not None:
        args.config, args.seed = config, seed
    op.launch(args, workspace, stream)
    kv = gpu.to_host(kvd, np.uint32, 2, stream=stream)
    return int(kv[0]), int(kv[1])


def val_of(bits, dtype):
    if dtype == f16:
        return float(np.array([bits & 0xFFFF], np.uint16).view(f16)[0])
    return float(np.array([bits], np.uint32).view(f32)[0])


def test_random_sample_benchmark_config(gpu, stream):
    """16 independent rows of f16 logits [32000] ~ N(0, 3) (variance 3), seed 1: argmax, then
    temperature 0.8 / top-k 50 / top-p 0.9 with the fixed draw 0.37."""
    rng = np.random.default_rng(1)
    rows = normal_f16(rng, (16, 32000), std=np.sqrt(3.0))
    op = ophip.RandomSample(gpu)
    cfg = ophip.SampleArgs(0.8, 0.9, 50)
    for r in range(16):
        say("random_sample row %d" % r)
        assert run_sample(gpu, stream, rows[r], op=op) == oracle.argmax(rows[r])
        idx, val = run_sample(gpu, stream, rows[r], cfg, 0.37, op=op)
        ridx, rval = oracle.random_sample(rows[r], 0.8, 0.9, 50, 0.37)
        assert (idx, val) == (ridx, rval)


def test_random_sample_batched_rows_match_single_launches(gpu, stream):
    """The batched entry point (an extension) returns, per row, what the per-row launch returns."""
    rng = np.random.default_rng(1)
    rows = normal_f16(rng, (16, 32000), std=np.sqrt(3.0))
    ld = gpu.from_host(rows)
    kvd = gpu.from_host(np.full(32, 0xFFFFFFFF, np.uint32))
    seeds = rng.random(16).astype(f32)
    sd = gpu.from_host(seeds)
    op = ophip.RandomSample(gpu)
    args = ophip.RandomSampleArgs.layout(dt.F16, 32000)
    args.kv_pair_base, args.logits_base = kvd, ld
    say("random_sample batch argmax")
    op.launch_batch(args, 16, 64000, None, None, stream)
    kv = gpu.to_host(kvd, np.uint32, 32, stream=stream).reshape(16, 2)
    for r in range(16):
        assert (int(kv[r, 0]), int(kv[r, 1])) == oracle.argmax(rows[r])
    args.config, args.seed = ophip.SampleArgs(0.8, 0.9, 50), 0.37
    say("random_sample batch sample, shared draw")
    op.launch_batch(args, 16, 64000, None, None, stream)
    kv = gpu.to_host(kvd, np.uint32, 32, stream=stream).reshape(16, 2)
    for r in range(16):
        assert int(kv[r, 0]) == oracle.random_sample(rows[r], 0.8, 0.9, 50, 0.37)[0]
    say("random_sample batch sample, per-row draws")
    op.launch_batch(args, 16, 64000, sd, None, stream)
    kv = gpu.to_host(kvd, np.uint32, 32, stream=stream).reshape(16, 2)
    for r in range(16):
        assert (int(kv[r, 0]), int(kv[r, 1])) == oracle.random_sample(rows[r], 0.8, 0.9, 50, float(seeds[r]))


def test_random_sample_reference_config_f32(gpu, stream):
    """random_sample/cuda/mod.rs:240-370: n = 32000 f32 logits U[0,1); argmax; T 0.9, top_p 0.9, top_k 200, draw 0.75."""
    rng = np.random.default_rng(0)
    logits = rng.random(32000).astype(f32)
    op = ophip.RandomSample(gpu)
    args = ophip.RandomSampleArgs.layout(dt.F32, 32000)
    ws = op.scheme(args, 2 ** 40)
    say("random_sample reference config, workspace=%d" % ws)
    assert run_sample(gpu, stream, logits, op=op)[0] == oracle.argmax(logits)[0]
    assert run_sample(gpu, stream, logits, ophip.SampleArgs(0.9, 0.9, 200), 0.75, op=op) == \
        oracle.random_sample(logits, 0.9, 0.9, 200, 0.75)


def test_argmax_ties_and_nans(gpu, stream):
    nan = float("nan")
    cases = [
        np.full(1000, 2.5, f16),
        np.array([0.0, -0.0, 0.0, -0.0], f16),
        np.array([1.0, 7.0, 3.0, 7.0, 2.0], f32),
        np.array([1.0, nan, 0.5], f32),
        np.array([1.0, nan, 0.5, 0.75, 0.1], f16),
        np.array([1.0, 2.0, nan], f32),
        np.array([nan, nan], f16),
        np.array([-np.inf, -np.inf, -np.inf], f32),
        np.array([5.0], f16),
    ]
    rng = np.random.default_rng(3)
    big = np.round(rng.standard_normal(32000) * 3).astype(f16)
    cases.append(big)
    withnan = big.copy()
    withnan[[5, 17000, 31000]] = nan
    cases.append(withnan)
    withnan2 = withnan.astype(f32)
    withnan2[31999] = nan
    cases.append(withnan2)
    op = ophip.RandomSample(gpu)
    for i, x in enumerate(cases):
        say("argmax case %d" % i)
        assert run_sample(gpu, stream, x, op=op) == oracle.argmax(x), i


@pytest.mark.parametrize("dtype", [f16, f32])
def test_random_sample_randomised_against_oracle(gpu, stream, dtype):
    rng = np.random.default_rng(5)
    op = ophip.RandomSample(gpu)
    for trial in range(60):
        n = int(rng.choice([1, 2, 7, 63, 64, 65, 1000, 5000, 32000, 50257]))
        x = (rng.standard_normal(n) * rng.choice([0.5, 1.7, 4.0])).astype(f32).astype(dtype)
        if rng.random() < 0.3:
            x = np.round(x).astype(dtype)  # many ties, also at the k-th value
        t = float(rng.uniform(0.3, 2.0))
        top_p = float(rng.uniform(0.05, 1.0))
        top_k = int(rng.choice([2, 5, 50, 200, 1024]))
        seed = float(rng.uniform(0, 1))
        say("sample trial %d n=%d k=%d t=%.3f p=%.3f seed=%.4f" % (trial, n, top_k, t, top_p, seed))
        # index and value (the running sum, rounded to the logits' type) bit for bit
        assert run_sample(gpu, stream, x, ophip.SampleArgs(t, top_p, top_k), seed, op=op) == \
            oracle.random_sample(x, t, top_p, top_k, seed)


def sample_rows(gpu, stream, op, rows, cfg, seeds):
    """One batched launch: rows [r, n] contiguous, one draw per row; returns [(idx, val)] * r."""
    r, n = rows.shape
    ld, sd = gpu.from_host(rows), gpu.from_host(np.asarray(seeds, f32))
    kvd = gpu.from_host(np.full(2 * r, 0xFFFFFFFF, np.uint32))
    args = ophip.RandomSampleArgs.layout(ophip.NP_DT[rows.dtype], n)
    args.kv_pair_base, args.logits_base = kvd, ld
    args.config, args.seed = cfg, 0.5
    op.launch_batch(args, r, n * rows.itemsize, sd, None, stream)
    kv = gpu.to_host(kvd, np.uint32, 2 * r, stream=stream).reshape(r, 2)
    return [(int(a), int(b)) for a, b in kv]


@pytest.mark.parametrize("dtype", [f16, f32])
def test_random_sample_seeded_sweep_is_exact(gpu, stream, dtype):
    """1 040 rows per dtype, vocabularies from 1 000 to 151 936, logits of three widths, a third of them rounded to
    few levels (ties at the k-th value), top_k from 2 to 1024 and top_p from 0.05 to 1: index and value equal the
    oracle's on every row.  (Whenever top_p decides, the sampled entry depends on the reference's sequential f32
    total over all n entries.)"""
    rng = np.random.default_rng(21)
    op = ophip.RandomSample(gpu)
    checked = 0
    for n, groups in [(1000, 12), (5000, 12), (32000, 12), (32768, 4), (50257, 8), (128256, 8), (151936, 9)]:
        for g in range(groups):
            r = 16
            x = (rng.standard_normal((r, n)) * rng.choice([0.5, 1.7, 4.0])).astype(f32).astype(dtype)
            if g % 3 == 2:
                x = np.round(x * 2).astype(dtype)
            t = float(rng.uniform(0.3, 2.0))
            top_p = float(rng.uniform(0.05, 1.0))
            top_k = int(rng.choice([2, 5, 50, 64, 200, 1024]))
            seeds = rng.random(r).astype(f32)
            say("sweep n=%d group %d k=%d t=%.3f p=%.3f" % (n, g, top_k, t, top_p))
            got = sample_rows(gpu, stream, op, x, ophip.SampleArgs(t, top_p, top_k), seeds)
            for i in range(r):
                assert got[i] == oracle.random_sample(x[i], t, top_p, top_k, float(seeds[i])), (n, g, i)
                checked += 1
    assert checked == 1040


@pytest.mark.parametrize("dtype", [f16, f32])
def test_random_sample_draws_on_the_boundaries(gpu, stream, dtype):
    """Draws placed on the boundary between two entries (and a few ulps, then 1e-4, to either side of it), with top_p
    deciding the bound: no interval around a parallel total can tell the two neighbours apart there, only the
    reference's sequential total can.  The boundaries come from a numpy replay of the running sums (its exp differs
    from libm's in the last bit now and then, which is why the draws are only *near* the boundary); the oracle
    says which neighbour is right."""
    rng = np.random.default_rng(22)
    op = ophip.RandomSample(gpu)
    hits = 0
    for n, std, t, top_p, top_k in [(32000, 1.7, 0.8, 0.9, 1024), (32000, 4.0, 1.0, 0.95, 50), (5000, 0.5, 0.7, 0.3, 1024),
                                    (50257, 4.0, 1.3, 0.9, 200), (151936, 4.0, 1.0, 0.9, 64), (32000, 1.7, 0.8, 0.05, 50),
                                    (128256, 1.7, 0.5, 0.5, 1024), (32000, 2.0, 1.0, 0.9, 5000), (32000, 1.7, 0.8, 0.9, 20000),
                                    (50257, 4.0, 1.0, 0.9, ophip.DYN_USIZE)]:
        x = (rng.standard_normal(n) * std).astype(f32).astype(dtype)
        v = np.sort(x.astype(f32))[::-1]
        e = np.exp((v - v[0]) / f32(t)).astype(f32)
        e[0] = 1.0
        cum = np.cumsum(e, dtype=f32)
        pp = f32(cum[-1] * f32(top_p))
        k = min(top_k, n)
        inside = [i for i in range(k) if cum[i] < min(pp, cum[k - 1])]
        assert len(inside) >= 1, "top_p does not decide in this case"
        seeds = []
        for i in rng.choice(inside, size=min(6, len(inside)), replace=False):
            s0 = float(cum[i]) / float(pp)
            seeds += [f32(s0 * (1 + d)) for d in (0.0, 1.2e-7, -1.2e-7, 6e-7, -6e-7, 1e-4, -1e-4)]
        seeds = [s_ for s_ in seeds if 0.0 <= s_ <= 1.0]
        say("boundary draws n=%d k=%d t=%g p=%g: %d draws" % (n, top_k, t, top_p, len(seeds)))
        rows = np.broadcast_to(x, (len(seeds), n)).copy()
        if top_k <= 8192:
            got = sample_rows(gpu, stream, op, rows, ophip.SampleArgs(t, top_p, top_k), seeds)
        else:
            got = [run_sample(gpu, stream, x, ophip.SampleArgs(t, top_p, top_k), float(s_), op=op) for s_ in seeds]
        for s_, g in zip(seeds, got):
            assert g == oracle.random_sample(x, t, top_p, top_k, float(s_)), (n, top_k, float(s_))
            hits += 1
    assert hits >= 200


@pytest.mark.parametrize("dtype", [f16, f32])
def test_random_sample_long_and_misaligned_rows(gpu, stream, dtype):
    """Rows that do not fit the workgroup's registers (more than 32768 logits, or not on a 16-byte boundary) go
    through the short-list kernel: vocabularies of today's models, with smooth logits (few candidates after the
    first radix digit), with logits rounded to a few levels (ties at the k-th value; the candidates overflow the
    list and the kernel falls back to sweeping the row), and a short row that starts 2 or 4 bytes off."""
    rng = np.random.default_rng(11)
    op = ophip.RandomSample(gpu)
    for n, off in [(40000, 0), (50257, 0), (128256, 0), (151936, 0), (32000, 1), (5000, 1), (70001, 1)]:
        for rounded in (False, True):
            x = (rng.standard_normal(n + off) * rng.choice([1.7, 4.0])).astype(f32).astype(dtype)
            if rounded:
                x = np.round(x).astype(dtype)
            for top_k in (50, 200, 1024):
                t, top_p, seed = float(rng.uniform(0.3, 2.0)), float(rng.uniform(0.05, 1.0)), float(rng.uniform(0, 1))
                say("long row n=%d off=%d rounded=%d k=%d t=%.3f p=%.3f seed=%.4f" % (n, off, rounded, top_k, t, top_p, seed))
                ld = gpu.from_host(x)
                kvd = gpu.from_host(np.array([0xFFFFFFFF, 0xFFFFFFFF], np.uint32))
                args = ophip.RandomSampleArgs.layout(ophip.NP_DT[np.dtype(dtype)], n)
                args.kv_pair_base, args.logits_base = kvd, ld.ptr + off * x.itemsize
                args.config, args.seed = ophip.SampleArgs(t, top_p, top_k), seed
                op.launch(args, None, stream)
                kv = gpu.to_host(kvd, np.uint32, 2, stream=stream)
                idx, val = int(kv[0]), int(kv[1])
                row = x[off:]
                assert (idx, val) == oracle.random_sample(row, t, top_p, top_k, seed)


def test_random_sample_all_equal_and_edge_draws(gpu, stream):
    op = ophip.RandomSample(gpu)
    x = np.full(5000, 1.25, f16)  # the k-th value is tied 5000 ways: indices 0..k-1 are the candidates
    for seed in [0.0, 0.37, 0.999, 1.0]:
        say("all-equal seed %g" % seed)
        got = run_sample(gpu, stream, x, ophip.SampleArgs(0.8, 1.0, 50), seed, op=op)
        assert got[0] == oracle.random_sample(x, 0.8, 1.0, 50, seed)[0]
    rng = np.random.default_rng(6)
    y = np.round(rng.standard_normal(3000) * 2).astype(f16)
    assert run_sample(gpu, stream, y, ophip.SampleArgs(0.8, 0.9, 50), 0.0, op=op)[0] == int(np.argmax(y))


@pytest.mark.parametrize("top_k", [1025, 5000, 8192, 8193, ophip.DYN_USIZE])
def test_random_sample_large_top_k_full_sort(gpu, stream, top_k):
    """top_k up to 8192 is sorted in LDS; beyond that (or with no top_k) the row is tried with 1024 and 8192
    candidates first and only goes through the full sort when those do not hold top_p of the probability:
    peaked logits (std 6) settle in the first try, std 1.7 in the second on 32000 logits, flat ones
    (std 0.3) need the full sort."""
    rng = np.random.default_rng(8)
    op = ophip.RandomSample(gpu)
    for n, dtype, std in [(32000, f16, 1.7), (3000, f32, 1.7), (50257, f16, 1.7), (32000, f16, 6.0), (128256, f16, 6.0),
                          (20000, f32, 0.3), (40000, f16, 0.3)]:
        x = (rng.standard_normal(n) * std).astype(f32).astype(dtype)
        args = ophip.RandomSampleArgs.layout(ophip.NP_DT[np.dtype(dtype)], n)
        need = op.scheme(args, 2 ** 40)
        assert need > 0
        for seed, ws in [(0.37, None), (0.93, gpu.malloc(need))]:
            say("full sort n=%d k=%d seed=%g own_ws=%s" % (n, min(top_k, n), seed, ws is not None))
            assert run_sample(gpu, stream, x, ophip.SampleArgs(0.8, 0.95, top_k), seed, op=op, workspace=ws) == \
                oracle.random_sample(x, 0.8, 0.95, top_k, seed)


def test_random_sample_errors_and_build_indices(gpu, stream):
    op = ophip.RandomSample(gpu)
    ptr = ophip.RandomSample.build_indices(1000, stream)
    assert np.array_equal(gpu.to_host(ptr, np.uint32, 1000, stream=stream), np.arange(1000, dtype=np.uint32))
    a = ophip.RandomSampleArgs.layout(dt.F64, 100)
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(a, 0)
    assert e.value.kind == "TypeNotSupport"
    a = ophip.RandomSampleArgs.layout(dt.F16, 100)
    a.indices = TensorLayout(dt.U64, [100], [8])
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(a, 0)
    assert e.value.kind == "TypeNotSupport"
    a = ophip.RandomSampleArgs.layout(dt.F16, 100)
    a.logits = TensorLayout(dt.F16, [100], [4])
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(a, None, stream)
    assert e.value.kind == "StridesNotSupport"
    # Args::layout (random_sample/args.rs:34-49) has null bases, for scheme(): launch refuses them, argmax or not
    for cfg in (ophip.SampleArgs.argmax(), ophip.SampleArgs(0.8, 0.9, 50)):
        a = ophip.RandomSampleArgs.layout(dt.F16, 100)
        a.config = cfg
        with pytest.raises(ophip.LaunchError) as e:
            op.launch(a, None, stream)
        assert e.value.kind == "ArgsNotSupport"
    a = ophip.RandomSampleArgs.layout(dt.F16, None)
    assert op.scheme(a, 0) == 0
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(a, None, stream)
    assert e.value.kind == "DynamicNotSupport"


# -------------------------------------------------------------- mat_mul ----

def run_mat_mul(gpu, stream, c, a, b, alpha, beta, op=None, workspace=None):
    """c, a, b: numpy views (any supported strides) over their own base buffers."""
    def base_of(v):
        b0 = v
        while b0.base is not None and isinstance(b0.base, np.ndarray):
            b0 = b0.base
        return b0

    bufs = []
    for v in (c, a, b):
        root = base_of(v)
        mem = gpu.from_host(np.ascontiguousarray(root).view(np.uint8).reshape(-1)) if root.flags.c_contiguous else None
        assert mem is not None
        off = v.__array_interface__["data"][0] - root.__array_interface__["data"][0]
        bufs.append((root, mem, off))
    op = op or ophip.MatMul(gpu)
    args = ophip.MatMulArgs(TensorLayout.of(c), bufs[0][1].ptr + bufs[0][2], beta,
                            TensorLayout.of(a), bufs[1][1].ptr + bufs[1][2],
                            TensorLayout.of(b), bufs[2][1].ptr + bufs[2][2], alpha)
    op.scheme(args, 0)
    op.launch(args, workspace, stream)
    root = bufs[0][0]
    out = gpu.to_host(bufs[0][1], np.uint8, root.nbytes, stream=stream)
    full = out.view(root.dtype).reshape(root.shape)
    return np.lib.stride_tricks.as_strided(full.reshape(-1)[bufs[0][2] // root.itemsize:], c.shape, c.strides)


def check_mat_mul(out, c0, a, b, alpha, beta, what, rel=1e-2):
    ref = c0.copy()
    oracle.mat_mul(ref, beta, a, b, alpha)
    r = ref.astype(np.float64)
    o = out.astype(np.float64)
    # relative to the magnitude a row of the product reaches (sum |a||b| scale), as the reference's rel metric does
    scale = np.maximum(np.abs(r), np.abs(r).mean() + 1e-6)
    err = np.abs(o - r) / scale
    assert err.max() <= rel, "%s: rel err %g" % (what, err.max())
    assert_close_f16(out, ref, what, abs_tol=2e-3 + 4e-3 * float(np.abs(r).max()), rel_tol=1e-2)


@pytest.mark.parametrize("m", [1, 7, 64, 255, 1024])
def test_mat_mul_reference_shapes(gpu, stream, m):
    """mat_mul/cuda/mod.rs:162-256: batch 4, k = 2048, n = 5632, alpha 0.5, beta 1, inputs U[0,1)."""
    rng = np.random.default_rng(m)
    bt, k, n = 4, 2048, 5632
    a = rng.random((bt, m, k)).astype(f16)
    b = rng.random((bt, k, n)).astype(f16)
    c = rng.random((bt, m, n)).astype(f16)
    say("mat_mul reference shape m=%d" % m)
    oracle.set_threads(8)
    try:
        out = run_mat_mul(gpu, stream, c, a, b, 0.5, 1.0)
        check_mat_mul(out, c, a, b, 0.5, 1.0, "mat_mul m=%d" % m)
        # the reference's own yardstick: f64 CPU result, abs f16 eps / rel 5e-3, <= 0.1 % outliers
        ref64 = 0.5 * a.astype(np.float64) @ b.astype(np.float64) + c.astype(np.float64)
        err = np.abs(out.astype(np.float64) - ref64)
        rel = err / (np.abs(out.astype(np.float64)) + np.abs(ref64) + 2.2e-16)
        assert ((err > 9.765625e-4) & (rel > 5e-3)).sum() * 1000 <= err.size
    finally:
        oracle.set_threads(1)


@pytest.mark.parametrize("shared_b", [False, True])
def test_mat_mul_more_batches_than_a_grid_holds(gpu, stream, shared_b):
    """65538 small products in one call (cuBLAS, which the reference calls at mat_mul/cuda/mod.rs:96-126, takes any batch
    count; a grid's z extent ends at 65535): the call goes out in two launches, the second on the last three batches."""
    rng = np.random.default_rng(7)
    bt, m, n, k = 65538, 3, 8, 16
    a = normal_f16(rng, (bt, m, k))
    b = normal_f16(rng, (1 if shared_b else bt, k, n))
    c = normal_f16(rng, (bt, m, n))
    say("mat_mul batch %d of %dx%dx%d, b %s" % (bt, m, n, k, "shared" if shared_b else "per batch"))
    out = run_mat_mul(gpu, stream, c, a, b, 0.5, 1.0)
    ref = (0.5 * a.astype(np.float64) @ b.astype(np.float64) + c.astype(np.float64))
    assert_close_f16(out, ref.astype(f16), "mat_mul 65538 batches")
    assert_close_f16(out[-3:], ref[-3:].astype(f16), "the batches of the second launch")


DECODE_GEMMS = [
    ("qkv", 1, 16, 12288, 4096, False),
    ("o_proj", 1, 16, 4096, 4096, False),
    ("gate_up", 1, 16, 22016, 4096, False),
    ("down", 1, 16, 4096, 11008, False),
    ("qk_t", 32, 16, 2048, 128, True),
    ("pv", 32, 16, 128, 2048, False),
    ("wide_288_strips", 1, 16, 36864, 1024, False),  # a few more column strips than CUs: K is halved
    ("qkv_32_rows", 1, 32, 12288, 4096, False),  # the 32- and 64-row builds of the paired-step streaming kernel
    ("gate_up_48_rows", 1, 48, 22016, 4096, False),
]


@pytest.mark.parametrize("name,bt,m,n,k,b_transposed", DECODE_GEMMS)
def test_mat_mul_decode_layer_shapes(gpu, stream, name, bt, m, n, k, b_transposed):
    """The six GEMMs of a Llama-7B decode layer, 16 tokens, weights ~ N(0, 0.02) (std 0.02), and one wider weight."""
    rng = np.random.default_rng(len(name) + n)
    shape = lambda *s: (bt,) + s if bt > 1 else s
    if name in ("qk_t", "pv"):
        a = normal_f16(rng, shape(m, k), std=1.0 if name == "qk_t" else 0.05)
        bfull = normal_f16(rng, shape(n, k) if b_transposed else shape(k, n), std=1.0)
        alpha = float(1.0 / np.sqrt(128.0)) if name == "qk_t" else 1.0
    else:
        a = normal_f16(rng, shape(m, k), std=1.0)
        bfull = normal_f16(rng, shape(k, n), std=0.02)
        alpha = 1.0
    b = bfull.swapaxes(-1, -2) if b_transposed else bfull
    c = np.zeros(shape(m, n), f16)
    say("mat_mul decode %s" % name)
    if name in ("qkv", "gate_up", "qkv_32_rows", "gate_up_48_rows", "o_proj", "down", "pv"):
        args = ophip.MatMulArgs(TensorLayout.of(c), None, 0.0, TensorLayout.of(a), None, TensorLayout.of(b), None, alpha)
        what = ophip.MatMul(gpu).describe(args)
        if m <= 16:  # up to 16 rows against an N-contiguous weight: the low-register streaming kernel
            assert what.startswith("stream"), what
        else:
            assert what.startswith("skinny") and "paired" in what, what
    oracle.set_threads(8)
    try:
        out = run_mat_mul(gpu, stream, c, a, b, alpha, 0.0)
        check_mat_mul(out, c, a, b, alpha, 0.0, "decode gemm %s" % name)
    finally:
        oracle.set_threads(1)


STREAM_CASES = [
    # m, n, k, batch, beta, forced ranges for the strips on slow granule classes (None: the planner's), column offset of B
    (16, 22016, 4096, 1, 0.0, None, 0),   # gate/up: the planner cuts the slow strips in two
    (16, 12288, 4096, 1, 0.0, None, 0),   # qkv: 2 ranges, 3 on the slow strips
    (16, 12288, 4096, 1, 0.5, 4, 128),    # forced 4, strips shifted by one granule
    (1, 4096, 4096, 1, 0.0, None, 0),
    (5, 2056, 1024, 1, 1.0, 3, 256),      # N no multiple of 128: the last strip is partial
    (16, 1024, 64, 1, 0.0, 2, 0),         # two K-steps, one per range
    (16, 1024, 32, 1, 0.0, None, 0),      # a single K-step: three of the four waves have nothing to do
    (9, 640, 11008, 1, 0.0, 11, 384),     # 344 K-steps in 11 ranges
    (16, 512, 2048, 3, 0.0, 2, 0),        # batched
    (16, 4096, 4096, 1, 0.0, 0, 0),       # every strip cut alike
]


@pytest.mark.parametrize("m,n,k,bt,beta,slow,shift", STREAM_CASES)
def test_mat_mul_stream_kernel(gpu, stream, monkeypatch, m, n, k, bt, beta, slow, shift):
    """gemm_stream (up to 16 rows, N-contiguous weight, K in whole steps of 32): its numbering of (strip, K range) units
    with the strips of the slow granule classes cut finer, for every alignment of the weight's first strip."""
    rng = np.random.default_rng(m * 7 + n + k + shift)
    if slow is not None:
        monkeypatch.setenv("OPHIP_GEMM_SLOW_SPLIT", str(slow))
    shape = lambda *s: (bt,) + s if bt > 1 else s
    a = normal_f16(rng, shape(m, k), std=1.0)
    wide = normal_f16(rng, shape(k, n + 512 + (-n) % 512), std=0.02)  # rows of whole KiB, at least 512 elements wider than B
    b = wide[..., shift:shift + n]
    c = normal_f16(rng, shape(m, n), std=1.0)
    op = ophip.MatMul(gpu)
    args = ophip.MatMulArgs(TensorLayout.of(c), None, beta, TensorLayout.of(a), None, TensorLayout.of(b), None, 1.0)
    what = op.describe(args)
    say("mat_mul stream %dx%dx%d bt=%d shift=%d: %s" % (m, n, k, bt, shift, what))
    assert what.startswith("stream"), what
    oracle.set_threads(8)
    try:
        out = run_mat_mul(gpu, stream, c, a, b, 1.0, beta, op=op)
        check_mat_mul(out, c, a, b, 1.0, beta, "mat_mul stream")
        again = run_mat_mul(gpu, stream, c, a, b, 1.0, beta, op=op)  # the counters are back at zero
        assert np.array_equal(out.view(np.uint16), again.view(np.uint16))
    finally:
        oracle.set_threads(1)


@pytest.mark.parametrize("m,n,k,bt,beta", [(16, 12288, 4096, 1, 0.0), (16, 4096, 11008, 1, 0.5), (16, 4096, 4096, 1, 0.0),
                                           (24, 1024, 2048, 2, 1.0), (40, 512, 1024, 2, 0.0), (64, 384, 512, 3, 0.5)])
def test_mat_mul_weights_stored_n_by_k(gpu, stream, m, n, k, bt, beta):
    """Weights kept as [N, K] (K-contiguous, the layout of a PyTorch Linear): the weight-streaming kernel's
    mode that reads 256 contiguous bytes per column and transposes through LDS, for 16, 32 and 64-row blocks,
    with and without split K, batched, with beta."""
    rng = np.random.default_rng(m + n + k)
    shape = lambda *s: (bt,) + s if bt > 1 else s
    a = normal_f16(rng, shape(m, k), std=1.0)
    w = normal_f16(rng, shape(n, k), std=0.02)
    b = w.swapaxes(-1, -2)
    c = normal_f16(rng, shape(m, n), std=1.0)
    args = ophip.MatMulArgs(TensorLayout.of(c), None, beta, TensorLayout.of(a), None, TensorLayout.of(b), None, 1.0)
    what = ophip.MatMul(gpu).describe(args)
    say("mat_mul [N,K] weights %dx%dx%d bt=%d: %s" % (m, n, k, bt, what))
    assert "qK256" in what, what
    oracle.set_threads(8)
    try:
        out = run_mat_mul(gpu, stream, c, a, b, 1.0, beta)
        check_mat_mul(out, c, a, b, 1.0, beta, "mat_mul [N,K] weights")
    finally:
        oracle.set_threads(1)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("tc", [False, True])
@pytest.mark.parametrize("m,n,k", [(16, 256, 512), (40, 136, 72), (3, 5, 7), (130, 70, 33)])
def test_mat_mul_all_layouts(gpu, stream, ta, tb, tc, m, n, k):
    rng = np.random.default_rng(m + n + k)
    bt = 3
    a = rng.standard_normal((bt, k, m) if ta else (bt, m, k)).astype(f32).astype(f16)
    b = rng.standard_normal((1, n, k) if tb else (1, k, n)).astype(f32).astype(f16)  # broadcast batch
    c = rng.standard_normal((bt, n, m) if tc else (bt, m, n)).astype(f32).astype(f16)
    av = a.transpose(0, 2, 1) if ta else a
    bv = b.transpose(0, 2, 1) if tb else b
    cv = c.transpose(0, 2, 1) if tc else c
    say("mat_mul layouts ta=%s tb=%s tc=%s %dx%dx%d" % (ta, tb, tc, m, n, k))
    out = run_mat_mul(gpu, stream, cv, av, bv, 0.75, 0.5)
    check_mat_mul(out, cv, av, bv, 0.75, 0.5, "mat_mul layouts")


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("tc", [False, True])
@pytest.mark.parametrize("m,n,k,bt", [(256, 512, 96, 2), (128, 384, 64, 1), (512, 256, 32, 1)])
def test_mat_mul_mfma_tile_kernel_layouts(gpu, stream, ta, tb, tc, m, n, k, bt):
    """Shapes that divide into 128 / 256 tiles run on the LDS-tiled MFMA kernel, in every operand layout."""
    rng = np.random.default_rng(m + n + k + 4 * ta + 2 * tb + tc)
    a = rng.standard_normal((bt, k, m) if ta else (bt, m, k)).astype(f32).astype(f16)
    b = rng.standard_normal((bt, n, k) if tb else (bt, k, n)).astype(f32).astype(f16)
    c = rng.standard_normal((bt, n, m) if tc else (bt, m, n)).astype(f32).astype(f16)
    av = a.transpose(0, 2, 1) if ta else a
    bv = b.transpose(0, 2, 1) if tb else b
    cv = c.transpose(0, 2, 1) if tc else c
    say("mat_mul tile ta=%s tb=%s tc=%s %dx%dx%d" % (ta, tb, tc, m, n, k))
    out = run_mat_mul(gpu, stream, cv, av, bv, 0.75, 0.5)
    check_mat_mul(out, cv, av, bv, 0.75, 0.5, "mat_mul tile layouts")
    cn = np.full(c.shape, np.nan, f16)
    cnv = cn.transpose(0, 2, 1) if tc else cn
    out0 = run_mat_mul(gpu, stream, cnv, av, bv, 1.0, 0.0)
    check_mat_mul(out0, np.zeros(cv.shape, f16), av, bv, 1.0, 0.0, "mat_mul tile beta 0")


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("tc", [False, True])
@pytest.mark.parametrize("m,n,k,bt", [(512, 768, 192, 2), (256, 256, 64, 1), (256, 512, 128, 1)])
def test_mat_mul_mfma_256_tile_kernel_layouts(gpu, stream, monkeypatch, ta, tb, tc, m, n, k, bt):
    """The 256 x 256 tile kernel (normally kept for shapes with at least 128 tiles) on one, two and
    three K-steps - the pipeline's last, second-last and steady-state iterations - in every layout."""
    monkeypatch.setenv("OPHIP_GEMM_TILE", "256")
    rng = np.random.default_rng(m + n + k + 4 * ta + 2 * tb + tc)
    a = rng.standard_normal((bt, k, m) if ta else (bt, m, k)).astype(f32).astype(f16)
    b = rng.standard_normal((bt, n, k) if tb else (bt, k, n)).astype(f32).astype(f16)
    c = rng.standard_normal((bt, n, m) if tc else (bt, m, n)).astype(f32).astype(f16)
    av = a.transpose(0, 2, 1) if ta else a
    bv = b.transpose(0, 2, 1) if tb else b
    cv = c.transpose(0, 2, 1) if tc else c
    say("mat_mul 256-tile ta=%s tb=%s tc=%s %dx%dx%d" % (ta, tb, tc, m, n, k))
    args = ophip.MatMulArgs(TensorLayout.of(cv), None, 0.5, TensorLayout.of(av), None, TensorLayout.of(bv), None, 0.75)
    assert ophip.MatMul(gpu).describe(args).startswith("tile256"), ophip.MatMul(gpu).describe(args)
    out = run_mat_mul(gpu, stream, cv, av, bv, 0.75, 0.5)
    check_mat_mul(out, cv, av, bv, 0.75, 0.5, "mat_mul 256-tile layouts")


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("tc", [False, True])
@pytest.mark.parametrize("m,n,k,bt,force256", [(256, 384, 2048, 1, False), (128, 256, 1056, 2, False), (256, 512, 1088, 1, True)])
def test_mat_mul_tile_kernel_split_k(gpu, stream, monkeypatch, ta, tb, tc, m, n, k, bt, force256):
    """Few tiles and a long K: the tile kernels split K (evenly or not), write f32 partials to the
    workspace and the reduce kernel applies alpha and beta, in every operand layout."""
    if force256:
        monkeypatch.setenv("OPHIP_GEMM_TILE", "256")
    rng = np.random.default_rng(m + n + k + 4 * ta + 2 * tb + tc)
    a = (rng.standard_normal((bt, k, m) if ta else (bt, m, k)) * 0.25).astype(f32).astype(f16)
    b = (rng.standard_normal((bt, n, k) if tb else (bt, k, n)) * 0.25).astype(f32).astype(f16)
    c = rng.standard_normal((bt, n, m) if tc else (bt, m, n)).astype(f32).astype(f16)
    av = a.transpose(0, 2, 1) if ta else a
    bv = b.transpose(0, 2, 1) if tb else b
    cv = c.transpose(0, 2, 1) if tc else c
    args = ophip.MatMulArgs(TensorLayout.of(cv), None, 0.5, TensorLayout.of(av), None, TensorLayout.of(bv), None, 0.75)
    op = ophip.MatMul(gpu)
    what = op.describe(args)
    say("mat_mul tile split-k ta=%s tb=%s tc=%s %dx%dx%d: %s" % (ta, tb, tc, m, n, k, what))
    assert what.startswith("tile256" if force256 else "tile128") and int(what.split("split_k=")[1]) > 1, what
    assert op.scheme(args, 2 ** 40) == int(what.split("split_k=")[1]) * bt * m * n * 4
    out = run_mat_mul(gpu, stream, cv, av, bv, 0.75, 0.5)
    check_mat_mul(out, cv, av, bv, 0.75, 0.5, "mat_mul tile split-k")


def test_mat_mul_compute_bound_shape(gpu, stream):
    rng = np.random.default_rng(12)
    n = 2048
    a = normal_f16(rng, (n, n), std=1.0)
    b = normal_f16(rng, (n, n), std=0.05)
    c = np.zeros((n, n), f16)
    say("mat_mul 2048^3")
    out = run_mat_mul(gpu, stream, c, a, b, 1.0, 0.0)
    ref = (a.astype(np.float32) @ b.astype(np.float32)).astype(np.float64)
    err = np.abs(out.astype(np.float64) - ref)
    assert (err <= 2e-3 + 1e-2 * np.abs(ref)).all(), err.max()
    oracle.set_threads(8)
    try:
        sub = oracle.mat_mul(np.zeros((64, n), f16), 0.0, a[:64], b, 1.0)  # oracle on a slice of rows
    finally:
        oracle.set_threads(1)
    assert_close_f16(out[:64], sub, "2048^3 rows 0..63", abs_tol=2e-3 + 4e-3 * float(np.abs(sub).max()))


@pytest.mark.parametrize("tokens,n,k,b_transposed,beta", [(509, 1536, 1024, False, 0.0), (509, 1536, 1024, True, 0.5),
                                                          (100, 12288, 4096, False, 0.0), (300, 1000, 2048, True, 1.0),
                                                          (65, 136, 64, False, 0.0)])
def test_mat_mul_prefill_with_any_token_count(gpu, stream, tokens, n, k, b_transposed, beta):
    """A prefill GEMM whose token count is no multiple of the tile (and a weight whose width is not either):
    still the MFMA tile kernel, with its last tiles cut."""
    rng = np.random.default_rng(tokens + n)
    a = normal_f16(rng, (tokens, k), std=1.0)
    b = normal_f16(rng, (n, k), std=0.02).T if b_transposed else normal_f16(rng, (k, n), std=0.02)
    c = normal_f16(rng, (tokens, n), std=1.0)
    args = ophip.MatMulArgs(TensorLayout.of(c), None, beta, TensorLayout.of(a), None, TensorLayout.of(b), None, 1.0)
    what = ophip.MatMul(gpu).describe(args)
    say("mat_mul prefill %d x %d x %d [%s]" % (tokens, n, k, what))
    assert what.startswith("tile") and "ragged" in what, what
    oracle.set_threads(8)
    try:
        out = run_mat_mul(gpu, stream, c, a, b, 1.0, beta)
        check_mat_mul(out, c, a, b, 1.0, beta, "prefill %d tokens" % tokens)
    finally:
        oracle.set_threads(1)


@pytest.mark.parametrize("bt,m,n,k", [(32, 16, 128, 2047), (4, 16, 128, 301), (2, 40, 256, 1001), (1, 7, 64, 33)])
def test_mat_mul_few_rows_with_any_k(gpu, stream, bt, m, n, k):
    """The PV product of a decode step: a handful of score rows (padded to 16 bytes, as the attention operator
    keeps them) times V[att, dh] for an att that is no multiple of 8.  Still the weight-streaming kernel: its
    last K-step masks the scores element by element and V by rows."""
    rng = np.random.default_rng(k)
    ld = (k + 7) // 8 * 8
    a = normal_f16(rng, (bt, m, ld), std=0.05)[:, :, :k]
    b = normal_f16(rng, (bt, k, n), std=1.0)
    c = np.zeros((bt, m, n), f16)
    args = ophip.MatMulArgs(TensorLayout.of(c), None, 0.0, TensorLayout.of(a), None, TensorLayout.of(b), None, 1.0)
    what = ophip.MatMul(gpu).describe(args)
    say("mat_mul %d x [%d x %d x %d] [%s]" % (bt, m, n, k, what))
    assert what.startswith("skinny"), what
    out = run_mat_mul(gpu, stream, c, a, b, 1.0, 0.0)
    check_mat_mul(out, c, a, b, 1.0, 0.0, "few rows, k = %d" % k)


def test_mat_mul_beta_zero_never_reads_c_and_scalars_round_to_f16(gpu, stream):
    a = np.ones((16, 2048), f16)
    a[:, 2047] = 0  # 2047 ones per row
    b = np.ones((2048, 128), f16)
    c = np.full((16, 128), np.nan, f16)
    say("mat_mul beta=0 over NaN")
    out = run_mat_mul(gpu, stream, c, a, b, 0.1, 0.0)
    assert (out == f16(204.625)).all()  # alpha rounded to f16 first; 0.1 unrounded would give 204.75
    c3 = np.full((3, 5), np.nan, f16)
    out = run_mat_mul(gpu, stream, c3, np.ones((3, 7), f16), np.ones((7, 5), f16), 1.0, 0.0)
    assert (out == f16(7)).all()


def test_mat_mul_split_k_workspace_paths(gpu, stream):
    rng = np.random.default_rng(11)
    a = normal_f16(rng, (16, 4096))
    b = normal_f16(rng, (4096, 1024), std=0.02)
    c = normal_f16(rng, (16, 1024))
    op = ophip.MatMul(gpu)
    args = ophip.MatMulArgs(TensorLayout.of(c), None, 1.0, TensorLayout.of(a), None, TensorLayout.of(b), None, 1.0)
    need = op.scheme(args, 2 ** 40)
    say("mat_mul split-k workspace need=%d" % need)
    assert need > 0 and op.scheme(args, 16) == 0
    ref = c.copy()
    oracle.mat_mul(ref, 1.0, a, b, 1.0)
    pool = ophip.StreamMemPool(gpu, stream)
    pool.put(need + 4096)
    for ws, qa in [(None, stream), (gpu.malloc(need), stream), (None, pool)]:
        out = run_mat_mul_with(gpu, stream, c, a, b, op, ws, qa)
        assert_close_f16(out, ref, "split-k", abs_tol=4e-3)
    # a caller's slice that starts off a 16-byte boundary: used from the next boundary on when enough of it is
    # left, otherwise it counts as too small and the queue allocator serves the launch
    slab = gpu.malloc(need + 64)
    for off, length in [(2, need + 14), (6, need + 32), (2, need), (12, need + 3)]:
        out = run_mat_mul_with(gpu, stream, c, a, b, op, (slab.ptr + off, length), stream)
        assert_close_f16(out, ref, "split-k, workspace at +%d" % off, abs_tol=4e-3)


@pytest.mark.parametrize("m,n,k", [(16, 12288, 4096), (16, 1024, 4096), (48, 4096, 11008), (16, 1160, 2048)])
def test_mat_mul_split_k_ignores_what_the_workspace_held(gpu, stream, m, n, k):
    """The workgroup of a column strip that arrives last sums the partial sums of all K ranges: it must
    see the other workgroups' partial sums, not what the workspace held before (NaNs here), however close
    together they finish.  Many launches, each bit-identical to the first, which is checked against the oracle."""
    rng = np.random.default_rng(m + n + k)
    a = normal_f16(rng, (m, k))
    b = normal_f16(rng, (k, n), std=0.02)
    c = np.zeros((m, n), f16)
    op = ophip.MatMul(gpu)
    cd, ad, bd = gpu.from_host(c), gpu.from_host(a), gpu.from_host(b)
    args = ophip.MatMulArgs(TensorLayout.of(c), cd, 0.0, TensorLayout.of(a), ad, TensorLayout.of(b), bd, 1.0)
    what = op.describe(args)
    assert what.split()[0] in ("skinny", "stream") and "split_k=1" not in what, what
    need = op.scheme(args, 2 ** 40)
    assert need > 0
    ws = gpu.malloc(need)
    say("mat_mul split-k over a dirty workspace %dx%dx%d: %s" % (m, n, k, what))
    ref = c.copy()
    oracle.mat_mul(ref, 0.0, a, b, 1.0)
    first = None
    for it in range(40):
        gpu.memset(ws, 0xFF, stream=stream)
        op.launch(args, ws, stream)
        out = gpu.to_host(cd, f16, c.size, stream=stream).reshape(c.shape)
        if first is None:
            first = out
            assert_close_f16(out, ref, "split-k over a dirty workspace", abs_tol=4e-3)
        else:
            assert np.array_equal(out.view(np.uint16), first.view(np.uint16)), "launch %d differs from the first" % it


def test_mat_mul_split_k_on_streams_that_come_and_go(gpu, stream):
    """The arrival counters of a split-K product belong to the operator, one buffer per stream.  A stream that is
    destroyed hands its buffer on: products on a row of short-lived streams, interleaved with the long-lived one, all
    match the first."""
    rng = np.random.default_rng(5)
    a = normal_f16(rng, (16, 4096))
    b = normal_f16(rng, (4096, 4096), std=0.02)
    c = np.zeros((16, 4096), f16)
    op = ophip.MatMul(gpu)
    cd, ad, bd = gpu.from_host(c), gpu.from_host(a), gpu.from_host(b)
    args = ophip.MatMulArgs(TensorLayout.of(c), cd, 0.0, TensorLayout.of(a), ad, TensorLayout.of(b), bd, 1.0)
    assert "split_k=1" not in op.describe(args)
    ws = gpu.malloc(op.scheme(args, 2 ** 40))
    ref = c.copy()
    oracle.mat_mul(ref, 0.0, a, b, 1.0)
    say("mat_mul split-k on streams that come and go")
    op.launch(args, ws, stream)
    first = gpu.to_host(cd, f16, c.size, stream=stream).reshape(c.shape)
    assert_close_f16(first, ref, "split-k, first stream", abs_tol=4e-3)
    for it in range(6):
        other = gpu.stream()
        gpu.memset(cd, 0xFF, stream=other)
        op.launch(args, ws, other)
        out = gpu.to_host(cd, f16, c.size, stream=other).reshape(c.shape)
        other.destroy()
        assert np.array_equal(out.view(np.uint16), first.view(np.uint16)), "stream %d differs" % it
        gpu.memset(cd, 0xFF, stream=stream)
        op.launch(args, ws, stream)
        out = gpu.to_host(cd, f16, c.size, stream=stream).reshape(c.shape)
        assert np.array_equal(out.view(np.uint16), first.view(np.uint16)), "back on the first stream, round %d" % it


def run_mat_mul_with(gpu, stream, c, a, b, op, ws, qa):
    cd, ad, bd = gpu.from_host(c), gpu.from_host(a), gpu.from_host(b)
    args = ophip.MatMulArgs(TensorLayout.of(c), cd, 1.0, TensorLayout.of(a), ad, TensorLayout.of(b), bd, 1.0)
    op.launch(args, ws, qa)
    return gpu.to_host(cd, f16, c.size, stream=stream).reshape(c.shape)


def test_mat_mul_errors(gpu, stream):
    op = ophip.MatMul(gpu)
    L = TensorLayout
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.MatMulArgs(L(dt.F16, [5, 7], [14, 2]), None, 0.0, L(dt.F16, [5, 4], [8, 2]), None,
                                   L(dt.F16, [3, 7], [14, 2]), None, 1.0), None, stream)
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.MatMulArgs(L(dt.U16, [5, 7], [14, 2]), None, 0.0, L(dt.U16, [5, 3], [6, 2]), None,
                                   L(dt.U16, [3, 7], [14, 2]), None, 1.0), None, stream)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.MatMulArgs(L(dt.F16, [5, None], [14, 2]), None, 0.0, L(dt.F16, [5, 3], [6, 2]), None,
                                   L(dt.F16, [3, 7], [14, 2]), None, 1.0), None, stream)
    assert e.value.kind == "DynamicNotSupport"


# ------------------------------------------------------ queue allocator ----

def test_stream_mem_pool_serves_workspaces(gpu, stream):
    pool = ophip.StreamMemPool(gpu, stream)
    pool.put(1 << 20)
    qa = pool.queue_alloc
    p1 = qa.alloc(qa.ctx, 1000)
    p2 = qa.alloc(qa.ctx, 5000)
    assert p1 and p2 and p1 != p2 and p1 % 256 == 0 and p2 % 256 == 0
    qa.free(qa.ctx, p1)
    p3 = qa.alloc(qa.ctx, 700)
    assert p3 == p1
    assert not qa.alloc(qa.ctx, 2 << 20)  # the reference panics "out of memory"; here the launch fails cleanly
    pool.destroy()


# ---------------------------------------------------------- launch graphs ----

def test_recorded_launch_sequence_replays_like_eager_launches(gpu, stream):
    """rms_norm -> split-K mat_mul -> swiglu recorded once and replayed: every replay must give the eager
    result, with eager work and synchronisations in between."""
    rng = np.random.default_rng(21)
    x = normal_f16(rng, (16, 4096))
    w = rng.uniform(0.5, 1.5, 4096).astype(f32).astype(f16)
    wgu = normal_f16(rng, (4096, 2048), std=0.02)
    xd, wd, wgud = gpu.from_host(x), gpu.from_host(w), gpu.from_host(wgu)
    xn, gu = gpu.malloc(x.nbytes), gpu.malloc(16 * 2048 * 2)
    L = TensorLayout
    c = lambda *s: L.new_contiguous(dt.F16, list(s))
    half = L(dt.F16, [16, 1024], [2048 * 2, 2])
    rms, mm, sw = ophip.RmsNorm(gpu), ophip.MatMul(gpu), ophip.Swiglu(gpu)
    a_rms = ophip.RmsNormArgs(c(16, 4096), xn, c(16, 4096), xd, c(4096), wd, 1e-5)
    a_mm = ophip.MatMulArgs(c(16, 2048), gu, 0.0, c(16, 4096), xn, c(4096, 2048), wgud, 1.0)
    a_sw = ophip.SwigluArgs(half, gu.ptr, half, gu.ptr + 1024 * 2)
    ws = gpu.malloc(max(mm.scheme(a_mm, 1 << 30), 1))

    def sequence():
        rms.launch(a_rms, None, stream)
        mm.launch(a_mm, ws, stream)
        sw.launch(a_sw, None, stream)

    say("launch graph: eager reference")
    sequence()
    want = gpu.to_host(gu, f16, 16 * 2048, stream=stream).copy()
    stream.begin_capture()
    sequence()
    graph = stream.end_capture()
    for rep in range(4):
        gpu.memset(gu, 0, stream=stream)
        say("launch graph: replay %d" % rep)
        graph.launch(stream)
        got = gpu.to_host(gu, f16, 16 * 2048, stream=stream)
        assert np.array_equal(got, want), "replay %d differs from the eager result" % rep
        rms.launch(a_rms, None, stream)  # eager work between replays
        stream.synchronize()
    graph.destroy()


def test_first_split_k_product_of_an_operator_may_be_recorded(gpu, stream):
    """An operator that has never launched on the stream sets up its arrival counters with its first split-K
    product; when that launch is being recorded, the set-up is part of the recording and every replay is right."""
    rng = np.random.default_rng(22)
    a, b = normal_f16(rng, (16, 4096)), normal_f16(rng, (4096, 1024), std=0.02)
    ad, bd = gpu.from_host(a), gpu.from_host(b)
    cd = gpu.malloc(16 * 1024 * 2)
    c = lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    args = ophip.MatMulArgs(c(16, 1024), cd, 0.0, c(16, 4096), ad, c(4096, 1024), bd, 1.0)
    eager = ophip.MatMul(gpu)
    assert "split_k=1" not in eager.describe(args)
    ws = gpu.malloc(eager.scheme(args, 1 << 30))
    eager.launch(args, ws, stream)
    want = gpu.to_host(cd, f16, 16 * 1024, stream=stream).copy()
    fresh = ophip.MatMul(gpu)
    say("launch graph: an operator's first split-K product, recorded")
    stream.begin_capture()
    fresh.launch(args, ws, stream)
    graph = stream.end_capture()
    for rep in range(4):
        gpu.memset(cd, 0xFF, stream=stream)
        gpu.memset(ws, 0xFF, stream=stream)
        graph.launch(stream)
        got = gpu.to_host(cd, f16, 16 * 1024, stream=stream)
        assert np.array_equal(got, want), "replay %d differs from the eager result" % rep
        fresh.launch(args, ws, stream)  # the same operator, eagerly, between replays
        assert np.array_equal(gpu.to_host(cd, f16, 16 * 1024, stream=stream), want)
    graph.destroy()


def test_memset_on_a_stream_any_alignment_and_recorded(gpu, stream):
    """ophip_memset with a stream is a kernel launch: any offset and length, bytes around the range untouched,
    and a recorded fill replays (over changed contents) like the eager one."""
    size = 1 << 16
    buf = gpu.malloc(size)
    for off, n, val in [(0, size, 0xAB), (1, 1, 0x01), (3, 29, 0x7F), (16, 4096, 0x00), (17, 4097, 0xFF), (5, 7, 0x3C),
                        (15, 1, 0x11), (15, 17, 0x22), (32, 15, 0x33), (1, size - 2, 0x5A)]:
        gpu.memset(buf, 0xEE)
        gpu.memset(buf, val, n, stream=stream, offset=off)
        got = gpu.to_host(buf, np.uint8, size, stream=stream)
        want = np.full(size, 0xEE, np.uint8)
        want[off:off + n] = val
        assert np.array_equal(got, want), (off, n, val)
    stream.begin_capture()
    gpu.memset(buf, 0x42, 1000, stream=stream, offset=7)
    graph = stream.end_capture()
    for rep in range(3):
        gpu.memset(buf, rep, stream=stream)
        graph.launch(stream)
        got = gpu.to_host(buf, np.uint8, size, stream=stream)
        want = np.full(size, rep, np.uint8)
        want[7:1007] = 0x42
        assert np.array_equal(got, want), "replay %d" % rep
    graph.destroy()


def test_time_next_launch_gives_the_kernels_own_duration(gpu, stream):
    """ophip_time_next_launch: the next kernel on the stream records its own begin and end; the one after is an
    ordinary launch again, and results are unaffected."""
    rng = np.random.default_rng(3)
    x = normal_f16(rng, (64, 4096))
    w = rng.uniform(0.5, 1.5, 4096).astype(f32).astype(f16)
    xd, wd, yd = gpu.from_host(x), gpu.from_host(w), gpu.malloc(x.nbytes)
    c = lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    op = ophip.RmsNorm(gpu)
    a = ophip.RmsNormArgs(c(64, 4096), yd, c(64, 4096), xd, c(4096), wd, 1e-5)
    op.launch(a, None, stream)
    e0, e1 = gpu.event(), gpu.event()
    gpu.time_next_launch(stream, e0, e1)
    op.launch(a, None, stream)
    op.launch(a, None, stream)
    stream.synchronize()
    us = e0.elapsed_ms(e1) * 1e3
    say("rms_norm [64, 4096] by its own events: %.2f us" % us)
    assert 0.5 < us < 200.0
    got = gpu.to_host(yd, f16, x.size, stream=stream).reshape(x.shape)
    assert_close_f16(got, oracle.rms_norm(np.empty_like(x), x, w, 1e-5), "rms_norm after a timed launch")


# ------------------------------------------------------------- threading ----

def test_one_operator_instance_launched_from_several_threads(gpu):
    """launch takes &self in the reference and is internally synchronised (rms_norm/cuda/mod.rs:16,90-96):
    one mat_mul and one rms_norm instance, four threads, each on its own stream with its own buffers."""
    import threading

    rms, mm = ophip.RmsNorm(gpu), ophip.MatMul(gpu)
    L = TensorLayout
    c = lambda *s: L.new_contiguous(dt.F16, list(s))
    errors = []

    def worker(seed):
        try:
            rng = np.random.default_rng(seed)
            st = gpu.stream()
            x = normal_f16(rng, (16, 2048))
            w = rng.uniform(0.5, 1.5, 2048).astype(f32).astype(f16)
            b = normal_f16(rng, (2048, 512), std=0.05)
            xd, wd, bd = gpu.from_host(x), gpu.from_host(w), gpu.from_host(b)
            xn, out = gpu.malloc(x.nbytes), gpu.malloc(16 * 512 * 2)
            ref_n = oracle.rms_norm(np.empty_like(x), x, w, 1e-5)
            ref = oracle.mat_mul(np.zeros((16, 512), f16), 0.0, ref_n, b, 1.0)
            for _ in range(25):
                rms.launch(ophip.RmsNormArgs(c(16, 2048), xn, c(16, 2048), xd, c(2048), wd, 1e-5), None, st)
                mm.launch(ophip.MatMulArgs(c(16, 512), out, 0.0, c(16, 2048), xn, c(2048, 512), bd, 1.0), None, st)
            got = gpu.to_host(out, f16, 16 * 512, stream=st).reshape(16, 512)
            assert_close_f16(got, ref, "thread %d" % seed, abs_tol=4e-3)
            st.synchronize()
        except Exception as e:  # surfaced in the main thread
            errors.append(e)

    say("4 threads x 25 launches of shared operator instances")
    threads = [threading.Thread(target=worker, args=(s,)) for s in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


@pytest.mark.gpu
@pytest.mark.parametrize("nbytes,off", [((64 << 20) + 4096, 0), ((64 << 20) + 16, 32), ((64 << 20) + 24, 0), ((70 << 20), 8)])
def test_rearrange_large_contiguous_run_is_bit_exact(gpu, stream, nbytes, off):
    """One contiguous run beyond 64 MiB: the copy kernel when bases and length are whole 16-byte chunks, the runtime's
    device-to-device copy otherwise; every byte, and nothing outside the run."""
    rng = np.random.default_rng(nbytes % 1000 + off)
    src = rng.integers(0, 256, nbytes + 64, dtype=np.uint8)
    sd, dd = gpu.from_host(src), gpu.malloc(nbytes + 128)
    gpu.memset(dd, 0xEE)
    lay = TensorLayout(dt.U8, [nbytes], [1])
    say("rearrange contiguous %d bytes, offset %d" % (nbytes, off))
    ophip.Rearrange(gpu).launch(ophip.RearrangeArgs(lay, dd.ptr + off, lay, sd.ptr + off), None, stream)
    out = gpu.to_host(dd, np.uint8, nbytes + 128, stream=stream)
    assert np.array_equal(out[off:off + nbytes], src[off:off + nbytes])
    assert (out[:off] == 0xEE).all() and (out[off + nbytes:] == 0xEE).all()


@pytest.mark.parametrize("shape,perm,dtype", [((8192, 4096), (1, 0), np.uint16), ((1000, 777), (1, 0), np.uint16), ((33, 4099), (1, 0), np.uint32),
                                              ((5, 300, 200), (0, 2, 1), np.uint16), ((3, 64, 5, 96), (2, 3, 0, 1), np.uint64),
                                              ((7, 129, 65), (2, 1, 0), np.uint32), ((40, 33, 32), (2, 0, 1), np.uint16)])
def test_rearrange_transposes_of_small_units_bit_exact(gpu, stream, shape, perm, dtype):
    """dst = src.transpose(perm), both contiguous, units of 2 / 4 / 8 bytes: the LDS-tiled kernel where the destination's
    and the source's contiguous dimensions are both at least 32 long, the element-wise one otherwise; every byte against
    numpy and the oracle."""
    rng = np.random.default_rng(sum(shape))
    src = rng.integers(0, np.iinfo(dtype).max, shape, dtype=dtype)
    want = np.ascontiguousarray(src.transpose(perm))
    nb = src.dtype.itemsize
    # the destination seen in the source's index order: contiguous strides of `want`, permuted back
    dstrides = [0] * len(shape)
    for k, ax in enumerate(perm):
        dstrides[ax] = want.strides[k]
    code = {2: dt.U16, 4: dt.U32, 8: dt.U64}[nb]
    sd, dd = gpu.from_host(src), gpu.malloc(src.nbytes + 64)
    gpu.memset(dd, 0xEE)
    say("rearrange transpose %s perm %s %d-byte units" % (shape, perm, nb))
    ophip.Rearrange(gpu).launch(ophip.RearrangeArgs(TensorLayout(code, list(shape), dstrides), dd, TensorLayout.of(src), sd), None, stream)
    out = gpu.to_host(dd, np.uint8, src.nbytes + 64, stream=stream)
    assert np.array_equal(out[:src.nbytes].view(dtype).reshape(want.shape), want)
    assert (out[src.nbytes:] == 0xEE).all()
