"""bf16 data on every floating-point operator, through the C ABI.

The reference's CUDA backend compiles rms_norm, layer_norm, add and add_rows for any pair of named types, bf16 included
(handle/cuda/mod.rs:188-210 with rms_norm/cuda/mod.rs:146-147, layer_norm/cuda/mod.rs:158-159, add/cuda/mod.rs:105-123,
add_rows/cuda/mod.rs:135-163); its CPU backend, which the oracle restates, has no bf16 kernel at all, and for rope,
softmax, swiglu, gelu and mat_mul neither backend has one.  PARITY UNPINNED against the reference: what is checked here is
the arithmetic the kernels document -- the f16 kernels' formulas in f32, one rounding to bf16 (nearest even) at the end --
against the same formula in f64 (within one bf16 step, 2^-7 relative) or in numpy f32 (the sums: every bit)."""
import numpy as np
import pytest

import ophip
from ophip import TensorLayout, dt

pytestmark = pytest.mark.gpu

f32, f64, u16, u32 = np.float32, np.float64, np.uint16, np.uint32


def say(msg):
    print(msg, flush=True)


def to_bf16(x):
    """f32 -> bf16 bit patterns, round to nearest even (no NaNs in these tests)."""
    u = np.ascontiguousarray(x, f32).view(u32)
    return ((u + (((u >> 16) & 1) + 0x7FFF)) >> 16).astype(u16)


def from_bf16(b):
    return (np.asarray(b, u16).astype(u32) << 16).view(f32)


def test_bf16_helpers_round_to_nearest_even():
    # 1 + 2^-8 is halfway between 1 and 1 + 2^-7: ties go to the even significand
    assert to_bf16(np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -2.5, 0.0], f32)).tolist() == \
        [0x3F80, 0x3F80, 0x3F82, 0xC020, 0]
    assert from_bf16(np.array([0x3F80, 0xC020], u16)).tolist() == [1.0, -2.5]


def L2(dtype, n, d, ld=None):
    nb = ophip.dtype_nbytes(dtype)
    return TensorLayout(dtype, [n, d], [(ld or d) * nb, nb])


def one_step(ref):
    return np.abs(ref) * 2.0 ** -7 + 1e-30


@pytest.mark.parametrize("wdt", ["bf16", "f32"])
@pytest.mark.parametrize("n,d", [(64, 4096), (16, 4096), (3, 1001), (5, 24), (300, 512), (2, 16384), (20000, 2048), (1, 8), (8200, 5120)])
def test_rms_norm_bf16(gpu, stream, n, d, wdt):
    rng = np.random.default_rng(n + d)
    xb = to_bf16(rng.standard_normal((n, d)).astype(f32))
    w = rng.uniform(0.5, 1.5, d).astype(f32)
    wb = to_bf16(w) if wdt == "bf16" else w
    wv = from_bf16(wb) if wdt == "bf16" else w
    xd, wd, yd = gpu.from_host(xb), gpu.from_host(wb), gpu.malloc(xb.nbytes)
    op = ophip.RmsNorm(gpu)
    wl = TensorLayout(dt.BF16 if wdt == "bf16" else dt.F32, [d], [2 if wdt == "bf16" else 4])
    args = ophip.RmsNormArgs(L2(dt.BF16, n, d), yd, L2(dt.BF16, n, d), xd, wl, wd, 1e-5)
    op.scheme(args, 0)
    say("rms_norm bf16 n=%d d=%d w=%s" % (n, d, wdt))
    op.launch(args, None, stream)
    y = from_bf16(gpu.to_host(yd, u16, n * d, stream=stream)).reshape(n, d).astype(f64)
    x = from_bf16(xb).astype(f64)
    k = 1.0 / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-5)
    ref = k * wv.astype(f64) * x
    assert (np.abs(y - ref) <= one_step(ref)).all(), np.abs(y - ref).max()
    # and nearly every element is the nearest bf16 of the exact value (the f32 product may sit on the other side of a tie)
    assert (to_bf16(ref.astype(f32)) == to_bf16(y.astype(f32))).mean() > 0.99


def test_rms_norm_bf16_strided_rows_and_scalar_path(gpu, stream):
    rng = np.random.default_rng(5)
    n, d, ld = 9, 1000, 1536
    host = to_bf16(rng.standard_normal((n, ld)).astype(f32))
    w = to_bf16(rng.uniform(0.5, 1.5, d).astype(f32))
    xd, wd = gpu.from_host(host), gpu.from_host(w)
    yd = gpu.malloc(host.nbytes)
    gpu.memset(yd, 0)
    op = ophip.RmsNorm(gpu)
    # rows 6 bytes into a padded buffer: no 16-byte vectors, the element-wise kernel
    args = ophip.RmsNormArgs(L2(dt.BF16, n, d, ld), yd.ptr + 6, L2(dt.BF16, n, d, ld), xd.ptr + 6, TensorLayout(dt.BF16, [d], [2]), wd, 1e-6)
    op.launch(args, None, stream)
    out = gpu.to_host(yd, u16, host.size, stream=stream).reshape(n, ld)
    x = from_bf16(host[:, 3:3 + d]).astype(f64)
    ref = (1.0 / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-6)) * from_bf16(w).astype(f64) * x
    y = from_bf16(out[:, 3:3 + d]).astype(f64)
    assert (np.abs(y - ref) <= one_step(ref)).all()
    assert (out[:, :3] == 0).all() and (out[:, 3 + d:] == 0).all()  # nothing outside the view was written


@pytest.mark.parametrize("adt,wdt", [("f16", "bf16"), ("bf16", "f16"), ("f32", "f16"), ("f32", "bf16")])
@pytest.mark.parametrize("n,d", [(16, 4096), (3, 1001), (64, 24)])
def test_rms_norm_mixed_activation_and_weight_types(gpu, stream, n, d, adt, wdt):
    """The pairs of f16 / bf16 / f32 that neither has a vector kernel nor exists in the reference's CPU backend (its CUDA
    backend compiles rms_norm for any pair of named types, rms_norm/cuda/mod.rs:117-122): parity unpinned against the
    reference; checked against the formula in f64, within one step of the activations' type."""
    rng = np.random.default_rng(n * 3 + d)
    enc = {"f16": lambda v: v.astype(np.float16), "bf16": to_bf16, "f32": lambda v: v.astype(f32)}
    dec = {"f16": lambda v: v.astype(f64), "bf16": lambda v: from_bf16(v).astype(f64), "f32": lambda v: v.astype(f64)}
    code = {"f16": dt.F16, "bf16": dt.BF16, "f32": dt.F32}
    xa, wa = enc[adt](rng.standard_normal((n, d)).astype(f32)), enc[wdt](rng.uniform(0.5, 1.5, d).astype(f32))
    xd, wd, yd = gpu.from_host(xa), gpu.from_host(wa), gpu.malloc(xa.nbytes)
    op = ophip.RmsNorm(gpu)
    args = ophip.RmsNormArgs(L2(code[adt], n, d), yd, L2(code[adt], n, d), xd, TensorLayout(code[wdt], [d], [wa.itemsize]), wd, 1e-5)
    op.scheme(args, 0)
    say("rms_norm n=%d d=%d activations %s weights %s" % (n, d, adt, wdt))
    op.launch(args, None, stream)
    y = dec[adt](gpu.to_host(yd, xa.dtype, n * d, stream=stream).reshape(n, d))
    x = dec[adt](xa)
    ref = (1.0 / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-5)) * dec[wdt](wa) * x
    # one step of the activations' type (f32: a few, the row sum is a parallel f32 sum), and half an f16 subnormal step
    step = {"f16": 2.0 ** -10, "bf16": 2.0 ** -7, "f32": 2.0 ** -18}[adt]
    floor = 2.0 ** -24 if adt == "f16" else 1e-30
    assert (np.abs(y - ref) <= np.abs(ref) * step + floor).all(), np.abs(y - ref).max()


def test_rms_norm_refuses_the_pairs_it_has_no_kernel_for(gpu):
    """f64 mixed with a narrower type (the CUDA backend would compute such a pair in f32) and non-floating types."""
    op = ophip.RmsNorm(gpu)
    for adt, wdt in ((dt.F64, dt.F32), (dt.F32, dt.F64), (dt.F16, dt.F64), (dt.F64, dt.BF16), (dt.U32, dt.U32), (dt.F16, dt.I32)):
        args = ophip.RmsNormArgs(L2(adt, 4, 64), None, L2(adt, 4, 64), None, TensorLayout(wdt, [64], [ophip.dtype_nbytes(wdt)]), None, 1e-5)
        with pytest.raises(ophip.SchemeError) as e:
            op.scheme(args, 0)
        assert e.value.kind == "TypeNotSupport", (adt, wdt)


@pytest.mark.parametrize("wdt", ["bf16", "f32"])
@pytest.mark.parametrize("n,d", [(64, 4096), (3, 1001), (300, 512), (2, 16384), (20000, 1024), (8200, 5120)])
def test_layer_norm_bf16(gpu, stream, n, d, wdt):
    rng = np.random.default_rng(n * 7 + d)
    xb = to_bf16(rng.standard_normal((n, d)).astype(f32) * f32(1.5) + f32(0.25))
    s, b = rng.uniform(0.5, 1.5, d).astype(f32), rng.uniform(-1, 1, d).astype(f32)
    if wdt == "bf16":
        sb, bb = to_bf16(s), to_bf16(b)
        s, b = from_bf16(sb), from_bf16(bb)
        wl = TensorLayout(dt.BF16, [d], [2])
    else:
        sb, bb = s, b
        wl = TensorLayout(dt.F32, [d], [4])
    xd, sd, bd, yd = gpu.from_host(xb), gpu.from_host(sb), gpu.from_host(bb), gpu.malloc(xb.nbytes)
    op = ophip.LayerNorm(gpu)
    args = ophip.LayerNormArgs(L2(dt.BF16, n, d), yd, L2(dt.BF16, n, d), xd, wl, sd, wl, bd, 1e-5)
    op.scheme(args, 0)
    say("layer_norm bf16 n=%d d=%d w=%s" % (n, d, wdt))
    op.launch(args, None, stream)
    y = from_bf16(gpu.to_host(yd, u16, n * d, stream=stream)).reshape(n, d).astype(f64)
    x = from_bf16(xb).astype(f64)
    e = x.mean(axis=1, keepdims=True)
    k = 1.0 / (np.sqrt((x * x).mean(axis=1, keepdims=True) - e * e) + 1e-5)
    ref = (x - e) * (s.astype(f64) * k) + b.astype(f64)
    # the difference x - e and the sum with the bias cancel: the f32 result is good to a few 2^-24 of the larger terms
    slack = (np.abs(x - e) * np.abs(s) * k + np.abs(b)) * 2.0 ** -20
    assert (np.abs(y - ref) <= one_step(ref) + slack).all(), (np.abs(y - ref) - one_step(ref) - slack).max()


@pytest.mark.parametrize("adt,wdt", [("f16", "bf16"), ("bf16", "f16"), ("f32", "f16"), ("f32", "bf16")])
@pytest.mark.parametrize("n,d", [(16, 4096), (3, 1001), (64, 24)])
def test_layer_norm_mixed_row_and_parameter_types(gpu, stream, n, d, adt, wdt):
    """The pairs of f16 / bf16 / f32 that have no vector kernel and do not exist in the reference's CPU backend (its CUDA
    backend compiles layer_norm for any pair of named types, layer_norm/cuda/mod.rs:158-159): parity unpinned against
    the reference; checked against the formula in f64 (the reference's: the standard deviation plus epsilon)."""
    rng = np.random.default_rng(n * 5 + d)
    enc = {"f16": lambda v: v.astype(np.float16), "bf16": to_bf16, "f32": lambda v: v.astype(f32)}
    dec = {"f16": lambda v: v.astype(f64), "bf16": lambda v: from_bf16(v).astype(f64), "f32": lambda v: v.astype(f64)}
    code = {"f16": dt.F16, "bf16": dt.BF16, "f32": dt.F32}
    xa = enc[adt](rng.standard_normal((n, d)).astype(f32) * f32(1.5) + f32(0.25))
    sa, ba = enc[wdt](rng.uniform(0.5, 1.5, d).astype(f32)), enc[wdt](rng.uniform(-1, 1, d).astype(f32))
    xd, sd, bd, yd = gpu.from_host(xa), gpu.from_host(sa), gpu.from_host(ba), gpu.malloc(xa.nbytes)
    wl = TensorLayout(code[wdt], [d], [sa.itemsize])
    op = ophip.LayerNorm(gpu)
    args = ophip.LayerNormArgs(L2(code[adt], n, d), yd, L2(code[adt], n, d), xd, wl, sd, wl, bd, 1e-5)
    op.scheme(args, 0)
    say("layer_norm n=%d d=%d rows %s parameters %s" % (n, d, adt, wdt))
    op.launch(args, None, stream)
    y = dec[adt](gpu.to_host(yd, xa.dtype, n * d, stream=stream).reshape(n, d))
    x, s, b = dec[adt](xa), dec[wdt](sa), dec[wdt](ba)
    e = x.mean(axis=1, keepdims=True)
    k = 1.0 / (np.sqrt((x * x).mean(axis=1, keepdims=True) - e * e) + 1e-5)
    ref = (x - e) * (s * k) + b
    step = {"f16": 2.0 ** -10, "bf16": 2.0 ** -7, "f32": 2.0 ** -18}[adt]
    slack = (np.abs(x - e) * np.abs(s) * k + np.abs(b)) * 2.0 ** -18 + (2.0 ** -24 if adt == "f16" else 1e-30)
    assert (np.abs(y - ref) <= np.abs(ref) * step + slack).all(), (np.abs(y - ref) - np.abs(ref) * step - slack).max()


def test_layer_norm_refuses_the_pairs_it_has_no_kernel_for(gpu, stream):
    """f64 mixed with a narrower type and non-floating types."""
    op = ophip.LayerNorm(gpu)
    for adt, wdt in ((dt.F64, dt.F32), (dt.F32, dt.F64), (dt.F16, dt.F64), (dt.U32, dt.U32), (dt.F16, dt.I32)):
        wl = TensorLayout(wdt, [64], [ophip.dtype_nbytes(wdt)])
        args = ophip.LayerNormArgs(L2(adt, 4, 64), None, L2(adt, 4, 64), None, wl, None, wl, None, 1e-5)
        with pytest.raises(ophip.LaunchError) as e:
            op.launch(args, None, stream)
        assert e.value.kind == "TypeNotSupport", (adt, wdt)


@pytest.mark.parametrize("shape", [(16, 4096), (3, 5, 7), (1,), (2, 1000, 33), (4100, 8192)])
def test_add_bf16_every_bit(gpu, stream, shape):
    rng = np.random.default_rng(sum(shape))
    a, b = (to_bf16(rng.standard_normal(shape).astype(f32)) for _ in range(2))
    ad, bd, cd = gpu.from_host(a), gpu.from_host(b), gpu.malloc(a.nbytes)
    lay = TensorLayout.new_contiguous(dt.BF16, list(shape))
    op = ophip.Add(gpu)
    args = ophip.AddArgs(lay, cd, lay, ad, lay, bd)
    op.scheme(args, 0)
    say("add bf16 %s" % (shape,))
    op.launch(args, None, stream)
    out = gpu.to_host(cd, u16, a.size, stream=stream).reshape(shape)
    assert np.array_equal(out, to_bf16(from_bf16(a) + from_bf16(b)))


def test_add_bf16_broadcast_row_element_wise(gpu, stream):
    rng = np.random.default_rng(11)
    x, bias = to_bf16(rng.standard_normal((6, 50)).astype(f32)), to_bf16(rng.standard_normal(50).astype(f32))
    xd, bd, cd = gpu.from_host(x), gpu.from_host(bias), gpu.malloc(x.nbytes)
    lay = TensorLayout.new_contiguous(dt.BF16, [6, 50])
    op = ophip.Add(gpu)
    op.launch(ophip.AddArgs(lay, cd, lay, xd, TensorLayout(dt.BF16, [6, 50], [0, 2]), bd), None, stream)
    out = gpu.to_host(cd, u16, x.size, stream=stream).reshape(6, 50)
    assert np.array_equal(out, to_bf16(from_bf16(x) + from_bf16(bias)[None, :]))


@pytest.mark.parametrize("idt", [np.uint32, np.uint64])
@pytest.mark.parametrize("b,m,n,k", [(2, 16, 4096, 100), (1, 5, 77, 9), (3, 4, 8, 4)])
def test_add_rows_bf16_every_bit(gpu, stream, b, m, n, k, idt):
    rng = np.random.default_rng(b + m + n + k)
    dst = to_bf16(rng.standard_normal((b, m, n)).astype(f32))
    src = to_bf16(rng.standard_normal((k, n)).astype(f32))
    idx = rng.integers(0, k, (b, m)).astype(idt)
    dd, sd, idd = gpu.from_host(dst), gpu.from_host(src), gpu.from_host(idx)
    op = ophip.AddRows(gpu)
    args = ophip.AddRowsArgs(TensorLayout.new_contiguous(dt.BF16, [b, m, n]), dd, TensorLayout.new_contiguous(dt.BF16, [k, n]), sd,
                             TensorLayout.of(idx), idd)
    op.scheme(args, 0)
    say("add_rows bf16 %s idx=%s" % ((b, m, n, k), idt.__name__))
    op.launch(args, None, stream)
    out = gpu.to_host(dd, u16, dst.size, stream=stream).reshape(b, m, n)
    assert np.array_equal(out, to_bf16(from_bf16(dst) + from_bf16(src)[idx.astype(np.int64)]))


# ---------------------------------------- rope, softmax, swiglu, gelu ----
# Neither backend of the reference has bf16 for these four (rope/cuda/mod.rs:94, fuesd_softmax/cuda/mod.rs:75,
# swiglu/cuda/mod.rs:69 and gelu's check for F16; the CPU backend lists f16, f32, f64): parity unpinned.  They are the f16
# kernels on bf16 elements, so that a bf16 model's layer runs end to end; checked against f64 within one bf16 step.

@pytest.mark.parametrize("n,d", [(16, 11008), (3, 1001), (1, 8), (9000, 4096)])
def test_swiglu_and_gelu_bf16(gpu, stream, n, d):
    rng = np.random.default_rng(n + d)
    g, u = to_bf16(rng.standard_normal((n, d)).astype(f32) * f32(2)), to_bf16(rng.standard_normal((n, d)).astype(f32))
    gd, ud = gpu.from_host(g), gpu.from_host(u)
    lay = L2(dt.BF16, n, d)
    say("swiglu bf16 n=%d d=%d" % (n, d))
    ophip.Swiglu(gpu).launch(ophip.SwigluArgs(lay, gd, lay, ud), None, stream)
    a, b = from_bf16(g).astype(f64), from_bf16(u).astype(f64)
    ref = a / (1 + np.exp(-a)) * b
    y = from_bf16(gpu.to_host(gd, u16, n * d, stream=stream)).reshape(n, d).astype(f64)
    assert (np.abs(y - ref) <= one_step(ref) + 1e-6).all(), np.abs(y - ref).max()
    xd = gpu.from_host(g)
    say("gelu bf16 n=%d d=%d" % (n, d))
    ophip.Gelu(gpu).launch(ophip.GeluArgs(lay, xd), None, stream)
    ref = 0.5 * a * (1 + np.tanh(np.sqrt(2 / np.pi) * (a + 0.044715 * a ** 3)))
    y = from_bf16(gpu.to_host(xd, u16, n * d, stream=stream)).reshape(n, d).astype(f64)
    assert (np.abs(y - ref) <= one_step(ref) + 1e-6).all(), np.abs(y - ref).max()


@pytest.mark.parametrize("pdt", [np.uint32, np.uint64])
@pytest.mark.parametrize("shape", [(16, 64, 128), (7, 3, 64), (5, 4, 20), (512, 32, 128), (4099, 8, 128)])
def test_rope_bf16(gpu, stream, shape, pdt):
    import oracle
    rng = np.random.default_rng(sum(shape))
    tb = to_bf16(rng.standard_normal(shape).astype(f32))
    pos = rng.integers(0, 4096, shape[0]).astype(pdt)
    td, pd = gpu.from_host(tb), gpu.from_host(pos)
    nt, nh, dh = shape
    t_lay = TensorLayout(dt.BF16, list(shape), [nh * dh * 2, dh * 2, 2])
    empty = TensorLayout(dt.BF16, [0, dh], [dh * 2, 2])
    say("rope bf16 %s %s" % (shape, np.dtype(pdt).name))
    ophip.Rope(gpu).launch(ophip.RopeArgs(t_lay, td, TensorLayout.of(pos), pd, empty, None, empty, None, 1e4), None, stream)
    y = from_bf16(gpu.to_host(td, u16, tb.size, stream=stream)).reshape(shape).astype(f64)
    ref = oracle.rope(from_bf16(tb).copy(), pos, 1e4).astype(f64)   # the oracle's f32 path on the same numbers
    # |a c - b s| is at most the pair's norm: one bf16 step of that
    norm = np.sqrt((from_bf16(tb).astype(f64).reshape(nt, nh, dh // 2, 2) ** 2).sum(-1, keepdims=True)).repeat(2, -1).reshape(shape)
    assert (np.abs(y - ref) <= norm * 2.0 ** -7 + 1e-6).all(), np.abs(y - ref).max()


@pytest.mark.parametrize("shape,causal", [((32, 16, 2048), True), ((4, 7, 511), True), ((2, 3, 8), False), ((3, 300, 300), True),
                                          ((1, 2, 20000), True), ((1, 1, 70000), False)])
def test_softmax_bf16(gpu, stream, shape, causal):
    rng = np.random.default_rng(sum(shape))
    ab = to_bf16(rng.standard_normal(shape).astype(f32) * f32(2))
    ad = gpu.from_host(ab)
    nh, seq, al = shape
    lay = TensorLayout(dt.BF16, list(shape), [seq * al * 2, al * 2, 2])
    say("softmax bf16 %s causal=%s" % (shape, causal))
    ophip.FusedSoftmax(gpu).launch(ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL if causal else ophip.AttnMask.NONE, lay, ad), None, stream)
    y = from_bf16(gpu.to_host(ad, u16, ab.size, stream=stream)).reshape(shape).astype(f64)
    x = from_bf16(ab).astype(f64)
    if causal:
        keep = np.arange(al)[None, :] <= (al - seq + np.arange(seq))[:, None]
        x = np.where(keep[None], x, -np.inf)
    e = np.exp(x - x.max(-1, keepdims=True))
    ref = e / e.sum(-1, keepdims=True)
    assert (np.abs(y - ref) <= one_step(ref) + 1e-12).all(), (np.abs(y - ref) / one_step(ref)).max()
    if causal:
        assert (y[~np.broadcast_to(keep[None], shape)] == 0).all()


def attention_f64_bf16(q, k, v, causal):
    """softmax(q . k^T / sqrt(dh), mask) . v in f64 on bf16 bit patterns; heads of q share kv heads in groups."""
    nh, seq, dh = q.shape
    nkvh, att, _ = k.shape
    g = nh // nkvh
    kk, vv = np.repeat(from_bf16(k).astype(f64), g, axis=0), np.repeat(from_bf16(v).astype(f64), g, axis=0)
    s = np.einsum("hsd,had->hsa", from_bf16(q).astype(f64), kk) / np.sqrt(dh)
    if causal:
        s = np.where((np.arange(att)[None, :] <= (att - seq + np.arange(seq))[:, None])[None], s, -np.inf)
    pr = np.exp(s - s.max(-1, keepdims=True))
    return np.einsum("hsa,had->hsd", pr / pr.sum(-1, keepdims=True), vv)


@pytest.mark.parametrize("fused", ["0", "1"])
def test_attention_bf16_composite_and_one_pass(gpu, stream, monkeypatch, fused):
    """mat_mul, softmax and rearrange all take bf16, so the composite of launches does (OPHIP_ATTN_FUSED=0); the one-pass
    kernel is built on bf16 elements as well (=1): both against f64."""
    monkeypatch.setenv("OPHIP_ATTN_FUSED", fused)
    rng = np.random.default_rng(31)
    nh, nkvh, seq, att, dh = 8, 2, 40, 136, 64
    q, k, v = (to_bf16(rng.standard_normal(s).astype(f32)) for s in ((nh, seq, dh), (nkvh, att, dh), (nkvh, att, dh)))
    qd, kd, vd, od = gpu.from_host(q), gpu.from_host(k), gpu.from_host(v), gpu.malloc(q.nbytes)
    c = lambda *s: TensorLayout.new_contiguous(dt.BF16, list(s))
    op = ophip.Attention(gpu)
    args = ophip.AttentionArgs(c(nh, seq, dh), qd, c(nkvh, att, dh), kd, c(nkvh, att, dh), vd, c(nh, seq, dh), od, ophip.AttnMask.CAUSAL)
    ws = gpu.malloc(max(op.scheme(args, 1 << 30), 16))
    say("attention bf16 fused=%s" % fused)
    op.launch(args, ws, stream)
    y = from_bf16(gpu.to_host(od, u16, q.size, stream=stream)).reshape(nh, seq, dh).astype(f64)
    ref = attention_f64_bf16(q, k, v, True)
    # the composite rounds scores and probabilities to bf16 between the launches: a few steps of the output's scale;
    # the one pass keeps them in f32 and rounds the probabilities once, for the second product
    steps = 4 if fused == "0" else 1.5
    assert np.abs(y - ref).max() <= steps * 2.0 ** -7 * np.abs(ref).max(), np.abs(y - ref).max()


@pytest.mark.parametrize("split", ["0", "1"])
@pytest.mark.parametrize("nh,nkvh,seq,att,dh,causal", [
    (32, 32, 512, 512, 128, True),     # a prefill step
    (8, 2, 300, 700, 64, True),        # grouped heads, a cache before the rows, ragged last block and tile
    (4, 4, 129, 129, 128, True),       # one row into the second block
    (6, 3, 100, 333, 64, False),       # no mask
    (2, 1, 1000, 1000, 128, True),
])
def test_attention_bf16_one_pass_shapes(gpu, stream, monkeypatch, split, nh, nkvh, seq, att, dh, causal):
    """The one-pass kernel's bf16 build, both of its workgroup shapes (OPHIP_ATTN_KEYSPLIT), against f64; q, left in
    place by the operator when o is another buffer and the heads do not merge with the tokens, is overwritten with the
    result when they do (contiguous q), as the reference's composite does."""
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "1")
    monkeypatch.setenv("OPHIP_ATTN_KEYSPLIT", split)
    rng = np.random.default_rng(nh * seq + att)
    q, k, v = (to_bf16(rng.standard_normal(s).astype(f32)) for s in ((nh, seq, dh), (nkvh, att, dh), (nkvh, att, dh)))
    qd, kd, vd, od = gpu.from_host(q), gpu.from_host(k), gpu.from_host(v), gpu.malloc(q.nbytes)
    gpu.memset(od, 0)
    c = lambda *s: TensorLayout.new_contiguous(dt.BF16, list(s))
    mask = ophip.AttnMask.CAUSAL if causal else ophip.AttnMask.NONE
    op = ophip.Attention(gpu)
    args = ophip.AttentionArgs(c(nh, seq, dh), qd, c(nkvh, att, dh), kd, c(nkvh, att, dh), vd, c(nh, seq, dh), od, mask)
    ws = gpu.malloc(max(op.scheme(args, 1 << 30), 16))
    say("attention bf16 one pass split=%s nh=%d nkvh=%d seq=%d att=%d dh=%d causal=%s" % (split, nh, nkvh, seq, att, dh, causal))
    op.launch(args, ws, stream)
    yb = gpu.to_host(od, u16, q.size, stream=stream).reshape(nh, seq, dh)
    ref = attention_f64_bf16(q, k, v, causal)
    y = from_bf16(yb).astype(f64)
    assert np.abs(y - ref).max() <= 1.5 * 2.0 ** -7 * np.abs(ref).max(), np.abs(y - ref).max()
    assert np.array_equal(gpu.to_host(qd, u16, q.size, stream=stream).reshape(nh, seq, dh), yb)


@pytest.mark.parametrize("nh,nkvh,seq,dh,buf,pos", [(32, 32, 16, 128, 2048, 2032), (32, 8, 1, 128, 4096, 4095), (32, 4, 7, 64, 1500, 1017),
                                                    (8, 8, 16, 64, 700, 0), (3, 3, 33, 64, 100, 10)])
def test_attention_kv_cached_bf16_one_pass(gpu, stream, nh, nkvh, seq, dh, buf, pos):
    """attention_kv_cached on bf16: decode shapes on the one-pass kernel's bf16 build.  o against f64 over the cache's
    first pos rows and the new ones; the appended cache rows bit for bit, the rest of the caches untouched."""
    rng = np.random.default_rng(nh + buf + pos)
    mk = lambda *s: to_bf16(rng.standard_normal(s).astype(f32))
    q, k, v, kc, vc = mk(nh, seq, dh), mk(nkvh, seq, dh), mk(nkvh, seq, dh), mk(nkvh, buf, dh), mk(nkvh, buf, dh)
    qd, kd, vd, kcd, vcd = (gpu.from_host(a) for a in (q, k, v, kc, vc))
    od = gpu.malloc(q.nbytes)
    c = lambda *s: TensorLayout.new_contiguous(dt.BF16, list(s))
    op = ophip.AttnKVCached(gpu)
    args = ophip.AttnKVCachedArgs(c(nh, seq, dh), qd, c(nkvh, seq, dh), kd, c(nkvh, seq, dh), vd, c(nh, seq, dh), od,
                                  c(nkvh, buf, dh), kcd, c(nkvh, buf, dh), vcd, ophip.AttnMask.CAUSAL, pos)
    ws = gpu.malloc(max(op.scheme(args, 1 << 30), 16))
    say("attention_kv_cached bf16 nh=%d nkvh=%d seq=%d dh=%d buf=%d pos=%d" % (nh, nkvh, seq, dh, buf, pos))
    op.launch(args, ws, stream)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    kc_ref[:, pos:pos + seq], vc_ref[:, pos:pos + seq] = k, v
    assert np.array_equal(gpu.to_host(kcd, u16, kc.size, stream=stream).reshape(kc.shape), kc_ref)
    assert np.array_equal(gpu.to_host(vcd, u16, vc.size, stream=stream).reshape(vc.shape), vc_ref)
    y = from_bf16(gpu.to_host(od, u16, q.size, stream=stream)).reshape(nh, seq, dh).astype(f64)
    ref = attention_f64_bf16(q, kc_ref[:, :pos + seq], vc_ref[:, :pos + seq], True)
    assert np.abs(y - ref).max() <= 1.5 * 2.0 ** -7 * np.abs(ref).max(), np.abs(y - ref).max()


def test_types_no_kernel_takes_are_refused(gpu, stream):
    U = dt.U16
    c = lambda *s: TensorLayout.new_contiguous(U, list(s))
    with pytest.raises(ophip.LaunchError) as e:
        ophip.Swiglu(gpu).launch(ophip.SwigluArgs(c(4, 8), None, c(4, 8), None), None, stream)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        ophip.Gelu(gpu).launch(ophip.GeluArgs(c(4, 8), None), None, stream)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        ophip.FusedSoftmax(gpu).scheme(ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL, c(1, 4, 4), None), 0)
    assert e.value.kind == "TypeNotSupport"


# --------------------------------------------------------------- mat_mul ----
# Neither backend of the reference multiplies bf16 (mat_mul/cuda/mod.rs:73 checks for F16, the CPU backend lists f16, f32,
# f64): parity unpinned.  The kernels are the f16 kernels compiled on bf16 elements; what is checked is the product in f64
# within one bf16 step of the result plus the f32 accumulation's share, and -- on operands whose products and sums are
# exact in f32 -- every bit of the result, beside the f16 build on the same numbers.

def layout_of_view(dtype, view):
    """Layout of a numpy view over 2-byte elements, with the given element type."""
    return TensorLayout(dtype, list(view.shape), list(view.strides))


def base_ptr(mem, view, buf):
    return mem.ptr + (view.__array_interface__["data"][0] - buf.__array_interface__["data"][0])


def run_mm_bits(gpu, stream, dtype, cv, cbuf, av, abuf, bv, bbuf, alpha, beta, op=None):
    ad, bd, cd = gpu.from_host(abuf), gpu.from_host(bbuf), gpu.from_host(cbuf)
    op = op or ophip.MatMul(gpu)
    args = ophip.MatMulArgs(layout_of_view(dtype, cv), base_ptr(cd, cv, cbuf), beta, layout_of_view(dtype, av), base_ptr(ad, av, abuf),
                            layout_of_view(dtype, bv), base_ptr(bd, bv, bbuf), alpha)
    what = op.describe(args)
    ws = gpu.malloc(max(op.scheme(args, 1 << 40), 16))
    op.launch(args, ws, stream)
    out = gpu.to_host(cd, u16, cbuf.size, stream=stream).reshape(cbuf.shape)
    return out, what


def views(bt, m, n, k, ta, tb, tc, rng, scale_b=0.05):
    a = to_bf16(rng.standard_normal((bt, k, m) if ta else (bt, m, k)).astype(f32) * f32(0.5))
    b = to_bf16(rng.standard_normal((bt, n, k) if tb else (bt, k, n)).astype(f32) * f32(scale_b))
    c = to_bf16(rng.standard_normal((bt, n, m) if tc else (bt, m, n)).astype(f32))
    return (a.transpose(0, 2, 1) if ta else a, a), (b.transpose(0, 2, 1) if tb else b, b), (c.transpose(0, 2, 1) if tc else c, c)


def check_bf16_product(out_view, c0, av, bv, alpha, beta, what):
    alpha_r, beta_r = from_bf16(to_bf16(np.array([alpha, beta], f32))).astype(f64)
    prod = np.matmul(from_bf16(av).astype(f64), from_bf16(bv).astype(f64))
    ref = alpha_r * prod + (beta_r * from_bf16(c0).astype(f64) if beta != 0 else 0.0)
    y = from_bf16(out_view).astype(f64)
    k = av.shape[-1]
    # one bf16 step of the result, and the f32 accumulation (k terms of the size of the row's and column's norms)
    norm = np.sqrt(np.matmul(from_bf16(av).astype(f64) ** 2, from_bf16(bv).astype(f64) ** 2))
    tol = np.abs(ref) * 2.0 ** -7 + norm * abs(alpha_r) * np.sqrt(k) * 2.0 ** -22 + 1e-30
    bad = np.abs(y - ref) > tol
    assert not bad.any(), "%s: %d of %d off, worst %g" % (what, bad.sum(), bad.size, (np.abs(y - ref) / tol).max())


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("tc", [False, True])
@pytest.mark.parametrize("m,n,k,bt", [(16, 256, 512, 3), (40, 136, 72, 2), (3, 5, 7, 2), (130, 70, 33, 1), (256, 512, 96, 2), (128, 384, 64, 1),
                                      (512, 768, 192, 1), (509, 1536, 1024, 1)])
def test_mat_mul_bf16_all_layouts(gpu, stream, ta, tb, tc, m, n, k, bt):
    rng = np.random.default_rng(m + n + k + 4 * ta + 2 * tb + tc)
    (av, a), (bv, b), (cv, c) = views(bt, m, n, k, ta, tb, tc, rng, scale_b=1.0 / np.sqrt(k))
    say("mat_mul bf16 ta=%s tb=%s tc=%s %dx%dx%d x%d" % (ta, tb, tc, m, n, k, bt))
    out, what = run_mm_bits(gpu, stream, dt.BF16, cv, c, av, a, bv, b, 0.75, 0.5)
    ov = out.transpose(0, 2, 1) if tc else out
    check_bf16_product(ov, cv, av, bv, 0.75, 0.5, "mat_mul bf16 " + what)


@pytest.mark.parametrize("name,bt,m,n,k,tb", [("qkv", 1, 16, 12288, 4096, False), ("qk_t", 32, 16, 2048, 128, True), ("pv", 32, 16, 128, 2048, False),
                                              ("o_proj", 1, 16, 4096, 4096, False), ("gate_up", 1, 16, 22016, 4096, False),
                                              ("down", 1, 16, 4096, 11008, False), ("down [N,K]", 1, 16, 4096, 11008, True),
                                              ("prefill", 1, 512, 4096, 4096, False), ("square", 1, 1024, 1024, 1024, True)])
def test_mat_mul_bf16_decode_layer_shapes(gpu, stream, name, bt, m, n, k, tb):
    rng = np.random.default_rng(bt + m + n + k)
    (av, a), (bv, b), (cv, c) = views(bt, m, n, k, False, tb, False, rng, scale_b=0.02)
    say("mat_mul bf16 %s" % name)
    out, what = run_mm_bits(gpu, stream, dt.BF16, cv, c, av, a, bv, b, 1.0, 0.0)
    say("  " + what)
    assert "generic" not in what
    check_bf16_product(out, cv, av, bv, 1.0, 0.0, "mat_mul bf16 %s (%s)" % (name, what))


@pytest.mark.parametrize("m,n,k,tb", [(16, 4096, 4096, False), (16, 1024, 4096, True), (48, 512, 2048, False), (256, 256, 4096, False),
                                      (384, 640, 1024, True), (100, 72, 520, False)])
def test_mat_mul_bf16_and_f16_builds_give_every_bit_on_exact_sums(gpu, stream, m, n, k, tb):
    """Operands k / 16 with |k| <= 32 are f16 and bf16 numbers alike, their products and any sum of up to 4096 of them are
    exact in f32 in any order: both builds must return the correctly rounded exact result in their type."""
    rng = np.random.default_rng(m + n + k)
    ai = rng.integers(-32, 33, (1, m, k))
    bi = rng.integers(-32, 33, (1, n, k) if tb else (1, k, n))
    exact = np.matmul(ai, bi.transpose(0, 2, 1) if tb else bi).astype(f64) / 256.0
    assert np.abs(exact).max() * 256 < 2 ** 24
    for dtype, enc, dec in ((dt.BF16, to_bf16, from_bf16), (dt.F16, lambda x: x.astype(np.float16).view(u16), lambda u: u.view(np.float16).astype(f32))):
        a, b = enc((ai / 16.0).astype(f32)), enc((bi / 16.0).astype(f32))
        c = np.zeros((1, m, n), u16)
        bv = b.transpose(0, 2, 1) if tb else b
        say("mat_mul exact sums %s %dx%dx%d" % ("bf16" if dtype == dt.BF16 else "f16", m, n, k))
        out, what = run_mm_bits(gpu, stream, dtype, c, c, a, a, bv, b, 1.0, 0.0)
        assert "generic" not in what or (k % 8)
        assert np.array_equal(out, enc(exact.astype(f32))), what


def test_mat_mul_bf16_scalars_round_to_bf16_and_beta_zero_never_reads_c(gpu, stream):
    rng = np.random.default_rng(9)
    (av, a), (bv, b), (cv, c) = views(1, 16, 256, 512, False, False, False, rng)
    nan = np.full(c.shape, 0x7FC0, u16)
    out, _ = run_mm_bits(gpu, stream, dt.BF16, nan, nan, av, a, bv, b, 1.0, 0.0)
    assert not np.isnan(from_bf16(out)).any()
    # alpha = 1 + 2^-9 rounds to 1 in bf16 (1 + 2^-8 is the tie, which goes to even: also 1)
    out1, _ = run_mm_bits(gpu, stream, dt.BF16, cv, c, av, a, bv, b, 1.0, 0.0)
    out2, _ = run_mm_bits(gpu, stream, dt.BF16, cv, c, av, a, bv, b, 1.0 + 2.0 ** -9, 0.0)
    assert np.array_equal(out1, out2)
