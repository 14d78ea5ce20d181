"""bf16 data on rms_norm, layer_norm, add and add_rows, through the C ABI.

The reference's CUDA backend compiles these four for any pair of named types, bf16 included (handle/cuda/mod.rs:188-210
with rms_norm/cuda/mod.rs:146-147, layer_norm/cuda/mod.rs:158-159, add/cuda/mod.rs:105-123, add_rows/cuda/mod.rs:135-163);
its CPU backend, which the oracle restates, has no bf16 kernel.  PARITY UNPINNED against the reference: what is checked here
is the arithmetic the kernels document -- the f16 kernels' formulas in f32, one rounding to bf16 (nearest even) at the end --
against the same formula in f64 (the norms: within one bf16 step, 2^-7 relative) or in numpy f32 (the sums: every bit)."""
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
@pytest.mark.parametrize("n,d", [(64, 4096), (16, 4096), (3, 1001), (5, 24), (300, 512), (2, 16384), (20000, 2048), (1, 8)])
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


@pytest.mark.parametrize("wdt", ["bf16", "f32"])
@pytest.mark.parametrize("n,d", [(64, 4096), (3, 1001), (300, 512), (2, 16384), (20000, 1024)])
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


def test_bf16_still_refused_where_no_backend_of_the_reference_takes_it(gpu, stream):
    # rope, softmax, swiglu, gelu, mat_mul: the CUDA backend checks for F16 (rope/cuda/mod.rs:94, fuesd_softmax/cuda/mod.rs:75,
    # swiglu/cuda/mod.rs:69, gelu/cuda/mod.rs, mat_mul/cuda/mod.rs:73) and the CPU backend has no bf16
    B = dt.BF16
    c = lambda *s: TensorLayout.new_contiguous(B, list(s))
    with pytest.raises(ophip.LaunchError) as e:
        ophip.Swiglu(gpu).launch(ophip.SwigluArgs(c(4, 8), None, c(4, 8), None), None, stream)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        ophip.Gelu(gpu).launch(ophip.GeluArgs(c(4, 8), None), None, stream)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        ophip.FusedSoftmax(gpu).scheme(ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL, c(1, 4, 4), None), 0)
    assert e.value.kind == "TypeNotSupport"
