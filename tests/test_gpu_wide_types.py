"""f32 and f64 data on the operators whose CPU backend in the reference accepts them (rope/common_cpu/mod.rs:121-126,
fuesd_softmax/common_cpu/mod.rs:76-78, swiglu/common_cpu/mod.rs:74-76, mat_mul/common_cpu/mod.rs:101-103,
layer_norm/common_cpu/mod.rs:94-97, gelu/common_cpu/mod.rs:62-64, add/common_cpu/mod.rs:60-62,
add_rows/common_cpu/mod.rs:99-104), against the oracle, through the C ABI.  The hot path is f16; these types run on plain
scalar kernels that compute in the element's own arithmetic, as the reference does.
Tolerances: f64 results differ from the oracle's only through the device library's exp / tanh / sin / cos / pow (an ulp or
two each) and through the order of a row's sum: relative 1e-12.  f32: relative 2e-5 (softmax rows of up to 5000 terms)."""
import numpy as np
import pytest

import ophip
import oracle
from ophip import TensorLayout, dt

pytestmark = pytest.mark.gpu

f32, f64 = np.float32, np.float64


def say(msg):
    print(msg, flush=True)


@pytest.mark.parametrize("pdt", [np.uint32, np.uint64])
@pytest.mark.parametrize("shape", [(7, 32, 64), (3, 5, 20), (2, 1, 2), (40, 4, 256)])
def test_rope_f64(gpu, stream, shape, pdt):
    rng = np.random.default_rng(sum(shape))
    t = rng.standard_normal(shape)
    pos = rng.integers(0, 4096, shape[0]).astype(pdt)
    td, pd = gpu.from_host(t), gpu.from_host(pos)
    op = ophip.Rope(gpu)
    L = TensorLayout
    empty = L(dt.F64, [0, shape[2]], [8 * shape[2], 8])
    args = ophip.RopeArgs(L.of(t), td, L.of(pos), pd, empty, None, empty, None, 1e4)
    op.scheme(args, 0)
    say("rope f64 %s %s" % (shape, pdt.__name__))
    op.launch(args, None, stream)
    out = gpu.to_host(td, f64, t.size, stream=stream).reshape(shape)
    ref = oracle.rope(t.copy(), pos, 1e4)
    # the angle reaches 4096 rad: sine and cosine carry ang * 2^-53 of the argument's rounding
    np.testing.assert_allclose(out, ref, rtol=0, atol=2e-12)
    norm = lambda x: x.reshape(shape[0], shape[1], -1, 2)
    np.testing.assert_allclose((norm(out) ** 2).sum(-1), (norm(t) ** 2).sum(-1), rtol=1e-13)  # rotations keep pair norms


@pytest.mark.parametrize("dtype", [f32, f64])
@pytest.mark.parametrize("shape,causal", [((32, 7, 511), True), ((2, 3, 8), True), ((1, 1, 1), True), ((2, 4, 1000), False),
                                          ((3, 300, 300), True), ((1, 2, 5000), True)])
def test_softmax_f32_f64(gpu, stream, dtype, shape, causal):
    rng = np.random.default_rng(sum(shape))
    att = (rng.standard_normal(shape) * 2).astype(dtype)
    ad = gpu.from_host(att)
    op = ophip.FusedSoftmax(gpu)
    args = ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL if causal else ophip.AttnMask.NONE, TensorLayout.of(att), ad)
    op.scheme(args, 0)
    say("softmax %s %s causal=%s" % (dtype.__name__, shape, causal))
    op.launch(args, None, stream)
    out = gpu.to_host(ad, dtype, att.size, stream=stream).reshape(shape)
    ref = oracle.fused_softmax(att.copy(), causal=causal)
    np.testing.assert_allclose(out, ref, rtol=2e-5 if dtype is f32 else 1e-12, atol=0)
    nh, seq, al = shape
    if causal:
        for r in range(seq):
            tail = out[:, r, al - seq + r + 1:]
            assert (tail == 0).all() and not np.signbit(tail).any(), "masked tail must be +0"


def test_softmax_f64_strided_rows(gpu, stream):
    rng = np.random.default_rng(3)
    nh, seq, al, ld = 3, 5, 40, 64
    host = rng.standard_normal((seq, nh, ld)) * 2  # heads interleaved, padded rows
    buf = gpu.from_host(host)
    lay = TensorLayout(dt.F64, [nh, seq, al], [ld * 8, nh * ld * 8, 8])
    op = ophip.FusedSoftmax(gpu)
    op.launch(ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL, lay, buf), None, stream)
    out = gpu.to_host(buf, f64, host.size, stream=stream).reshape(host.shape)
    ref = host.copy()
    oracle.fused_softmax(ref.transpose(1, 0, 2)[:, :, :al], causal=True)
    np.testing.assert_allclose(out, ref, rtol=1e-12, atol=0)
    assert np.array_equal(out[:, :, al:], host[:, :, al:])  # the padding was not touched


@pytest.mark.parametrize("n,d,ld", [(5, 77, 200), (16, 1024, 2048), (1, 1, 2)])
def test_swiglu_f64(gpu, stream, n, d, ld):
    rng = np.random.default_rng(n + d)
    host = rng.standard_normal((n, ld)) * 2
    host[0, 0] = -800.0  # exp(800) overflows to inf: the sigmoid is exactly 0
    buf = gpu.from_host(host)
    lay = TensorLayout(dt.F64, [n, d], [ld * 8, 8])
    op = ophip.Swiglu(gpu)
    say("swiglu f64 n=%d d=%d" % (n, d))
    op.launch(ophip.SwigluArgs(lay, buf.ptr, lay, buf.ptr + d * 8), None, stream)
    out = gpu.to_host(buf, f64, host.size, stream=stream).reshape(host.shape)
    ref = host.copy()
    oracle.swiglu(ref[:, :d], ref[:, d:2 * d])
    np.testing.assert_allclose(out, ref, rtol=1e-14, atol=1e-300)
    assert np.array_equal(out[:, d:], host[:, d:]) and out[0, 0] == 0


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("bt,m,n,k,alpha,beta", [(1, 5, 7, 3, 1.0, 0.0), (2, 70, 65, 130, 0.5, 1.0), (1, 128, 1, 257, -1.25, 0.25)])
def test_mat_mul_f64(gpu, stream, ta, tb, bt, m, n, k, alpha, beta):
    rng = np.random.default_rng(m + n + k + 2 * ta + tb)
    a = rng.standard_normal((bt, k, m) if ta else (bt, m, k))
    b = rng.standard_normal((bt, n, k) if tb else (bt, k, n))
    c = rng.standard_normal((bt, m, n))
    av = a.transpose(0, 2, 1) if ta else a
    bv = b.transpose(0, 2, 1) if tb else b
    cd, ad, bd = gpu.from_host(c), gpu.from_host(a), gpu.from_host(b)
    L = TensorLayout
    op = ophip.MatMul(gpu)
    args = ophip.MatMulArgs(L.of(c), cd, beta, L.of(av), ad, L.of(bv), bd, alpha)
    assert op.describe(args) == "generic" and op.scheme(args, 1 << 30) == 0
    say("mat_mul f64 ta=%s tb=%s %dx%dx%d" % (ta, tb, m, n, k))
    op.launch(args, None, stream)
    out = gpu.to_host(cd, f64, c.size, stream=stream).reshape(c.shape)
    ref = c.copy()
    oracle.mat_mul(ref, beta, av, bv, alpha)
    # the same k-ascending sum; the device may fuse a multiply and an add where the oracle rounds twice
    np.testing.assert_allclose(out, ref, rtol=1e-13, atol=1e-13 * np.sqrt(k))
    np.testing.assert_allclose(out, alpha * (av @ bv) + beta * c, rtol=1e-12, atol=1e-12 * np.sqrt(k))


@pytest.mark.parametrize("n,d", [(6, 300), (3, 4097), (1, 1)])
def test_layer_norm_f64(gpu, stream, n, d):
    rng = np.random.default_rng(n * 7 + d)
    x = rng.standard_normal((n, d)) * 1.5 + 0.25
    s, b = rng.uniform(0.5, 1.5, d), rng.uniform(-1, 1, d)
    xd, sd, bd, yd = gpu.from_host(x), gpu.from_host(s), gpu.from_host(b), gpu.malloc(x.nbytes)
    lay = TensorLayout.of
    op = ophip.LayerNorm(gpu)
    args = ophip.LayerNormArgs(lay(x), yd, lay(x), xd, lay(s), sd, lay(b), bd, 1e-5)
    op.scheme(args, 0)
    say("layer_norm f64 n=%d d=%d" % (n, d))
    op.launch(args, None, stream)
    y = gpu.to_host(yd, f64, n * d, stream=stream).reshape(n, d)
    ref = oracle.layer_norm(np.empty_like(x), x, s, b, 1e-5)
    if d == 1:
        assert np.array_equal(y, b.reshape(1, 1) + 0 * x)  # x - mean = 0: the bias comes back exactly
    else:
        # e2 - e * e cancels a few digits: the order of the two row sums shows at about 1e-13 relative
        np.testing.assert_allclose(y, ref, rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("n,d", [(5, 77), (40, 1000)])
def test_gelu_f64(gpu, stream, n, d):
    rng = np.random.default_rng(n + d)
    x = rng.standard_normal((n, d)) * 2.5
    x[0, :4] = [0.0, -0.0, 30.0, -30.0]
    xd = gpu.from_host(x)
    op = ophip.Gelu(gpu)
    op.launch(ophip.GeluArgs(TensorLayout.of(x), xd), None, stream)
    y = gpu.to_host(xd, f64, n * d, stream=stream).reshape(n, d)
    np.testing.assert_allclose(y, oracle.gelu(x.copy()), rtol=1e-13, atol=1e-15)
    assert y[0, 0] == 0 and y[0, 2] == 30.0 and y[0, 3] == 0


@pytest.mark.parametrize("shape", [(1, 768), (3, 5, 7), (1000, 33)])
def test_add_f64(gpu, stream, shape):
    rng = np.random.default_rng(sum(shape))
    a, b = rng.standard_normal(shape), rng.standard_normal(shape)
    c = np.zeros(shape)
    cd, ad, bd = gpu.from_host(c), gpu.from_host(a), gpu.from_host(b)
    lay = TensorLayout.of
    op = ophip.Add(gpu)
    args = ophip.AddArgs(lay(c), cd, lay(a), ad, lay(b), bd)
    op.scheme(args, 0)
    op.launch(args, None, stream)
    out = gpu.to_host(cd, f64, c.size, stream=stream).reshape(shape)
    assert np.array_equal(out, oracle.add(c, a, b)) and np.array_equal(out, a + b)
    # a row broadcast over the rows of a permuted view
    if len(shape) == 2:
        row = rng.standard_normal(shape[1])
        rd = gpu.from_host(row)
        bl = TensorLayout(dt.F64, list(shape), [0, 8])
        op.launch(ophip.AddArgs(lay(c), cd, lay(a), ad, bl, rd), None, stream)
        out = gpu.to_host(cd, f64, c.size, stream=stream).reshape(shape)
        assert np.array_equal(out, a + row[None, :])


@pytest.mark.parametrize("batch,m,n,k,idt", [(2, 5, 100, 9, np.uint32), (1, 3, 64, 4, np.uint64)])
def test_add_rows_f64(gpu, stream, batch, m, n, k, idt):
    rng = np.random.default_rng(batch + m + n)
    dst = rng.standard_normal((batch, m, n))
    src = rng.standard_normal((k, n))
    idx = rng.integers(0, k, (batch, m)).astype(idt)
    dd, sd, idd = gpu.from_host(dst), gpu.from_host(src), gpu.from_host(idx)
    lay = TensorLayout.of
    op = ophip.AddRows(gpu)
    args = ophip.AddRowsArgs(lay(dst), dd, lay(src), sd, lay(idx), idd)
    op.scheme(args, 0)
    op.launch(args, None, stream)
    out = gpu.to_host(dd, f64, dst.size, stream=stream).reshape(dst.shape)
    assert np.array_equal(out, oracle.add_rows(dst.copy(), src, idx))


def test_null_bases_are_refused_before_any_launch(gpu, stream):
    """A launch whose arguments pass every check but carry a null base address returns ArgsNotSupport."""
    L = TensorLayout
    c = lambda d_, *s: L.new_contiguous(d_, list(s))
    cases = [
        (ophip.Swiglu(gpu), ophip.SwigluArgs(c(dt.F64, 4, 8), None, c(dt.F64, 4, 8), None)),
        (ophip.Gelu(gpu), ophip.GeluArgs(c(dt.F64, 4, 8), None)),
        (ophip.Add(gpu), ophip.AddArgs(c(dt.F64, 4, 8), None, c(dt.F64, 4, 8), None, c(dt.F64, 4, 8), None)),
        (ophip.AddRows(gpu), ophip.AddRowsArgs(c(dt.F64, 2, 3, 8), None, c(dt.F64, 5, 8), None, c(dt.U32, 2, 3), None)),
        (ophip.LayerNorm(gpu), ophip.LayerNormArgs(c(dt.F64, 4, 8), None, c(dt.F64, 4, 8), None, c(dt.F64, 8), None, c(dt.F64, 8), None, 1e-5)),
        (ophip.FusedSoftmax(gpu), ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL, c(dt.F64, 1, 4, 4), None)),
        (ophip.MatMul(gpu), ophip.MatMulArgs(c(dt.F64, 5, 7), None, 0.0, c(dt.F64, 5, 3), None, c(dt.F64, 3, 7), None, 1.0)),
        (ophip.Rope(gpu), ophip.RopeArgs(c(dt.F64, 4, 2, 16), None, c(dt.U32, 4), None, c(dt.F64, 0, 16), None, c(dt.F64, 0, 16), None, 1e4)),
    ]
    for op, args in cases:
        with pytest.raises(ophip.LaunchError) as e:
            op.launch(args, None, stream)
        assert e.value.kind == "ArgsNotSupport", type(op).__name__
