"""layer_norm, gelu, add and add_rows on the HIP backend against the oracle, through the C ABI.
Shapes follow the reference's device tests (layer_norm/cuda/mod.rs:296-377: n 4, d 2^k;
gelu/cuda/mod.rs:160-208: 1024 x 2048; add/cuda/mod.rs:176-247: 1 x 768;
add_rows/cuda/mod.rs:218-290: batch 1, m 10, n 2048) plus strided, odd and broadcast cases.
add and add_rows are a single f32 addition rounded once: exact."""
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


class Dev:
    """Host bytes mirrored on the device, with numpy views (byte strides) on the host side."""

    def __init__(self, gpu, host):
        self.gpu = gpu
        self.host = np.ascontiguousarray(host).view(np.uint8).reshape(-1).copy()
        self.mem = gpu.from_host(self.host)
        self.ptr = self.mem.ptr

    def back(self, stream):
        return self.gpu.to_host(self.mem, np.uint8, self.host.size, stream=stream)


def view(buf_u8, dtype, shape, strides, offset=0):
    return np.lib.stride_tricks.as_strided(buf_u8[offset:].view(dtype), shape=shape, strides=strides, writeable=True)


# ------------------------------------------------------------ layer_norm ----

@pytest.mark.parametrize("n,d,adt,wdt", [(4, 256, f16, f32), (4, 8192, f16, f32), (64, 4096, f16, f16),
                                         (8200, 5120, f16, f16), (8193, 8192, f16, f32),  # many rows beyond 4096 elements: 16 vectors a lane
                                         (32772, 512, f16, f16), (22003, 768, f16, f32), (16387, 1600, f16, f16), (16390, 2048, f16, f16),  # 8 / 4 / 2 / 2 rows per trip
                                         (3, 16384, f16, f16), (5, 80000, f16, f32), (7, 1001, f16, f16),
                                         (300, 768, f32, f32), (2, 130, f32, f32), (5000, 1024, f16, f16),
                                         (20001, 1024, f16, f16), (17000, 1024, f16, f32)])  # the last two: rows streamed by persistent waves
def test_layer_norm(gpu, stream, n, d, adt, wdt):
    rng = np.random.default_rng(n * 7 + d)
    x = (rng.standard_normal((n, d)).astype(f32) * f32(1.5) + f32(0.25)).astype(adt)
    s, b = rng.uniform(0.5, 1.5, d).astype(wdt), rng.uniform(-1, 1, d).astype(wdt)
    xd, sd, bd, yd = gpu.from_host(x), gpu.from_host(s), gpu.from_host(b), gpu.malloc(x.nbytes)
    lay = TensorLayout.of
    op = ophip.LayerNorm(gpu)
    args = ophip.LayerNormArgs(lay(x), yd, lay(x), xd, lay(s), sd, lay(b), bd, 1e-5)
    op.scheme(args, 0)
    say("layer_norm n=%d d=%d %s/%s" % (n, d, adt.__name__, wdt.__name__))
    op.launch(args, None, stream)
    y = gpu.to_host(yd, adt, n * d, stream=stream).reshape(n, d)
    ref = oracle.layer_norm(np.empty_like(x), x, s, b, 1e-5)
    if adt is f16:
        assert_close_f16(y, ref, "layer_norm")
    else:
        np.testing.assert_allclose(y, ref, rtol=3e-5, atol=3e-6)


def test_layer_norm_strided_rows_and_dynamic_scheme(gpu, stream):
    rng = np.random.default_rng(8)
    n, d, ld = 16, 1024, 3072
    xb = Dev(gpu, normal_f16(rng, (n, ld)))
    yb = Dev(gpu, np.zeros((n, ld), f16))
    s, b = rng.uniform(0.5, 1.5, d).astype(f32), rng.uniform(-1, 1, d).astype(f32)
    sd, bd = gpu.from_host(s), gpu.from_host(b)
    L = TensorLayout
    op = ophip.LayerNorm(gpu)
    # layer_norm/cuda/mod.rs:242-262: n and the strides unknown at scheme time
    assert op.scheme(ophip.LayerNormArgs(L(dt.F16, [None, d], [None, None]), None, L(dt.F16, [None, d], [None, None]),
                                         None, L(dt.F32, [d], [None]), None, L(dt.F32, [d], [None]), None, 1e-5), 0) == 0
    row = L(dt.F16, [n, d], [ld * 2, 2])
    op.launch(ophip.LayerNormArgs(row, yb.ptr + d * 2, row, xb.ptr + 2 * d * 2, L.of(s), sd, L.of(b), bd, 1e-5), None,
              stream)
    out = yb.back(stream)
    xv = view(xb.host, f16, (n, d), (ld * 2, 2), offset=2 * d * 2)
    ref = oracle.layer_norm(np.empty((n, d), f16), xv, s, b, 1e-5)
    assert_close_f16(view(out, f16, (n, d), (ld * 2, 2), offset=d * 2), ref, "layer_norm strided")
    full = out.view(f16).reshape(n, ld)
    assert (full[:, :d] == 0).all() and (full[:, 2 * d:] == 0).all()  # nothing outside the view was written


def test_layer_norm_errors(gpu, stream):
    op = ophip.LayerNorm(gpu)
    c = lambda d_, *s: TensorLayout.new_contiguous(d_, list(s))
    F, W = dt.F16, dt.F32
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.LayerNormArgs(c(F, 4, 8), None, c(F, 4, 8), None, c(W, 8), None, c(W, 9), None, 1e-5), 0)
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.LayerNormArgs(c(F, 4, 8), None, c(F, 4, 8), None, c(W, 8), None, c(F, 8), None, 1e-5), 0)
    assert e.value.kind == "TypeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.LayerNormArgs(c(F, 4, 8), None, c(F, 8), None, c(W, 8), None, c(W, 8), None, 1e-5), 0)
    assert e.value.kind == "RankNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.LayerNormArgs(c(dt.F64, 4, 8), None, c(dt.F64, 4, 8), None, c(F, 8), None, c(F, 8), None, 1e-5), None,
                  stream)
    assert e.value.kind == "TypeNotSupport"


# ------------------------------------------------------------------ gelu ----

@pytest.mark.parametrize("n,d,dtype", [(1024, 2048, f16), (16, 11008, f16), (3, 1001, f16), (5, 77, f32), (1, 8, f16)])
def test_gelu(gpu, stream, n, d, dtype):
    rng = np.random.default_rng(n + d)
    x = (rng.standard_normal((n, d)).astype(f32) * f32(2.5)).astype(dtype)
    x[0, :4] = [0.0, -0.0, 30.0, -30.0][: min(4, d)]
    xd = gpu.from_host(x)
    op = ophip.Gelu(gpu)
    args = ophip.GeluArgs(TensorLayout.of(x), xd)
    assert op.scheme(ophip.GeluArgs(TensorLayout(ophip.NP_DT[np.dtype(dtype)], [None, None], [None, None]), None), 0) == 0
    say("gelu n=%d d=%d %s" % (n, d, dtype.__name__))
    op.launch(args, None, stream)
    y = gpu.to_host(xd, dtype, n * d, stream=stream).reshape(n, d)
    ref = oracle.gelu(x.copy())
    if dtype is f16:
        assert_close_f16(y, ref, "gelu")
    else:
        np.testing.assert_allclose(y, ref, rtol=2e-5, atol=1e-6)
    assert y[0, 0] == 0 and y[0, 2] == dtype(30.0) and y[0, 3] == 0


def test_gelu_strided_rows_and_errors(gpu, stream):
    rng = np.random.default_rng(9)
    n, d, ld = 8, 512, 1536
    buf = Dev(gpu, normal_f16(rng, (n, ld), std=2.0))
    op = ophip.Gelu(gpu)
    op.launch(ophip.GeluArgs(TensorLayout(dt.F16, [n, d], [ld * 2, 2]), buf.ptr + d * 2), None, stream)
    out = buf.back(stream).view(f16).reshape(n, ld)
    ref = buf.host.view(f16).reshape(n, ld).copy()
    oracle.gelu(ref[:, d:2 * d])
    assert_close_f16(out, ref, "gelu strided")
    assert np.array_equal(out[:, :d], ref[:, :d]) and np.array_equal(out[:, 2 * d:], ref[:, 2 * d:])
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.GeluArgs(TensorLayout(dt.F16, [8], [2]), None), 0)
    assert e.value.kind == "RankNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.GeluArgs(TensorLayout(dt.F16, [4, 8], [32, 4]), None), None, stream)
    assert e.value.kind == "StridesNotSupport"


# ------------------------------------------------------------------- add ----

def run_add(gpu, stream, c_view, c_buf, a_view, a_buf, b_view, b_buf):
    cd, ad, bd = Dev(gpu, c_buf), Dev(gpu, a_buf), Dev(gpu, b_buf)
    def off(v, base):  # byte offset of a view inside its buffer; a view of another array would send a wild pointer
        o = v.__array_interface__["data"][0] - base.__array_interface__["data"][0]
        assert 0 <= o < max(base.nbytes, 1), "view does not belong to the buffer"
        return o

    args = ophip.AddArgs(TensorLayout.of(c_view), cd.ptr + off(c_view, c_buf), TensorLayout.of(a_view),
                         ad.ptr + off(a_view, a_buf), TensorLayout.of(b_view), bd.ptr + off(b_view, b_buf))
    op = ophip.Add(gpu)
    op.scheme(args, 0)
    op.launch(args, None, stream)
    return cd.back(stream)


@pytest.mark.parametrize("dtype", [f16, f32])
@pytest.mark.parametrize("shape", [(1, 768), (16, 4096), (3, 5, 7), (1000, 33), (8200, 4096)])  # the last: a sum of more than 64 MiB
def test_add_contiguous(gpu, stream, dtype, shape):
    rng = np.random.default_rng(sum(shape))
    a, b = (rng.standard_normal(shape).astype(f32).astype(dtype) for _ in range(2))
    c = np.zeros(shape, dtype)
    say("add %s %s" % (shape, dtype.__name__))
    out = run_add(gpu, stream, c, c, a, a, b, b).view(dtype).reshape(shape)
    assert np.array_equal(out, oracle.add(c, a, b))


@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.uint16, np.int16, np.uint32, np.int32, np.uint64, np.int64])
def test_add_and_add_rows_integers_wrap_like_the_cuda_kernels(gpu, stream, dtype):
    """The reference's CUDA backend compiles add and add_rows for any named type (add/cuda/mod.rs:105-123,
    add_rows/cuda/mod.rs:135-163): integer sums are modulo 2^bits.  Its CPU backend has no integer kernels, so the
    expected values are numpy's (which wraps the same way)."""
    rng = np.random.default_rng(np.dtype(dtype).itemsize * 7 + (1 if np.dtype(dtype).kind == "i" else 0))
    info = np.iinfo(dtype)
    draw = lambda shape: rng.integers(info.min, info.max, shape, dtype=dtype, endpoint=True)
    a, b = draw((5, 77)), draw((5, 77))
    c = np.zeros((5, 77), dtype)
    say("add %s" % np.dtype(dtype).name)
    out = run_add(gpu, stream, c, c, a, a, b, b).view(dtype).reshape(5, 77)
    assert np.array_equal(out, a + b)   # numpy wraps silently on arrays
    bias = draw((77,))
    at = a.T.copy()  # a stored column-major, read through its transposed view
    out = run_add(gpu, stream, c, c, at.T, at, np.lib.stride_tricks.as_strided(bias, (5, 77), (0, bias.itemsize)), bias)
    assert np.array_equal(out.view(dtype).reshape(5, 77), a + bias[None, :])
    dst, src = draw((2, 3, 40)), draw((6, 40))
    idx = rng.integers(0, 6, (2, 3)).astype(np.uint32)
    dd, sd, idd = gpu.from_host(dst), gpu.from_host(src), gpu.from_host(idx)
    L = TensorLayout
    ophip.AddRows(gpu).launch(ophip.AddRowsArgs(L.of(dst), dd, L.of(src), sd, L.of(idx), idd), None, stream)
    got = gpu.to_host(dd, dtype, dst.size, stream=stream).reshape(dst.shape)
    assert np.array_equal(got, dst + src[idx])


def test_add_and_add_rows_bool(gpu, stream):
    rng = np.random.default_rng(5)
    a, b = rng.integers(0, 2, (4, 50)).astype(np.uint8), rng.integers(0, 2, (4, 50)).astype(np.uint8)
    ad, bd, cd = gpu.from_host(a), gpu.from_host(b), gpu.malloc(a.nbytes)
    lay = TensorLayout.new_contiguous(dt.BOOL, [4, 50])
    ophip.Add(gpu).launch(ophip.AddArgs(lay, cd, lay, ad, lay, bd), None, stream)
    assert np.array_equal(gpu.to_host(cd, np.uint8, a.size, stream=stream).reshape(4, 50), a | b)   # true + true is true
    idx = rng.integers(0, 4, (1, 4)).astype(np.uint32)
    dst = rng.integers(0, 2, (1, 4, 50)).astype(np.uint8)
    dd, idd = gpu.from_host(dst), gpu.from_host(idx)
    ophip.AddRows(gpu).launch(ophip.AddRowsArgs(TensorLayout.new_contiguous(dt.BOOL, [1, 4, 50]), dd, lay, ad,
                                                TensorLayout.of(idx), idd), None, stream)
    assert np.array_equal(gpu.to_host(dd, np.uint8, dst.size, stream=stream).reshape(1, 4, 50), dst | a[idx])


def test_add_permuted_and_broadcast_views(gpu, stream):
    rng = np.random.default_rng(10)
    a = normal_f16(rng, (6, 5, 64))
    b = normal_f16(rng, (64,))
    av = a.transpose(1, 0, 2)                                               # [5, 6, 64]
    bv = np.lib.stride_tricks.as_strided(b, (5, 6, 64), (0, 0, 2))          # one row broadcast everywhere
    cbuf = np.zeros((5, 6, 80), f16)
    cv = cbuf[:, :, 8:72]                                                   # padded rows
    say("add permuted + broadcast")
    out = run_add(gpu, stream, cv, cbuf, av, a, bv, b).view(f16).reshape(5, 6, 80)
    ref = cbuf.copy()
    oracle.add(ref[:, :, 8:72], av, bv)
    assert np.array_equal(out, ref)
    bias = normal_f16(rng, (4096,))
    x = normal_f16(rng, (16, 4096))
    say("add bias rows")
    cz = np.zeros_like(x)
    out = run_add(gpu, stream, cz, cz, x, x,
                  np.lib.stride_tricks.as_strided(bias, (16, 4096), (0, 2)), bias).view(f16).reshape(16, 4096)
    assert np.array_equal(out, (x.astype(f32) + bias.astype(f32)).astype(f16))


def test_add_plan_and_errors(gpu, stream):
    L = TensorLayout
    c = lambda *s: L.new_contiguous(dt.F16, list(s))
    # contiguous tensors merge into one dimension: [count, 1 | c, a, b strides]
    assert ophip.Add.plan(ophip.AddArgs(c(4, 5, 6), None, c(4, 5, 6), None, c(4, 5, 6), None)) == [120, 1, 2, 2, 2]
    # a row broadcast over 16 rows: two dimensions, b does not advance with the row
    assert ophip.Add.plan(ophip.AddArgs(c(16, 64), None, c(16, 64), None, L(dt.F16, [16, 64], [0, 2]), None)) == \
        [1024, 64, 1, 128, 2, 128, 2, 0, 2]
    op = ophip.Add(gpu)
    for args, kind in ((ophip.AddArgs(c(2, 3), None, c(6), None, c(2, 3), None), "RankMismatch"),
                       (ophip.AddArgs(c(2, 3), None, c(2, 4), None, c(2, 3), None), "ShapeMismatch"),
                       (ophip.AddArgs(L(dt.F16, [2, 3], [0, 2]), None, c(2, 3), None, c(2, 3), None), "ShapeNotSupport"),
                       (ophip.AddArgs(L(dt.F16, [2, None], [6, 2]), None, c(2, 3), None, c(2, 3), None), "DynamicNotSupport")):
        with pytest.raises(ophip.LaunchError) as e:
            op.launch(args, None, stream)
        assert e.value.kind == kind
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.AddArgs(c(2, 3), None, c(2, 3), None, L.new_contiguous(dt.F32, [2, 3]), None), 0)
    assert e.value.kind == "TypeMismatch"
    assert op.scheme(ophip.AddArgs(*[L(dt.F16, [None, None], [None, None]), None] * 3), 0) == 0  # add/cuda/mod.rs:134-138


# -------------------------------------------------------------- add_rows ----

@pytest.mark.parametrize("batch,m,n,k,idt,dtype", [(1, 10, 2048, 100, np.uint32, f16), (4, 7, 4096, 32000, np.uint64, f16),
                                                   (2, 3, 77, 5, np.uint32, f16), (2, 5, 100, 9, np.uint32, f32)])
def test_add_rows(gpu, stream, batch, m, n, k, idt, dtype):
    rng = np.random.default_rng(batch + m + n)
    dst = rng.standard_normal((batch, m, n)).astype(f32).astype(dtype)
    src = rng.standard_normal((k, n)).astype(f32).astype(dtype)
    idx = rng.integers(0, k, (batch, m)).astype(idt)
    idx[0, 0], idx[0, 1] = k - 1, k - 1
    dd, sd, idd = gpu.from_host(dst), gpu.from_host(src), gpu.from_host(idx)
    lay = TensorLayout.of
    op = ophip.AddRows(gpu)
    args = ophip.AddRowsArgs(lay(dst), dd, lay(src), sd, lay(idx), idd)
    op.scheme(args, 0)
    say("add_rows b=%d m=%d n=%d k=%d" % (batch, m, n, k))
    op.launch(args, None, stream)
    out = gpu.to_host(dd, dtype, dst.size, stream=stream).reshape(dst.shape)
    assert np.array_equal(out, oracle.add_rows(dst.copy(), src, idx))


def test_add_rows_strided_out_of_range_and_errors(gpu, stream):
    rng = np.random.default_rng(11)
    batch, m, n, k, ld = 2, 4, 256, 6, 640
    dbuf = Dev(gpu, normal_f16(rng, (batch, m, ld)))
    src = normal_f16(rng, (k, n))
    idx = np.array([[0, 5, 6, 2], [1, 1, 9, 3]], np.uint32)     # 6 and 9 are out of range: rows left alone
    sd, idd = gpu.from_host(src), gpu.from_host(idx)
    L = TensorLayout
    op = ophip.AddRows(gpu)
    dl = L(dt.F16, [batch, m, n], [m * ld * 2, ld * 2, 2])
    say("add_rows strided with out-of-range indices")
    op.launch(ophip.AddRowsArgs(dl, dbuf.ptr + 128 * 2, L.of(src), sd, L.of(idx), idd), None, stream)
    out = dbuf.back(stream).view(f16).reshape(batch, m, ld)
    ref = dbuf.host.view(f16).reshape(batch, m, ld).copy()
    with pytest.raises(oracle.OracleError):
        oracle.add_rows(ref[:, :, 128:128 + n], src, idx)       # the oracle adds the valid rows, then reports
    assert np.array_equal(out, ref)
    c = lambda d_, *s: L.new_contiguous(d_, list(s))
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.AddRowsArgs(c(dt.F16, 2, 3, 8), None, c(dt.F16, 5, 8), None, c(dt.I32, 2, 3), None), 0)
    assert e.value.kind == "TypeNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.AddRowsArgs(c(dt.F16, 2, 3, 8), None, c(dt.F16, 5, 9), None, c(dt.U32, 2, 3), None), 0)
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.AddRowsArgs(c(dt.F16, 3, 8), None, c(dt.F16, 5, 8), None, c(dt.U32, 2, 3), None), 0)
    assert e.value.kind == "RankNotSupport"


def test_one_null_base_is_refused_by_every_launch(gpu, stream):
    """Arguments with null bases are what every `Args::layout` of the reference makes for scheme(); a launch must refuse
    them (ArgsNotSupport) before any kernel sees them, whichever single base is missing and whichever kernel the
    shapes would have gone to (one-pass attention at decode and prefill shapes included)."""
    c = lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    u32 = lambda *s: TensorLayout.new_contiguous(dt.U32, list(s))
    mem = lambda: gpu.from_host(np.zeros(1 << 16, f16))
    empty = TensorLayout(dt.F16, [0, 64], [128, 2])
    cases = [
        ("rms_norm", ophip.RmsNorm, lambda b: ophip.RmsNormArgs(c(16, 256), b[0], c(16, 256), b[1], c(256), b[2], 1e-5), 3),
        ("layer_norm", ophip.LayerNorm, lambda b: ophip.LayerNormArgs(c(16, 256), b[0], c(16, 256), b[1], c(256), b[2], c(256), b[3], 1e-5), 4),
        ("rope", ophip.Rope, lambda b: ophip.RopeArgs(c(8, 4, 64), b[0], u32(8), b[1], empty, None, empty, None, 1e4), 2),
        ("fused_softmax", ophip.FusedSoftmax, lambda b: ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL, c(4, 8, 64), b[0]), 1),
        ("rearrange", ophip.Rearrange, lambda b: ophip.RearrangeArgs(TensorLayout(dt.F16, [8, 64], [2, 16]), b[0], c(8, 64), b[1]), 2),
        ("swiglu", ophip.Swiglu, lambda b: ophip.SwigluArgs(c(16, 256), b[0], c(16, 256), b[1]), 2),
        ("gelu", ophip.Gelu, lambda b: ophip.GeluArgs(c(16, 256), b[0]), 1),
        ("add", ophip.Add, lambda b: ophip.AddArgs(c(16, 256), b[0], c(16, 256), b[1], c(16, 256), b[2]), 3),
        ("add_rows", ophip.AddRows, lambda b: ophip.AddRowsArgs(c(2, 4, 64), b[0], c(8, 64), b[1], u32(2, 4), b[2]), 3),
        ("mat_mul, few rows", ophip.MatMul, lambda b: ophip.MatMulArgs(c(1, 16, 256), b[0], 0.0, c(1, 16, 128), b[1], c(1, 128, 256), b[2], 1.0), 3),
        ("mat_mul, tiles", ophip.MatMul, lambda b: ophip.MatMulArgs(c(1, 128, 128), b[0], 0.0, c(1, 128, 64), b[1], c(1, 64, 128), b[2], 1.0), 3),
        ("attention, decode shape", ophip.Attention, lambda b: ophip.AttentionArgs(c(4, 16, 64), b[0], c(4, 16, 64), b[1], c(4, 16, 64), b[2], c(4, 16, 64), b[3], 1), 4),
        ("attention, prefill shape", ophip.Attention, lambda b: ophip.AttentionArgs(c(4, 128, 64), b[0], c(4, 128, 64), b[1], c(4, 128, 64), b[2], c(4, 128, 64), b[3], 1), 4),
        ("attention_kv_cached", ophip.AttnKVCached, lambda b: ophip.AttnKVCachedArgs(c(4, 16, 64), b[0], c(4, 16, 64), b[1], c(4, 16, 64), b[2], c(4, 16, 64), b[3],
                                                                                     c(4, 64, 64), b[4], c(4, 64, 64), b[5], 1, 5), 6),
    ]
    for name, cls, make, nbases in cases:
        op = cls(gpu)
        for missing in range(nbases):
            bases = [mem() for _ in range(nbases)]
            bases[missing] = None
            say("%s, base %d null" % (name, missing))
            with pytest.raises(ophip.LaunchError) as e:
                op.launch(make(bases), None, stream)
            assert e.value.kind == "ArgsNotSupport", (name, missing, e.value.kind)
    rs = ophip.RandomSample(gpu)
    for missing in ("kv_pair_base", "logits_base"):
        a = ophip.RandomSampleArgs.layout(dt.F16, 1000)
        a.kv_pair_base, a.logits_base = mem(), mem()
        setattr(a, missing, None)
        a.config = ophip.SampleArgs(0.8, 0.9, 50)
        with pytest.raises(ophip.LaunchError) as e:
            rs.launch(a, None, stream)
        assert e.value.kind == "ArgsNotSupport", missing
    stream.synchronize()


def test_mat_mul_with_nothing_to_multiply(gpu, stream):
    """Empty products: zero rows, columns or batches plan nothing and launch nothing (scheme once divided by the number
    of column strips, which was zero); K = 0 leaves c = beta * c."""
    c = lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    op = ophip.MatMul(gpu)
    for bt, m, n, k in ((1, 0, 128, 64), (1, 16, 0, 64), (0, 16, 128, 64), (3, 0, 0, 0)):
        a, b, cc = gpu.malloc(max(1, bt * m * k * 2)), gpu.malloc(max(1, bt * k * n * 2)), gpu.malloc(max(1, bt * m * n * 2))
        args = ophip.MatMulArgs(c(bt, m, n), cc, 0.5, c(bt, m, k), a, c(bt, k, n), b, 1.0)
        say("mat_mul %dx(%dx%dx%d)" % (bt, m, n, k))
        assert op.scheme(args, 2 ** 40) == 0
        assert op.describe(args) == "empty"
        op.launch(args, None, stream)
    for bt, m, n in ((1, 16, 128), (2, 300, 300)):
        c0 = normal_f16(np.random.default_rng(m), (bt, m, n))
        cd, a, b = gpu.from_host(c0), gpu.malloc(16), gpu.malloc(16)
        args = ophip.MatMulArgs(c(bt, m, n), cd, 0.5, c(bt, m, 0), a, c(bt, 0, n), b, 1.0)
        say("mat_mul %dx(%dx%dx0)" % (bt, m, n))
        op.scheme(args, 2 ** 40)
        op.launch(args, None, stream)
        got = gpu.to_host(cd, f16, c0.size, stream=stream).reshape(c0.shape)
        assert np.array_equal(got, (c0.astype(f32) * f32(0.5)).astype(f16))
