"""attention and attention_kv_cached on the HIP backend against the oracle's composites,
through the C ABI.  Shapes: the reference's device test (attention/cuda.rs:97-160:
nh 32, nkvh 4, seq 7, att 127, dh 64), its kv-cached counterpart, and the Llama-7B decode
layer (q and o as strided views of the fused QKV / token-major buffers)."""
import numpy as np
import pytest

import ophip
import oracle
from helpers import assert_close_f16, normal_f16
from ophip import TensorLayout, dt

pytestmark = pytest.mark.gpu

f16 = np.float16
CAUSAL, NONE = ophip.AttnMask.CAUSAL, ophip.AttnMask.NONE


def say(msg):
    print(msg, flush=True)


def attention_f64(q, k, v, causal):
    nh, seq, dh = q.shape
    nkvh, att, _ = k.shape
    g = nh // nkvh
    kk, vv = np.repeat(k.astype(np.float64), g, axis=0), np.repeat(v.astype(np.float64), g, axis=0)
    s = np.einsum("hsd,had->hsa", q.astype(np.float64), kk) / np.sqrt(dh)
    if causal:
        keep = np.arange(att)[None, :] <= (att - seq + np.arange(seq))[:, None]
        s = np.where(keep[None], s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return np.einsum("hsa,had->hsd", p, vv)


def upload(gpu, a):
    return gpu.from_host(np.ascontiguousarray(a))


def download(gpu, stream, mem, like):
    return gpu.to_host(mem, like.dtype, like.size, stream=stream).reshape(like.shape)


@pytest.mark.parametrize("nh,nkvh,seq,att,dh,mask", [(32, 4, 7, 127, 64, CAUSAL), (8, 8, 33, 33, 128, CAUSAL),
                                                     (6, 2, 3, 40, 16, NONE), (4, 1, 1, 300, 64, CAUSAL),
                                                     # prefill: more than 64 rows per kv head, odd att (the MFMA tile
                                                     # kernels with cut last tiles and a partial last K-step)
                                                     (8, 2, 200, 333, 64, CAUSAL), (4, 4, 509, 509, 128, CAUSAL),
                                                     (4, 2, 100, 1001, 128, NONE)])
def test_attention_contiguous(gpu, stream, nh, nkvh, seq, att, dh, mask):
    rng = np.random.default_rng(nh * 1000 + att)
    q, k, v = (rng.random(s).astype(f16) for s in ((nh, seq, dh), (nkvh, att, dh), (nkvh, att, dh)))
    qd, kd, vd = upload(gpu, q), upload(gpu, k), upload(gpu, v)
    od = gpu.malloc(q.nbytes)
    op = ophip.Attention(gpu)
    lay = TensorLayout.of
    args = ophip.AttentionArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(q), od, mask)
    need = op.scheme(args, 2 ** 40)
    assert need >= (nh * seq * dh + nh * seq * att) * 2
    say("attention nh=%d nkvh=%d seq=%d att=%d dh=%d" % (nh, nkvh, seq, att, dh))
    op.launch(args, None, stream)
    out = download(gpu, stream, od, q)
    q_after = download(gpu, stream, qd, q)
    ref = oracle.attention(q.copy(), k, v, np.zeros_like(q), causal=(mask == CAUSAL))
    assert_close_f16(out, ref, "attention vs oracle")
    assert_close_f16(out, attention_f64(q, k, v, mask == CAUSAL), "attention vs f64")
    assert np.array_equal(q_after, out)  # q receives att . v, as in the reference


def test_attention_decode_layer_views(gpu, stream):
    """Llama-7B decode: q is the [token, head, dh] slice of the [16, 12288] QKV buffer viewed head-major,
    o the same view of a [16, 4096] buffer, k / v the first 2048 rows of [32, 2048, 128] caches."""
    rng = np.random.default_rng(16)
    nt, nh, dh, att = 16, 32, 128, 2048
    qkv = normal_f16(rng, (nt, 3 * nh * dh))
    k, v = normal_f16(rng, (nh, att, dh)), normal_f16(rng, (nh, att, dh))
    qkv_d, kd, vd = upload(gpu, qkv), upload(gpu, k), upload(gpu, v)
    obuf = np.zeros((nt, nh * dh), f16)
    od = upload(gpu, obuf)
    q_lay = TensorLayout(dt.F16, [nh, nt, dh], [dh * 2, 3 * nh * dh * 2, 2])
    o_lay = TensorLayout(dt.F16, [nh, nt, dh], [dh * 2, nh * dh * 2, 2])
    op = ophip.Attention(gpu)
    args = ophip.AttentionArgs(q_lay, qkv_d, TensorLayout.of(k), kd, TensorLayout.of(v), vd, o_lay, od, CAUSAL)
    need = op.scheme(args, 2 ** 40)
    ws = gpu.malloc(need)
    pool = ophip.StreamMemPool(gpu, stream)
    pool.put(need + (1 << 20))
    q_view = qkv[:, :nh * dh].reshape(nt, nh, dh).transpose(1, 0, 2)
    ref = oracle.attention(q_view, k, v, np.zeros((nt, nh * dh), f16).reshape(nt, nh, dh).transpose(1, 0, 2))
    for label, w, qa in (("own workspace", ws, stream), ("stream allocator", None, stream), ("pool", None, pool)):
        say("attention decode views, %s" % label)
        gpu.memset(od, 0)
        op.launch(args, w, qa)
        out = download(gpu, stream, od, obuf).reshape(nt, nh, dh).transpose(1, 0, 2)
        assert_close_f16(out, ref, "attention decode " + label)
    assert np.array_equal(download(gpu, stream, qkv_d, qkv), qkv)  # a staged q is left alone


def test_attention_scheme_workspace_rules(gpu):
    """WorkspaceCollector (common/workspace.rs:54-90): q, att, then the largest sub-operator need,
    each added only while the total still fits; unknown shapes plan nothing."""
    op = ophip.Attention(gpu)
    nh, nkvh, seq, att, dh = 32, 4, 7, 127, 64
    c = lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    args = ophip.AttentionArgs(c(nh, seq, dh), None, c(nkvh, att, dh), None, c(nkvh, att, dh), None, c(nh, seq, dh),
                               None, CAUSAL)
    # score rows are padded to 16 bytes (127 -> 128 columns): the operator's own buffer, MFMA-friendly
    q_size, att_size = nh * seq * dh * 2, nh * seq * ((att + 7) // 8 * 8) * 2
    assert op.scheme(args, 2 ** 40) >= q_size + att_size
    assert op.scheme(args, q_size + att_size) == q_size + att_size
    assert op.scheme(args, q_size + att_size - 1) == q_size
    assert op.scheme(args, q_size - 1) == 0
    dyn = ophip.AttentionArgs.new_null(CAUSAL, dt.F16, 32, None, 7, 127, None)  # attention/cuda.rs:10-21
    assert op.scheme(dyn, 2 ** 40) == 0


def test_attention_errors(gpu, stream):
    op = ophip.Attention(gpu)
    c = lambda d, *s: TensorLayout.new_contiguous(d, list(s))
    F = dt.F16
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.AttentionArgs(c(F, 4, 8), None, c(F, 4, 3, 8), None, c(F, 4, 3, 8), None, c(F, 4, 2, 8), None,
                                      CAUSAL), 0)
    assert e.value.kind == "RankNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.AttentionArgs(c(F, 4, 2, 8), None, c(F, 4, 3, 8), None, c(dt.F32, 4, 3, 8), None,
                                      c(F, 4, 2, 8), None, CAUSAL), 0)
    assert e.value.kind == "TypeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.AttentionArgs(c(F, 4, 2, 8), None, c(F, 4, 3, 8), None, c(F, 4, 3, 16), None, c(F, 4, 2, 8),
                                      None, CAUSAL), 0)
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.AttentionArgs.new_null(CAUSAL, F, 32, 4, None, 127, 64), None, stream)
    assert e.value.kind == "DynamicNotSupport"


@pytest.mark.parametrize("nh,nkvh,seq,dh,buf,pos", [(32, 4, 7, 64, 160, 120), (32, 32, 16, 128, 2048, 2032),
                                                    (8, 2, 1, 32, 50, 0)])
def test_attention_kv_cached(gpu, stream, nh, nkvh, seq, dh, buf, pos):
    rng = np.random.default_rng(nh + buf + pos)
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, seq, dh)), normal_f16(rng, (nkvh, seq, dh))
    kc, vc = normal_f16(rng, (nkvh, buf, dh)), normal_f16(rng, (nkvh, buf, dh))
    qd, kd, vd, kcd, vcd = (upload(gpu, a) for a in (q, k, v, kc, vc))
    od = gpu.malloc(q.nbytes)
    lay = TensorLayout.of
    op = ophip.AttnKVCached(gpu)
    args = ophip.AttnKVCachedArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(q), od, lay(kc), kcd, lay(vc), vcd, CAUSAL, pos)
    op.scheme(args, 2 ** 40)
    say("attention_kv_cached nh=%d nkvh=%d seq=%d dh=%d buf=%d pos=%d" % (nh, nkvh, seq, dh, buf, pos))
    op.launch(args, None, stream)
    out = download(gpu, stream, od, q)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    ref = oracle.attention_kv_cached(q.copy(), k, v, np.zeros_like(q), kc_ref, vc_ref, pos)
    assert np.array_equal(download(gpu, stream, kcd, kc), kc_ref)  # caches: appended rows exact, rest untouched
    assert np.array_equal(download(gpu, stream, vcd, vc), vc_ref)
    assert_close_f16(out, ref, "attention_kv_cached vs oracle")
    assert_close_f16(out, attention_f64(q, kc_ref[:, :pos + seq], vc_ref[:, :pos + seq], True), "kv cached vs f64")


def kv_cached_case(gpu, stream, op, nh, nkvh, seq, dh, buf, pos, mask, rng, strided=False):
    """One launch on fresh buffers; returns (o, q afterwards, k cache, v cache) and the host inputs."""
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, seq, dh)), normal_f16(rng, (nkvh, seq, dh))
    kc, vc = normal_f16(rng, (nkvh, buf, dh)), normal_f16(rng, (nkvh, buf, dh))
    lay = TensorLayout.of
    if strided:
        # q, k, v as the head-major views of one token-major [seq, (nh + 2 nkvh) * dh] buffer (a fused QKV
        # product), o as the same view of a [seq, nh * dh] buffer: heads and tokens do not merge
        row = (nh + 2 * nkvh) * dh
        qkv = np.zeros((seq, row), f16)
        qkv[:, :nh * dh] = q.transpose(1, 0, 2).reshape(seq, nh * dh)
        qkv[:, nh * dh:(nh + nkvh) * dh] = k.transpose(1, 0, 2).reshape(seq, nkvh * dh)
        qkv[:, (nh + nkvh) * dh:] = v.transpose(1, 0, 2).reshape(seq, nkvh * dh)
        qkv_d = upload(gpu, qkv)
        q_lay = TensorLayout(dt.F16, [nh, seq, dh], [dh * 2, row * 2, 2])
        kv_lay = TensorLayout(dt.F16, [nkvh, seq, dh], [dh * 2, row * 2, 2])
        o_lay = TensorLayout(dt.F16, [nh, seq, dh], [dh * 2, nh * dh * 2, 2])
        qd, kd, vd = qkv_d.ptr, qkv_d.ptr + nh * dh * 2, qkv_d.ptr + (nh + nkvh) * dh * 2
        k_lay = v_lay = kv_lay
    else:
        qd, kd, vd = (upload(gpu, a) for a in (q, k, v))
        q_lay, k_lay, v_lay, o_lay = lay(q), lay(k), lay(v), lay(q)
    kcd, vcd = upload(gpu, kc), upload(gpu, vc)
    od = gpu.malloc(q.nbytes)
    gpu.memset(od, 0)
    args = ophip.AttnKVCachedArgs(q_lay, qd, k_lay, kd, v_lay, vd, o_lay, od, lay(kc), kcd, lay(vc), vcd, mask, pos)
    op.scheme(args, 2 ** 40)
    op.launch(args, None, stream)
    if strided:
        out = download(gpu, stream, od, np.zeros((seq, nh, dh), f16)).transpose(1, 0, 2)
        q_after = download(gpu, stream, qkv_d, qkv)[:, :nh * dh].reshape(seq, nh, dh).transpose(1, 0, 2)
    else:
        out, q_after = download(gpu, stream, od, q), download(gpu, stream, qd, q)
    return out, q_after, download(gpu, stream, kcd, kc), download(gpu, stream, vcd, vc), (q, k, v, kc, vc)


@pytest.mark.parametrize("nh,nkvh,seq,dh,buf,pos,mask,strided", [
    (32, 32, 16, 128, 2048, 2032, CAUSAL, True),    # the decode layer, q / k / v inside a fused QKV buffer
    (32, 8, 1, 128, 4096, 4095, CAUSAL, False),     # one token, grouped heads: 4 rows per kv head, 16 chunks
    (32, 4, 7, 64, 160, 120, CAUSAL, False),        # attention_kv_cached/cuda.rs: 56 rows per kv head, one chunk
    (32, 4, 7, 64, 1500, 1017, CAUSAL, True),       # the same over 4 chunks, the last one ragged (att 1024)
    (8, 8, 16, 64, 700, 0, CAUSAL, False),          # empty cache: everything comes from k and v
    (12, 4, 5, 128, 300, 251, NONE, False),         # no mask: 15 rows, att 256 = exactly one chunk
    (12, 4, 5, 128, 300, 252, NONE, False),         # att 257: a second chunk with one key
    (16, 2, 8, 128, 520, 500, CAUSAL, False),       # 64 rows per kv head, the append straddles chunks 1 and 2
    (3, 3, 33, 64, 100, 10, CAUSAL, False),         # 33 rows per kv head
])
def test_attention_kv_cached_one_pass(gpu, stream, monkeypatch, nh, nkvh, seq, dh, buf, pos, mask, strided):
    """Decode shapes run on the one-pass kernel: against the oracle's composite (which rounds the scores and the
    probabilities to f16 between the steps), against f64, and against the composite of launches
    (OPHIP_ATTN_ONE_PASS=0) for everything the reference makes observable: o, the appended cache rows bit for bit
    and the rest of the caches untouched, q overwritten with the result when its heads and tokens merge and left
    alone when they do not."""
    say("kv cached one pass nh=%d nkvh=%d seq=%d dh=%d buf=%d pos=%d strided=%s" % (nh, nkvh, seq, dh, buf, pos, strided))
    fused = ophip.AttnKVCached(gpu)
    monkeypatch.setenv("OPHIP_ATTN_ONE_PASS", "0")
    composite = ophip.AttnKVCached(gpu)  # the switch is read when an operator is created
    monkeypatch.delenv("OPHIP_ATTN_ONE_PASS")
    seed = nh * 7919 + buf * 31 + pos
    out, q_after, kc_out, vc_out, (q, k, v, kc, vc) = kv_cached_case(gpu, stream, fused, nh, nkvh, seq, dh, buf, pos, mask,
                                                                     np.random.default_rng(seed), strided)
    out_c, q_after_c, kc_c, vc_c, _ = kv_cached_case(gpu, stream, composite, nh, nkvh, seq, dh, buf, pos, mask,
                                                     np.random.default_rng(seed), strided)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    ref = oracle.attention_kv_cached(q.copy(), k, v, np.zeros_like(q), kc_ref, vc_ref, pos, causal=(mask == CAUSAL))
    assert np.array_equal(kc_out, kc_ref) and np.array_equal(vc_out, vc_ref)
    assert np.array_equal(kc_c, kc_ref) and np.array_equal(vc_c, vc_ref)
    assert_close_f16(out, ref, "one pass vs oracle")
    assert_close_f16(out, attention_f64(q, kc_ref[:, :pos + seq], vc_ref[:, :pos + seq], mask == CAUSAL), "one pass vs f64")
    assert_close_f16(out, out_c, "one pass vs composite")
    merged = not strided or nh == 1 or seq == 1
    assert np.array_equal(q_after, out if merged else q)
    assert np.array_equal(q_after_c, out_c if merged else q)


def test_attention_kv_cached_errors_and_scheme(gpu, stream):
    op = ophip.AttnKVCached(gpu)
    c = lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    mk = lambda pos, buf=16: ophip.AttnKVCachedArgs(c(8, 3, 32), None, c(2, 3, 32), None, c(2, 3, 32), None, c(8, 3, 32),
                                                    None, c(2, buf, 32), None, c(2, buf, 32), None, CAUSAL, pos)
    assert op.scheme(mk(None), 2 ** 40) == 0   # position unknown: nothing planned (attention/… new_null, att dynamic)
    assert op.scheme(mk(5), 2 ** 40) >= (8 * 3 * 32 + 8 * 3 * 8) * 2
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(mk(14), None, stream)   # 14 + 3 > 16
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(mk(None), None, stream)
    assert e.value.kind == "DynamicNotSupport"
    bad = mk(0)
    bad.v_cache_layout = c(3, 16, 32)
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(bad, 0)
    assert e.value.kind == "ShapeMismatch"


def test_decode_layer_chain_matches_the_oracle_end_to_end(gpu, stream):
    """The benchmark's step - rms_norm, QKV mat_mul, rope (q, k), QK^T, causal softmax, PV, O-proj, rms_norm,
    gate/up, swiglu, down at Llama-7B decode shapes - run once on the GPU and once through the oracle on
    the same seeded weights; every intermediate rounding to f16 happens in both."""
    import bench

    rng = np.random.default_rng(0)
    layer = bench.Layer(ophip, gpu, rng, host=True)
    print("decode layer chain, 12 launches", flush=True)
    layer.step(stream)
    out = gpu.to_host(layer.d["out"], f16, bench.NT * bench.D, stream=stream).reshape(bench.NT, bench.D)
    ref = bench.cpu_layer_step(oracle, layer.h, min(oracle.max_threads(), 16))
    # Twelve chained operators, each rounding to f16: single-ulp differences of an intermediate (summation
    # order in mat_mul) spread through the later products, so the per-operator outlier rule does not apply.
    # The bar here: every element within 1e-2 of the output scale, and the typical element much closer.
    err = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    scale = float(np.abs(ref.astype(np.float64)).max())
    print("decode layer: max err %.3g, median err %.3g, output scale %.3g" % (err.max(), np.median(err), scale), flush=True)
    assert err.max() <= 1e-2 * scale, err.max() / scale
    assert np.median(err) <= 1e-3 * scale, np.median(err) / scale


def test_decode_layer_chain_with_the_attention_operator_matches_the_oracle_end_to_end(gpu, stream):
    """The same layer with the crate's composite attention_kv_cached in place of the QK^T / softmax / PV launches (the
    second figure of the benchmark: nine launches of the operator API): against the oracle's composite on the same
    seeded weights, and the 16 appended rows of both caches bit for bit."""
    import bench

    rng = np.random.default_rng(0)
    layer = bench.Layer(ophip, gpu, rng, host=True)
    print("decode layer chain through attention_kv_cached, 9 launches", flush=True)
    layer.step(stream, order=layer.order_attention_op)
    out = gpu.to_host(layer.d["out"], f16, bench.NT * bench.D, stream=stream).reshape(bench.NT, bench.D)
    ref = bench.cpu_layer_step(oracle, layer.h, min(oracle.max_threads(), 16), attention_op=True)
    err = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    scale = float(np.abs(ref.astype(np.float64)).max())
    print("decode layer with attention op: max err %.3g, median err %.3g, output scale %.3g" % (err.max(), np.median(err), scale), flush=True)
    assert err.max() <= 1e-2 * scale, err.max() / scale
    assert np.median(err) <= 1e-3 * scale, np.median(err) / scale
    # the caches: rows below KV - NT untouched, the appended rows are the k / v columns of the qkv rows the GPU made
    nt, d, nh, dh, kv = bench.NT, bench.D, bench.NH, bench.DH, bench.KV
    qkv = gpu.to_host(layer.d["qkv"], f16, nt * 3 * d, stream=stream).reshape(nt, 3 * d)
    for name, col in (("k_cache", d), ("v_cache", 2 * d)):
        cache = gpu.to_host(layer.d[name], f16, nh * kv * dh, stream=stream).reshape(nh, kv, dh)
        assert np.array_equal(cache[:, :kv - nt], layer.h[name][:, :kv - nt]), name
        new = qkv[:, col:col + d].reshape(nt, nh, dh).transpose(1, 0, 2)
        assert np.array_equal(cache[:, kv - nt:].view(np.uint16), new.view(np.uint16)), name


# ------------------------------------------------ one pass, prefill shapes ----
# Where its walk over the keys is shorter than the composite's passes over the score matrix (prefill shapes), attention
# runs on one kernel that keeps the scores on the chip (attention_prefill.hip).  Same bar as the composite: the oracle's composite and the f64 formula, within the f16 tolerance.

def run_attention(gpu, stream, q, k, v, mask, op=None):
    qd, kd, vd = upload(gpu, q), upload(gpu, k), upload(gpu, v)
    od = gpu.malloc(q.nbytes)
    gpu.memset(od, 0xFF)
    op = op or ophip.Attention(gpu)
    lay = TensorLayout.of
    args = ophip.AttentionArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(q), od, mask)
    op.launch(args, None, stream)
    return download(gpu, stream, od, q), download(gpu, stream, qd, q)


@pytest.mark.parametrize("nh,nkvh,seq,att,dh,mask", [(4, 4, 128, 128, 128, CAUSAL), (2, 1, 64, 64, 128, NONE), (8, 2, 256, 256, 64, CAUSAL),
                                                     (3, 1, 130, 257, 128, CAUSAL), (3, 3, 65, 64 + 65, 64, CAUSAL),
                                                     (4, 2, 1000, 1000, 64, CAUSAL), (2, 2, 300, 77, 128, NONE),
                                                     (32, 32, 512, 512, 128, CAUSAL), (8, 8, 1024, 1536, 128, CAUSAL)])
def test_attention_one_pass_prefill(gpu, stream, monkeypatch, nh, nkvh, seq, att, dh, mask):
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "1")  # (the planner would take the composite for some of the small ones)
    rng = np.random.default_rng(nh + seq + att + dh)
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, att, dh)), normal_f16(rng, (nkvh, att, dh))
    say("attention one pass nh=%d nkvh=%d seq=%d att=%d dh=%d mask=%d" % (nh, nkvh, seq, att, dh, mask))
    out, q_after = run_attention(gpu, stream, q, k, v, mask)
    assert_close_f16(out, attention_f64(q, k, v, mask == CAUSAL), "one pass vs f64")
    oracle.set_threads(8)
    try:
        ref = oracle.attention(q.copy(), k, v, np.zeros_like(q), causal=(mask == CAUSAL))
    finally:
        oracle.set_threads(1)
    assert_close_f16(out, ref, "one pass vs oracle")
    assert np.array_equal(q_after, out)  # contiguous q: heads and tokens merge, q receives att . v as in the reference
    again, _ = run_attention(gpu, stream, q, k, v, mask)
    assert np.array_equal(again, out)  # the same bits on every launch


@pytest.mark.parametrize("nh,nkvh,seq,att,dh,mask", [(32, 4, 7, 127, 64, CAUSAL), (5, 5, 1, 9, 64, CAUSAL), (6, 2, 40, 40, 128, NONE),
                                                     (8, 8, 33, 33, 128, CAUSAL)])
def test_attention_one_pass_forced_on_few_rows_agrees_with_the_composite(gpu, stream, monkeypatch, nh, nkvh, seq, att, dh, mask):
    rng = np.random.default_rng(nh + seq + att)
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, att, dh)), normal_f16(rng, (nkvh, att, dh))
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "1")
    fused = ophip.Attention(gpu)
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "0")
    composite = ophip.Attention(gpu)
    say("attention one pass forced nh=%d seq=%d att=%d" % (nh, seq, att))
    a, qa = run_attention(gpu, stream, q, k, v, mask, op=fused)
    b, qb = run_attention(gpu, stream, q, k, v, mask, op=composite)
    ref = attention_f64(q, k, v, mask == CAUSAL)
    assert_close_f16(a, ref, "one pass")
    assert_close_f16(b, ref, "composite")
    assert np.array_equal(qa, a) and np.array_equal(qb, b)


@pytest.mark.parametrize("split", ["0", "1"])
@pytest.mark.parametrize("nh,nkvh,seq,att,dh,mask", [(4, 2, 384, 384, 128, CAUSAL), (3, 3, 130, 257, 64, CAUSAL), (2, 1, 100, 64, 128, NONE),
                                                     (2, 2, 128, 1, 64, NONE), (4, 4, 70, 70, 128, CAUSAL)])
def test_attention_one_pass_both_builds(gpu, stream, monkeypatch, split, nh, nkvh, seq, att, dh, mask):
    """Four waves on all key tiles, or eight waves of which four take the even and four the odd tiles (one tile only: the
    second group has nothing to add): the planner picks by shape, OPHIP_ATTN_KEYSPLIT keeps one."""
    rng = np.random.default_rng(nh + seq + att + dh)
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, att, dh)), normal_f16(rng, (nkvh, att, dh))
    monkeypatch.setenv("OPHIP_ATTN_KEYSPLIT", split)
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "1")
    op = ophip.Attention(gpu)
    say("attention one pass key split=%s nh=%d seq=%d att=%d dh=%d" % (split, nh, seq, att, dh))
    out, q_after = run_attention(gpu, stream, q, k, v, mask, op=op)
    assert_close_f16(out, attention_f64(q, k, v, mask == CAUSAL), "one pass, split " + split)
    assert np.array_equal(q_after, out)
    again, _ = run_attention(gpu, stream, q, k, v, mask, op=op)
    assert np.array_equal(again, out)


def test_attention_one_pass_on_views_of_a_fused_qkv_buffer(gpu, stream, monkeypatch):
    """q, k, v are column slices of one [seq, 3 * nh * dh] buffer viewed head-major, o is token-major: heads and tokens
    of q do not merge, so q is left alone (the reference works on a copy of it)."""
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "1")
    rng = np.random.default_rng(21)
    seq, nh, dh = 300, 8, 128
    qkv = normal_f16(rng, (seq, 3 * nh * dh))
    obuf = np.zeros((seq, nh * dh), f16)
    qkv_d, od = upload(gpu, qkv), upload(gpu, obuf)
    row = 3 * nh * dh * 2
    lay = lambda: TensorLayout(dt.F16, [nh, seq, dh], [dh * 2, row, 2])
    o_lay = TensorLayout(dt.F16, [nh, seq, dh], [dh * 2, nh * dh * 2, 2])
    op = ophip.Attention(gpu)
    args = ophip.AttentionArgs(lay(), qkv_d.ptr, lay(), qkv_d.ptr + nh * dh * 2, lay(), qkv_d.ptr + 2 * nh * dh * 2, o_lay, od, CAUSAL)
    say("attention one pass, views of a fused QKV buffer")
    op.launch(args, None, stream)
    out = download(gpu, stream, od, obuf).reshape(seq, nh, dh).transpose(1, 0, 2)
    view = lambda i: qkv[:, i * nh * dh:(i + 1) * nh * dh].reshape(seq, nh, dh).transpose(1, 0, 2)
    assert_close_f16(out, attention_f64(view(0), view(1), view(2), True), "one pass on views")
    assert np.array_equal(download(gpu, stream, qkv_d, qkv), qkv)


def test_attention_one_pass_with_o_in_place_of_q(gpu, stream, monkeypatch):
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "1")
    rng = np.random.default_rng(22)
    nh, seq, dh = 4, 192, 64
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nh, seq, dh))
    qd, kd, vd = upload(gpu, q), upload(gpu, k), upload(gpu, v)
    lay = TensorLayout.of
    op = ophip.Attention(gpu)
    op.launch(ophip.AttentionArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(q), qd, CAUSAL), None, stream)
    assert_close_f16(download(gpu, stream, qd, q), attention_f64(q, k, v, True), "o = q")


def test_attention_kv_cached_prefill_goes_through_the_one_pass_kernel(gpu, stream):
    rng = np.random.default_rng(23)
    op = ophip.AttnKVCached(gpu)
    for pos, seq, strided in ((0, 256, False), (100, 200, False), (40, 128, True)):
        say("attention_kv_cached prefill pos=%d seq=%d strided=%s" % (pos, seq, strided))
        out, q_after, kc_out, vc_out, (q, k, v, kc, vc) = kv_cached_case(gpu, stream, op, 8, 2, seq, 128, 512, pos, CAUSAL, rng, strided)
        kc_ref, vc_ref = kc.copy(), vc.copy()
        ref = oracle.attention_kv_cached(q.copy(), k, v, np.zeros_like(q), kc_ref, vc_ref, pos, causal=True)
        assert np.array_equal(kc_out, kc_ref) and np.array_equal(vc_out, vc_ref)
        assert_close_f16(out, ref, "kv cached prefill vs oracle")
        assert_close_f16(out, attention_f64(q, kc_ref[:, :pos + seq], vc_ref[:, :pos + seq], True), "kv cached prefill vs f64")
        assert np.array_equal(q_after, q if strided else out)


def test_prefill_layer_chain_matches_the_oracle_end_to_end(gpu, stream):
    """A prefill step of a small Llama-shaped layer (192 tokens, d 1024, 8 heads of 128, FFN 2752) on the operators a model
    runs it with -- rms_norm, QKV mat_mul, rope on q and k, attention_kv_cached from an empty cache (the append and the
    one-pass attention over views of the QKV buffer), O-proj, rms_norm, gate/up, swiglu, down -- and the same chain
    through the oracle on the same seeded weights."""
    nt, d, nh, dh, di, buf = 192, 1024, 8, 128, 2752, 256
    rng = np.random.default_rng(1)
    L, c = TensorLayout, lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    h = {"x": normal_f16(rng, (nt, d)), "w1": rng.uniform(0.5, 1.5, d).astype(np.float32), "w2": rng.uniform(0.5, 1.5, d).astype(np.float32),
         "wqkv": (rng.standard_normal((d, 3 * d)) * 0.03).astype(f16), "wo": (rng.standard_normal((d, d)) * 0.03).astype(f16),
         "wgu": (rng.standard_normal((d, 2 * di)) * 0.03).astype(f16), "wd": (rng.standard_normal((di, d)) * 0.02).astype(f16),
         "pos": np.arange(nt, dtype=np.uint32)}
    dev = {k: upload(gpu, v) for k, v in h.items()}
    xn, qkv, o, y, yn, gu, out = (gpu.malloc(n * 2) for n in (nt * d, nt * 3 * d, nt * d, nt * d, nt * d, nt * 2 * di, nt * d))
    kc, vc = gpu.malloc(nh * buf * dh * 2), gpu.malloc(nh * buf * dh * 2)
    gpu.memset(kc, 0); gpu.memset(vc, 0)
    w32 = lambda n: L(dt.F32, [n], [4])
    rms, mm, rope, akv, sw = ophip.RmsNorm(gpu), ophip.MatMul(gpu), ophip.Rope(gpu), ophip.AttnKVCached(gpu), ophip.Swiglu(gpu)
    ws = gpu.malloc(64 << 20)
    say("prefill layer chain")
    rms.launch(ophip.RmsNormArgs(c(nt, d), xn, c(nt, d), dev["x"], w32(d), dev["w1"], 1e-5), None, stream)
    mm.launch(ophip.MatMulArgs(c(nt, 3 * d), qkv, 0.0, c(nt, d), xn, c(d, 3 * d), dev["wqkv"], 1.0), ws, stream)
    row = 3 * d * 2
    tok = L(dt.F16, [nt, 2 * nh, dh], [row, dh * 2, 2])  # q and k heads side by side in a QKV row
    empty = L(dt.F16, [0, dh], [dh * 2, 2])
    rope.launch(ophip.RopeArgs(tok, qkv, L.of(h["pos"]), dev["pos"], empty, None, empty, None, 1e4), None, stream)
    head = lambda: L(dt.F16, [nh, nt, dh], [dh * 2, row, 2])
    args = ophip.AttnKVCachedArgs(head(), qkv.ptr, head(), qkv.ptr + d * 2, head(), qkv.ptr + 2 * d * 2,
                                  L(dt.F16, [nh, nt, dh], [dh * 2, d * 2, 2]), o, c(nh, buf, dh), kc, c(nh, buf, dh), vc, CAUSAL, 0)
    akv.launch(args, ws, stream)
    mm.launch(ophip.MatMulArgs(c(nt, d), y, 0.0, c(nt, d), o, c(d, d), dev["wo"], 1.0), ws, stream)
    rms.launch(ophip.RmsNormArgs(c(nt, d), yn, c(nt, d), y, w32(d), dev["w2"], 1e-5), None, stream)
    mm.launch(ophip.MatMulArgs(c(nt, 2 * di), gu, 0.0, c(nt, d), yn, c(d, 2 * di), dev["wgu"], 1.0), ws, stream)
    half = L(dt.F16, [nt, di], [2 * di * 2, 2])
    sw.launch(ophip.SwigluArgs(half, gu, half, gu.ptr + di * 2), None, stream)
    mm.launch(ophip.MatMulArgs(c(nt, d), out, 0.0, half, gu, c(di, d), dev["wd"], 1.0), ws, stream)
    got = gpu.to_host(out, f16, nt * d, stream=stream).reshape(nt, d)
    kc_got = gpu.to_host(kc, f16, nh * buf * dh, stream=stream).reshape(nh, buf, dh)

    oracle.set_threads(8)
    try:
        r_xn = oracle.rms_norm(np.empty_like(h["x"]), h["x"], h["w1"], 1e-5)
        r_qkv = oracle.mat_mul(np.zeros((nt, 3 * d), f16), 0.0, r_xn, h["wqkv"], 1.0)
        oracle.set_threads(1)
        oracle.rope(r_qkv[:, :2 * d].reshape(nt, 2 * nh, dh), h["pos"], 1e4)
        oracle.set_threads(8)
        view = lambda i: r_qkv[:, i * d:(i + 1) * d].reshape(nt, nh, dh).transpose(1, 0, 2)
        r_o = np.zeros((nt, d), f16)
        r_kc, r_vc = np.zeros((nh, buf, dh), f16), np.zeros((nh, buf, dh), f16)
        oracle.attention_kv_cached(view(0), view(1), view(2), r_o.reshape(nt, nh, dh).transpose(1, 0, 2), r_kc, r_vc, 0, causal=True)
        r_y = oracle.mat_mul(np.zeros((nt, d), f16), 0.0, r_o, h["wo"], 1.0)
        r_yn = oracle.rms_norm(np.empty_like(r_y), r_y, h["w2"], 1e-5)
        r_gu = oracle.mat_mul(np.zeros((nt, 2 * di), f16), 0.0, r_yn, h["wgu"], 1.0)
        oracle.set_threads(1)
        oracle.swiglu(r_gu[:, :di], r_gu[:, di:])
        oracle.set_threads(8)
        ref = oracle.mat_mul(np.zeros((nt, d), f16), 0.0, r_gu[:, :di], h["wd"], 1.0)
    finally:
        oracle.set_threads(1)
    # the appended keys went through rms_norm, a product and rope on both sides: close, not bit-equal
    assert_close_f16(kc_got[:, :nt], r_kc[:, :nt], "appended keys", abs_tol=8e-3)
    assert (kc_got[:, nt:] == 0).all()
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    scale = float(np.abs(ref.astype(np.float64)).max())
    say("prefill layer: max err %.3g, median err %.3g, output scale %.3g" % (err.max(), np.median(err), scale))
    assert err.max() <= 1e-2 * scale, err.max() / scale
    assert np.median(err) <= 1e-3 * scale, np.median(err) / scale


# ------------------------------------------------ attention at decode shapes ----
# `attention` with few query rows per kv head against many keys (a runtime that keeps its own cache and calls attention
# on it) runs on the decode kernel of attention_kv_cached with nothing to append, when k and v have one layout.

@pytest.mark.parametrize("nh,nkvh,seq,att,dh,mask", [
    (32, 32, 16, 2048, 128, CAUSAL),   # the decode layer's shape: 16 rows per kv head, 8 chunks
    (32, 8, 1, 4096, 128, CAUSAL),     # one token, grouped heads
    (32, 4, 7, 127, 64, CAUSAL),       # attention/cuda.rs: 56 rows per kv head, one ragged chunk
    (12, 4, 5, 257, 128, NONE),        # no mask, a second chunk with one key
    (3, 3, 33, 100, 64, CAUSAL),       # 33 rows per kv head
    (8, 8, 64, 64, 128, CAUSAL),       # as many rows as keys
])
def test_attention_at_decode_shapes_runs_in_one_pass(gpu, stream, monkeypatch, nh, nkvh, seq, att, dh, mask):
    """Against f64 and the oracle's composite, and against the composite of launches (OPHIP_ATTN_FUSED=0) for what the
    reference makes observable besides o: q overwritten with the result (contiguous q: heads and tokens merge), k and v
    untouched."""
    rng = np.random.default_rng(nh + seq + att + dh)
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, att, dh)), normal_f16(rng, (nkvh, att, dh))
    say("attention at a decode shape nh=%d nkvh=%d seq=%d att=%d dh=%d mask=%d" % (nh, nkvh, seq, att, dh, mask))
    qd, kd, vd = upload(gpu, q), upload(gpu, k), upload(gpu, v)
    od = gpu.malloc(q.nbytes)
    gpu.memset(od, 0xFF)
    lay = TensorLayout.of
    args = ophip.AttentionArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(q), od, mask)
    ophip.Attention(gpu).launch(args, None, stream)
    out, q_after = download(gpu, stream, od, q), download(gpu, stream, qd, q)
    assert np.array_equal(download(gpu, stream, kd, k), k) and np.array_equal(download(gpu, stream, vd, v), v)
    assert_close_f16(out, attention_f64(q, k, v, mask == CAUSAL), "decode kernel vs f64")
    assert_close_f16(out, oracle.attention(q.copy(), k, v, np.zeros_like(q), causal=(mask == CAUSAL)), "decode kernel vs oracle")
    assert np.array_equal(q_after, out)
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "0")
    b, qb = run_attention(gpu, stream, q, k, v, mask)
    assert_close_f16(b, attention_f64(q, k, v, mask == CAUSAL), "composite vs f64")
    assert np.array_equal(qb, b)
    # the two paths differ where the composite rounds scores and probabilities to f16: well inside the bar of either
    assert np.abs(out.astype(np.float32) - b.astype(np.float32)).max() <= 4e-3


def test_attention_at_a_decode_shape_with_strided_views_and_separate_layouts(gpu, stream):
    """q inside a token-major QKV buffer (heads and tokens do not merge: q stays as it was), k and v as views of caches
    longer than att; then v with another layout than k, which the decode kernel does not take (the other paths do)."""
    rng = np.random.default_rng(99)
    nh, nkvh, seq, att, dh, buf = 8, 2, 4, 300, 128, 512
    q, kc, vc = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, buf, dh)), normal_f16(rng, (nkvh, buf, dh))
    row = nh * dh
    qkv = np.ascontiguousarray(q.transpose(1, 0, 2).reshape(seq, row))
    qd, kd, vd = upload(gpu, qkv), upload(gpu, kc), upload(gpu, vc)
    od = gpu.malloc(q.nbytes)
    q_lay = TensorLayout(dt.F16, [nh, seq, dh], [dh * 2, row * 2, 2])
    kv_lay = TensorLayout(dt.F16, [nkvh, att, dh], [buf * dh * 2, dh * 2, 2])
    o_lay = TensorLayout.new_contiguous(dt.F16, [nh, seq, dh])
    say("attention at a decode shape, strided views")
    ophip.Attention(gpu).launch(ophip.AttentionArgs(q_lay, qd, kv_lay, kd, kv_lay, vd, o_lay, od, CAUSAL), None, stream)
    ref = attention_f64(q, kc[:, :att], vc[:, :att], True)
    assert_close_f16(download(gpu, stream, od, q), ref, "views vs f64")
    assert np.array_equal(download(gpu, stream, qd, qkv), qkv)  # staged in the reference, left alone here
    # v stored [att, nkvh, dh]: another layout than k's
    vt = np.ascontiguousarray(vc[:, :att].transpose(1, 0, 2))
    vtd = upload(gpu, vt)
    v_lay = TensorLayout(dt.F16, [nkvh, att, dh], [dh * 2, nkvh * dh * 2, 2])
    ophip.Attention(gpu).launch(ophip.AttentionArgs(q_lay, qd, kv_lay, kd, v_lay, vtd, o_lay, od, CAUSAL), None, stream)
    assert_close_f16(download(gpu, stream, od, q), ref, "separate layouts vs f64")


def test_attention_at_a_decode_shape_with_o_over_other_operands(gpu, stream):
    """The decode kernel's workgroups (one per kv head and chunk of keys) write o while others still read q, k and v;
    the reference's composite reads everything before it writes o.  A call whose o lies over v, or over q in another
    layout, must therefore give what the composite gives: attention over the operands as they were."""
    rng = np.random.default_rng(123)
    nh, nkvh, seq, att, dh = 8, 2, 4, 100, 64
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, att, dh)), normal_f16(rng, (nkvh, att, dh))
    ref = attention_f64(q, k, v, True)
    lay = TensorLayout.of
    # (a) o at the start of v's buffer
    say("attention at a decode shape, o over v")
    qd, kd, vd = upload(gpu, q), upload(gpu, k), upload(gpu, v)
    ophip.Attention(gpu).launch(ophip.AttentionArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(q), vd, CAUSAL), None, stream)
    out = gpu.to_host(vd, np.float16, q.size, stream=stream).reshape(q.shape)
    assert_close_f16(out, ref, "o over v")
    # (b) q as a view of a token-major buffer (heads and tokens do not merge: the reference stages it), o contiguous
    # [nh, seq, dh] over the same bytes
    say("attention at a decode shape, o over q in another layout")
    row = nh * dh
    qkv = np.ascontiguousarray(q.transpose(1, 0, 2).reshape(seq, row))
    bd, kd, vd = upload(gpu, qkv), upload(gpu, k), upload(gpu, v)
    q_lay = TensorLayout(dt.F16, [nh, seq, dh], [dh * 2, row * 2, 2])
    o_lay = TensorLayout.new_contiguous(dt.F16, [nh, seq, dh])
    ophip.Attention(gpu).launch(ophip.AttentionArgs(q_lay, bd, lay(k), kd, lay(v), vd, o_lay, bd, CAUSAL), None, stream)
    out = gpu.to_host(bd, np.float16, q.size, stream=stream).reshape(q.shape)
    assert_close_f16(out, ref, "o over q in another layout")
