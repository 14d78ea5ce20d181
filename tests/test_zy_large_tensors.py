"""The streaming operators on tensors larger than 2^32 bytes (and 2^31 elements): what a card with 288 GB invites.

An offset kept in 32 bits, or an element index in a signed int, works at every benchmark shape and wraps here.  Each
tensor is a [n, d] f16 matrix of about 4.6 GiB whose rows all differ from the rows an address that wrapped by 2^31 or
2^32 bytes or elements would hit instead (row r is row r mod 8191 of a random base block, with a sign and a scale that
depend on r), uploaded a block of 8191 rows at a time; the operator runs once over the whole tensor; rows are read back
around every such boundary, at both ends and at random places, and compared with the oracle on the same rows.
"""
import numpy as np
import pytest

import ophip
import oracle
from helpers import assert_close_f16
from ophip import TensorLayout, dt

pytestmark = pytest.mark.gpu
f16, f32 = np.float16, np.float32
PERIOD = 8191  # rows of the base block: prime, so no power-of-two distance maps a row onto an equal one


def say(msg):
    print(msg, flush=True)


class Big:
    """An [n, d] f16 tensor on the device whose rows can be regenerated on the host one by one."""

    def __init__(self, gpu, n, d, seed, fill=True):
        self.gpu, self.n, self.d = gpu, n, d
        rng = np.random.default_rng(seed)
        self.base = rng.standard_normal((PERIOD, d)).astype(f32).astype(f16)
        self.mem = gpu.malloc(n * d * 2)
        if fill:  # the factor of a row repeats every 8 blocks of PERIOD rows: eight blocks made once, then copies
            blocks = [self.rows(np.arange(v * PERIOD, (v + 1) * PERIOD)) for v in range(8)]
            for b in range((n + PERIOD - 1) // PERIOD):
                gpu.upload(self.mem, blocks[b % 8][:min(PERIOD, n - b * PERIOD)], offset=b * PERIOD * d * 2)

    def rows(self, idx):
        idx = np.asarray(idx, dtype=np.int64)
        factor = np.where((idx // PERIOD) % 2 == 0, 1.0, -1.0) * (1.0 + ((idx // (2 * PERIOD)) % 4) * 0.25)
        return (self.base[idx % PERIOD] * factor[:, None].astype(f16)).astype(f16)

    def fetch(self, stream, idx):
        return np.stack([self.gpu.to_host(self.mem, f16, self.d, offset=int(r) * self.d * 2, stream=stream) for r in idx])

    def layout(self):
        return TensorLayout.new_contiguous(dt.F16, [self.n, self.d])


def sample_rows(n, d, seed=0):
    rows = {0, 1, 2, n - 1, n - 2, n // 2}
    for boundary in (2 ** 31, 2 ** 32, 2 ** 33):  # bytes, then elements
        for per_row in (d * 2, d):
            r = boundary // per_row
            rows.update(x for x in (r - 2, r - 1, r, r + 1) if 0 <= x < n)
    rows.update(int(x) for x in np.random.default_rng(seed).integers(0, n, 24))
    return np.array(sorted(rows))


SHAPES = {"wide rows": (600000, 4096), "narrow rows": (1200000, 2048)}  # 4.58 GiB either way


@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_rms_norm_and_layer_norm_past_4_gib(gpu, stream, shape):
    n, d = SHAPES[shape]
    say("rms_norm, layer_norm [%d, %d] f16" % (n, d))
    x, y = Big(gpu, n, d, 1), Big(gpu, n, d, 2, fill=False)
    rng = np.random.default_rng(3)
    w, b = rng.uniform(0.5, 1.5, d).astype(f32).astype(f16), rng.uniform(-0.5, 0.5, d).astype(f32).astype(f16)
    wd, bd = gpu.from_host(w), gpu.from_host(b)
    vec = TensorLayout.new_contiguous(dt.F16, [d])
    idx = sample_rows(n, d)
    xs = x.rows(idx)
    ophip.RmsNorm(gpu).launch(ophip.RmsNormArgs(y.layout(), y.mem, x.layout(), x.mem, vec, wd, 1e-5), None, stream)
    assert_close_f16(y.fetch(stream, idx), oracle.rms_norm(np.empty_like(xs), xs, w, 1e-5), "rms_norm past 4 GiB")
    ophip.LayerNorm(gpu).launch(ophip.LayerNormArgs(y.layout(), y.mem, x.layout(), x.mem, vec, wd, vec, bd, 1e-5), None, stream)
    assert_close_f16(y.fetch(stream, idx), oracle.layer_norm(np.empty_like(xs), xs, w, b, 1e-5), "layer_norm past 4 GiB")


def test_swiglu_gelu_and_add_past_4_gib(gpu, stream):
    n, d = SHAPES["narrow rows"]
    say("swiglu, gelu, add [%d, %d] f16" % (n, d))
    gate, up, out = Big(gpu, n, d, 4), Big(gpu, n, d, 5), Big(gpu, n, d, 6, fill=False)
    idx = sample_rows(n, d)
    gs, us = gate.rows(idx), up.rows(idx)
    ophip.Add(gpu).launch(ophip.AddArgs(out.layout(), out.mem, gate.layout(), gate.mem, up.layout(), up.mem), None, stream)
    assert np.array_equal(out.fetch(stream, idx).view(np.uint16), (gs + us).view(np.uint16)), "add past 4 GiB"
    ophip.Swiglu(gpu).launch(ophip.SwigluArgs(gate.layout(), gate.mem, up.layout(), up.mem), None, stream)
    assert_close_f16(gate.fetch(stream, idx), oracle.swiglu(gs.copy(), us), "swiglu past 4 GiB")
    ophip.Gelu(gpu).launch(ophip.GeluArgs(up.layout(), up.mem), None, stream)
    assert_close_f16(up.fetch(stream, idx), oracle.gelu(us.copy()), "gelu past 4 GiB")


def test_rope_and_softmax_past_4_gib(gpu, stream):
    n, d = SHAPES["wide rows"]
    nh, dh = d // 128, 128
    say("rope [%d, %d, %d], softmax [%d, 8, %d] f16" % (n, nh, dh, n // 8, d))
    t = Big(gpu, n, d, 7)
    pos = (np.arange(n, dtype=np.uint64) * 7 % 4099).astype(np.uint32)
    pd = gpu.from_host(pos)
    idx = sample_rows(n, d)
    ts = t.rows(idx)
    empty = TensorLayout(dt.F16, [0, dh], [2 * dh, 2])
    ophip.Rope(gpu).launch(ophip.RopeArgs(TensorLayout.new_contiguous(dt.F16, [n, nh, dh]), t.mem, TensorLayout.new_contiguous(dt.U32, [n]), pd,
                                          empty, None, empty, None, 1e4), None, stream)
    ref = oracle.rope(ts.reshape(len(idx), nh, dh).copy(), pos[idx], 1e4).reshape(len(idx), d)
    assert_close_f16(t.fetch(stream, idx), ref, "rope past 4 GiB")
    # the same memory as n rows of d scores (what rope left there: the reference result, up to the bar)
    before = t.fetch(stream, idx)
    ophip.FusedSoftmax(gpu).launch(ophip.FusedSoftmaxArgs(ophip.AttnMask.NONE, TensorLayout.new_contiguous(dt.F16, [n // 8, 8, d]), t.mem), None, stream)
    ref = oracle.fused_softmax(before.copy().reshape(len(idx), 1, d), causal=False).reshape(len(idx), d)
    assert_close_f16(t.fetch(stream, idx), ref, "softmax past 4 GiB")


def test_rearrange_past_4_gib(gpu, stream):
    """[n / 16, 16, d] -> [16, n / 16, d]: whole rows move across the 4 GiB line in both directions."""
    n, d = SHAPES["narrow rows"]
    say("rearrange [%d, 16, %d] -> [16, %d, %d] f16" % (n // 16, d, n // 16, d))
    src, dst = Big(gpu, n, d, 8), Big(gpu, n, d, 9, fill=False)
    s0 = n // 16
    ophip.Rearrange(gpu).launch(ophip.RearrangeArgs(TensorLayout(dt.F16, [s0, 16, d], [d * 2, s0 * d * 2, 2]), dst.mem,
                                                    TensorLayout.new_contiguous(dt.F16, [s0, 16, d]), src.mem), None, stream)
    idx = sample_rows(n, d)  # rows of the destination: row j * s0 + i holds the source's row i * 16 + j
    assert np.array_equal(dst.fetch(stream, idx).view(np.uint16), src.rows((idx % s0) * 16 + idx // s0).view(np.uint16)), "rearrange past 4 GiB"


def rel_error(got, ref):
    """against the magnitude a row of the product reaches, as the mat_mul parity tests measure it"""
    err = np.abs(got - ref)
    return float((err / np.maximum(np.abs(ref), np.abs(ref).mean())).max())


def test_mat_mul_weight_past_4_gib(gpu, stream):
    """c[16, N] = a[16, K] . W[K, N] with a 4.5 GiB weight (the decode-shaped product of a very wide layer):
    W[k, j] = T[(7919 k + j) mod L] for a random table T (a row is a run of the table, so filling is copying), and no
    element 2^31, 2^32 or 2^33 bytes or elements further on holds the same place of the table."""
    m, k, n, L, P = 16, 16384, 147456, 1000003, 7919
    say("mat_mul 16 x %d . %d x %d f16" % (k, k, n))
    assert all((b // n * P + b % n) % L for b in (2 ** 30, 2 ** 31, 2 ** 32, 2 ** 33))
    rng = np.random.default_rng(10)
    table = (rng.standard_normal(L).astype(f32) * f32(0.05)).astype(f16)
    w = gpu.malloc(k * n * 2)
    twice = np.concatenate([table, table])
    for k0 in range(0, k, 256):
        gpu.upload(w, np.stack([twice[kk * P % L:kk * P % L + n] for kk in range(k0, min(k, k0 + 256))]), offset=k0 * n * 2)
    a = rng.standard_normal((m, k)).astype(f32).astype(f16)
    ad, cd = gpu.from_host(a), gpu.malloc(m * n * 2)
    lay = lambda r, c: TensorLayout.new_contiguous(dt.F16, [1, r, c])
    op = ophip.MatMul(gpu)
    args = ophip.MatMulArgs(lay(m, n), cd, 0.0, lay(m, k), ad, lay(k, n), w, 1.0)
    say("  kernel: " + op.describe(args))
    op.launch(args, None, stream)
    got = gpu.to_host(cd, f16, m * n, stream=stream).reshape(m, n)
    cols = np.array(sorted({0, 1, n - 2, n - 1} | {int(x) for x in rng.integers(0, n, 96)}
                           | {(b // 2) % n + o for b in (2 ** 31, 2 ** 32, 2 ** 33) for o in (-1, 0, 1)}), dtype=np.int64)
    cols = cols[(cols >= 0) & (cols < n)]
    wc = table[(np.arange(k, dtype=np.int64)[:, None] * P + cols[None, :]) % L].astype(np.float64)
    assert rel_error(got[:, cols].astype(np.float64), a.astype(np.float64) @ wc) <= 1e-2


def test_mat_mul_rows_past_4_gib(gpu, stream):
    """C[M, 128] = A[M, 2048] . B[2048, 128] with a 4.6 GiB A (a long prefill batch through a narrow projection)."""
    m, k, n = 1200000, 2048, 128
    say("mat_mul %d x %d . %d x %d f16" % (m, k, k, n))
    a = Big(gpu, m, k, 11)
    rng = np.random.default_rng(12)
    b = (rng.standard_normal((k, n)).astype(f32) * f32(0.05)).astype(f16)
    bd, cd = gpu.from_host(b), gpu.malloc(m * n * 2)
    lay = lambda r, c: TensorLayout.new_contiguous(dt.F16, [1, r, c])
    op = ophip.MatMul(gpu)
    args = ophip.MatMulArgs(lay(m, n), cd, 0.0, lay(m, k), a.mem, lay(k, n), bd, 1.0)
    say("  kernel: " + op.describe(args))
    op.launch(args, None, stream)
    idx = sample_rows(m, k)
    got = np.stack([gpu.to_host(cd, f16, n, offset=int(r) * n * 2, stream=stream) for r in idx]).astype(np.float64)
    assert rel_error(got, a.rows(idx).astype(np.float64) @ b.astype(np.float64)) <= 1e-2


def test_attention_kv_cached_caches_past_4_gib(gpu, stream):
    """40 heads of 480000 cached tokens of 128 (4.6 GiB for either cache), ten new tokens appended at the end: the
    appended rows are read back, and the results of the heads at the caches' ends and around 2 and 4 GiB are compared with softmax(q k^T / sqrt(dh)) v in f64."""
    nh = nkvh = 40
    seq, dh, buf = 10, 128, 480000
    pos = buf - seq
    say("attention_kv_cached nh=%d seq=%d dh=%d buf=%d pos=%d" % (nh, seq, dh, buf, pos))
    kc, vc = Big(gpu, nkvh * buf, dh, 13), Big(gpu, nkvh * buf, dh, 14)
    rng = np.random.default_rng(15)
    # q eight times the usual size: the scores then single out a few of the 480000 keys, and the result is of the
    # size of single v rows instead of their average (which would be near zero whatever the kernel read)
    q, k, v = ((rng.standard_normal(s).astype(f32) * f32(m)).astype(f16) for s, m in (((nh, seq, dh), 8), ((nkvh, seq, dh), 1), ((nkvh, seq, dh), 1)))
    qd, kd, vd, od = gpu.from_host(q), gpu.from_host(k), gpu.from_host(v), gpu.malloc(q.nbytes)
    c = lambda *shape: TensorLayout.new_contiguous(dt.F16, list(shape))
    op = ophip.AttnKVCached(gpu)
    args = ophip.AttnKVCachedArgs(c(nh, seq, dh), qd, c(nkvh, seq, dh), kd, c(nkvh, seq, dh), vd, c(nh, seq, dh), od,
                                  c(nkvh, buf, dh), kc.mem, c(nkvh, buf, dh), vc.mem, ophip.AttnMask.CAUSAL, pos)
    op.scheme(args, 2 ** 40)
    op.launch(args, None, stream)
    out = gpu.to_host(od, f16, q.size, stream=stream).reshape(q.shape)
    for h in (0, nkvh // 2, nkvh - 1):  # the appended rows, where the caches start, cross 4 GiB and end
        rows = np.arange(h * buf + pos, h * buf + pos + seq)
        assert np.array_equal(kc.fetch(stream, rows), k[h]) and np.array_equal(vc.fetch(stream, rows), v[h])
        before = np.arange(h * buf + pos - 2, h * buf + pos)
        assert np.array_equal(kc.fetch(stream, before), kc.rows(before)) and np.array_equal(vc.fetch(stream, before), vc.rows(before))
    for h in (0, 1, 17, 18, 34, 35, nh - 1):  # the 2 GiB and 4 GiB lines run through the caches of heads 17 and 34
        rows = np.arange(h * buf, h * buf + pos)
        keys = np.concatenate([kc.rows(rows), k[h]]).astype(np.float64)
        vals = np.concatenate([vc.rows(rows), v[h]]).astype(np.float64)
        scores = q[h].astype(np.float64) @ keys.T / np.sqrt(dh)
        for i in range(seq):
            scores[i, pos + i + 1:] = -np.inf
        p = np.exp(scores - scores.max(axis=1, keepdims=True))
        ref = (p / p.sum(axis=1, keepdims=True)) @ vals
        assert np.abs(ref).max() > 0.25  # (the comparison below means something)
        assert_close_f16(out[h], ref, "attention_kv_cached past 4 GiB, head %d" % h)


def test_batched_mat_mul_whose_batches_lie_past_4_gib(gpu, stream):
    """q . K^T through mat_mul over a 4.6 GiB K cache (40 heads of 480000 keys of 128, K-contiguous): the batch stride
    carries the later heads past 2^32 bytes.  K[h, j, :] = T[(131 h + 7 j + 13 t) mod L] for a random table T."""
    nh, seq, dh, buf, L = 40, 16, 128, 480000, 1000003
    say("mat_mul %d x (%d x %d . %d x %d), B stored [N, K]" % (nh, seq, dh, dh, buf))
    rng = np.random.default_rng(16)
    table = rng.standard_normal(L).astype(f32).astype(f16)

    def keys(h, j):
        j = np.asarray(j, dtype=np.int64)
        return table[(h * 131 + j[:, None] * 7 + np.arange(dh, dtype=np.int64)[None, :] * 13) % L]

    kc = gpu.malloc(nh * buf * dh * 2)
    piece = 120000  # keys per upload; a piece's places in the table are one piece's moved on by 131 h + 7 j0
    twice = np.concatenate([table, table])
    first = (np.arange(piece, dtype=np.int64)[:, None] * 7 + np.arange(dh, dtype=np.int64)[None, :] * 13) % L
    for h in range(nh):
        for j0 in range(0, buf, piece):
            gpu.upload(kc, twice[first + (h * 131 + j0 * 7) % L], offset=(h * buf + j0) * dh * 2)
    q = rng.standard_normal((nh, seq, dh)).astype(f32).astype(f16)
    qd, cd = gpu.from_host(q), gpu.malloc(nh * seq * buf * 2)
    op = ophip.MatMul(gpu)
    args = ophip.MatMulArgs(TensorLayout.new_contiguous(dt.F16, [nh, seq, buf]), cd, 0.0, TensorLayout.new_contiguous(dt.F16, [nh, seq, dh]), qd,
                            TensorLayout(dt.F16, [nh, dh, buf], [buf * dh * 2, 2, dh * 2]), kc, 0.125)
    say("  kernel: " + op.describe(args))
    op.launch(args, None, stream)
    stream.synchronize()
    for h in (0, 1, 17, 18, 34, 35, 39):  # the 2 GiB and 4 GiB lines run through the keys of heads 17 and 34
        js = sorted({0, 1, buf - 2, buf - 1} | {int(x) for x in rng.integers(0, buf, 40)})
        ref = 0.125 * q[h].astype(np.float64) @ keys(h, js).astype(np.float64).T
        got = np.array([[gpu.to_host(cd, f16, 1, offset=((h * seq + i) * buf + j) * 2, stream=stream)[0] for j in js] for i in range(seq)])
        assert rel_error(got.astype(np.float64), ref) <= 1e-2, h
