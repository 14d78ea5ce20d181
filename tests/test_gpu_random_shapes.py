"""Seeded sweeps over random shapes and row paddings for every operator, against the oracle.
Each device tensor sits inside a buffer with 4 KiB of guard bytes on both sides and random
padding between rows; after the launch everything outside the tensor's elements must be
unchanged, so a stray store is caught as a failed assertion."""
import os

import numpy as np
import pytest

import ophip
import oracle
from helpers import assert_close_f16, normal_f16
from ophip import TensorLayout, dt

pytestmark = pytest.mark.gpu

f16, f32 = np.float16, np.float32
GUARD = 4096
# OPHIP_TEST_SWEEPS=<n> repeats every sweep with n different seeds (default 1)
SWEEPS = pytest.mark.parametrize("sweep", range(int(os.environ.get("OPHIP_TEST_SWEEPS", "1"))))


def say(msg):
    print(msg, flush=True)


class Guarded:
    """A [rows.., cols] tensor with row pitch `cols + pad` elements inside guard bytes."""

    def __init__(self, gpu, rng, shape, dtype, pad, fill=None, scale=1.0):
        self.gpu, self.shape, self.dtype = gpu, tuple(shape), np.dtype(dtype)
        lead = int(np.prod(shape[:-1])) if len(shape) > 1 else 1
        pitch = shape[-1] + pad
        n = lead * pitch
        body = (rng.standard_normal(n).astype(f32) * f32(scale)).astype(dtype) if fill is None else np.full(n, fill, dtype)
        raw = np.concatenate([rng.integers(0, 256, GUARD, dtype=np.uint8), body.view(np.uint8),
                              rng.integers(0, 256, GUARD, dtype=np.uint8)])
        self.raw = raw
        it = self.dtype.itemsize
        strides = [it]
        mul = pitch * it
        for d in reversed(shape[:-1]):
            strides.append(mul)
            mul *= d
        self.strides = tuple(reversed(strides))
        self.mem = gpu.from_host(raw)
        self.ptr = self.mem.ptr + GUARD
        self.layout = TensorLayout(ophip.NP_DT[self.dtype], list(shape), list(self.strides))

    def view(self, raw=None):
        raw = self.raw if raw is None else raw
        return np.lib.stride_tricks.as_strided(raw[GUARD:].view(self.dtype), self.shape, self.strides, writeable=True)

    def fetch(self, stream):
        """Device contents; asserts that nothing outside the tensor's elements changed."""
        got = self.gpu.to_host(self.mem, np.uint8, self.raw.size, stream=stream)
        mask = np.ones(self.raw.size, bool)
        inside = np.lib.stride_tricks.as_strided(mask[GUARD:].view(np.uint8), tuple(self.shape) + (self.dtype.itemsize,),
                                                 self.strides + (1,), writeable=True)
        inside[...] = 0
        assert np.array_equal(got[mask.view(bool)], self.raw[mask.view(bool)]), "bytes outside the tensor were written"
        return self.view(got)


@SWEEPS
def test_random_rms_norm_and_layer_norm(gpu, stream, sweep):
    rng = np.random.default_rng(100 + 1000 * sweep)
    rms, ln = ophip.RmsNorm(gpu), ophip.LayerNorm(gpu)
    for case in range(30):
        n = int(rng.integers(1, 70))
        d = int(rng.choice([8, 24, 120, 128, 1000, 1024, 4096, 4104, 5000, 8192, 16384, 16400]))
        adt, wdt = (f16, f16) if case % 3 == 0 else (f16, f32) if case % 3 == 1 else (f32, f32)
        pad = int(rng.choice([0, 8, 3]))
        x, y = Guarded(gpu, rng, (n, d), adt, pad), Guarded(gpu, rng, (n, d), adt, int(rng.choice([0, 8])))
        w, b = Guarded(gpu, rng, (d,), wdt, 0), Guarded(gpu, rng, (d,), wdt, 0)
        say("random rms_norm/layer_norm %d: n=%d d=%d pad=%d %s/%s" % (case, n, d, pad, adt.__name__, wdt.__name__))
        rms.launch(ophip.RmsNormArgs(y.layout, y.ptr, x.layout, x.ptr, w.layout, w.ptr, 1e-5), None, stream)
        got = y.fetch(stream)
        ref = oracle.rms_norm(np.empty((n, d), adt), x.view(), w.view(), 1e-5)
        if adt is f16: assert_close_f16(got, ref, "rms_norm")
        else: np.testing.assert_allclose(got, ref, rtol=3e-5, atol=3e-6)
        ln.launch(ophip.LayerNormArgs(y.layout, y.ptr, x.layout, x.ptr, w.layout, w.ptr, b.layout, b.ptr, 1e-5), None, stream)
        got = y.fetch(stream)
        ref = oracle.layer_norm(np.empty((n, d), adt), x.view(), w.view(), b.view(), 1e-5)
        if adt is f16: assert_close_f16(got, ref, "layer_norm", abs_tol=4e-3)
        else: np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-4)


@SWEEPS
def test_random_softmax_swiglu_gelu(gpu, stream, sweep):
    rng = np.random.default_rng(101 + 1000 * sweep)
    sm, sw, ge = ophip.FusedSoftmax(gpu), ophip.Swiglu(gpu), ophip.Gelu(gpu)
    for case in range(30):
        nh, seq = int(rng.integers(1, 5)), int(rng.integers(1, 20))
        att = seq + int(rng.choice([0, 1, 7, 100, 500, 2040, 2049, 5000]))
        pad = int(rng.choice([0, 8, 5]))
        a = Guarded(gpu, rng, (nh, seq, att), f16, pad, scale=2.0)
        mask = ophip.AttnMask.CAUSAL if case % 4 else ophip.AttnMask.NONE
        say("random softmax %d: nh=%d seq=%d att=%d pad=%d mask=%d" % (case, nh, seq, att, pad, mask))
        sm.launch(ophip.FusedSoftmaxArgs(mask, a.layout, a.ptr), None, stream)
        got = a.fetch(stream)
        ref = oracle.fused_softmax(a.view().copy(), causal=bool(mask))
        assert_close_f16(got, ref, "softmax")
        assert np.array_equal(got == 0, ref == 0)
        n, d = int(rng.integers(1, 40)), int(rng.choice([8, 40, 1001, 2048, 11008]))
        g, u = Guarded(gpu, rng, (n, d), f16, pad, scale=2.0), Guarded(gpu, rng, (n, d), f16, int(rng.choice([0, 8])))
        say("random swiglu/gelu %d: n=%d d=%d" % (case, n, d))
        sw.launch(ophip.SwigluArgs(g.layout, g.ptr, u.layout, u.ptr), None, stream)
        assert_close_f16(g.fetch(stream), oracle.swiglu(g.view().copy(), u.view()), "swiglu")
        ge.launch(ophip.GeluArgs(u.layout, u.ptr), None, stream)
        assert_close_f16(u.fetch(stream), oracle.gelu(u.view().copy()), "gelu")


@SWEEPS
def test_random_rope(gpu, stream, sweep):
    rng = np.random.default_rng(102 + 1000 * sweep)
    rope = ophip.Rope(gpu)
    for case in range(20):
        nt, nh = int(rng.integers(1, 40)), int(rng.integers(1, 9))
        dh = int(rng.choice([2, 8, 20, 64, 128, 256]))
        pad = int(rng.choice([0, 8, 2]))
        t = Guarded(gpu, rng, (nt, nh, dh), f16, pad)
        pdt = np.uint32 if case % 2 else np.uint64
        pos = rng.integers(0, 5000, nt).astype(pdt)
        pd = gpu.from_host(pos)
        empty = TensorLayout(dt.F16, [0, dh], [2 * dh, 2])
        say("random rope %d: nt=%d nh=%d dh=%d pad=%d %s" % (case, nt, nh, dh, pad, pdt.__name__))
        rope.launch(ophip.RopeArgs(t.layout, t.ptr, TensorLayout.of(pos), pd, empty, None, empty, None, 1e4), None, stream)
        assert_close_f16(t.fetch(stream), oracle.rope(t.view().copy(), pos, 1e4), "rope")


@SWEEPS
def test_random_rearrange_and_add(gpu, stream, sweep):
    rng = np.random.default_rng(103 + 1000 * sweep)
    re, ad = ophip.Rearrange(gpu), ophip.Add(gpu)
    for case in range(30):
        nd = int(rng.integers(1, 5))
        shape = [int(rng.integers(1, 9)) for _ in range(nd - 1)] + [int(rng.choice([1, 3, 8, 16, 40]))]
        perm = list(rng.permutation(nd))
        src = Guarded(gpu, rng, shape, f16, int(rng.choice([0, 8, 1])))
        dst_store = Guarded(gpu, rng, [shape[p] for p in perm], f16, int(rng.choice([0, 8])), fill=0)
        inv = list(np.argsort(perm))
        dst_layout = TensorLayout(dt.F16, shape, [dst_store.strides[inv[i]] for i in range(nd)])
        say("random rearrange %d: shape=%s perm=%s" % (case, shape, perm))
        re.launch(ophip.RearrangeArgs(dst_layout, dst_store.ptr, src.layout, src.ptr), None, stream)
        got = dst_store.fetch(stream)
        assert np.array_equal(got.view(np.uint16), src.view().transpose(perm).view(np.uint16))
        b = Guarded(gpu, rng, shape, f16, int(rng.choice([0, 8])))
        c = Guarded(gpu, rng, shape, f16, int(rng.choice([0, 8])), fill=0)
        bl = b.layout
        if nd > 1 and case % 3 == 0:  # broadcast b over the first dimension
            bl = TensorLayout(dt.F16, shape, [0] + list(b.strides[1:]))
        say("random add %d" % case)
        ad.launch(ophip.AddArgs(c.layout, c.ptr, src.layout, src.ptr, bl, b.ptr), None, stream)
        bv = b.view() if bl is b.layout else np.broadcast_to(b.view()[:1], shape)
        assert np.array_equal(c.fetch(stream), (src.view().astype(f32) + bv.astype(f32)).astype(f16))


@SWEEPS
def test_random_mat_mul(gpu, stream, sweep):
    """Shapes straddle the kernel boundaries: 64 / 65 rows, widths that are not multiples of 8 or 128, K that is
    not a multiple of 32, tile-sized multiples of 128 / 256, batches with broadcast b."""
    rng = np.random.default_rng(104 + 1000 * sweep)
    mm = ophip.MatMul(gpu)
    oracle.set_threads(8)
    try:
        for case in range(40):
            m = int(rng.choice([1, 5, 16, 17, 33, 64, 65, 100, 128, 256, 384]))
            n = int(rng.choice([8, 24, 100, 128, 136, 256, 512, 1000]))
            k = int(rng.choice([1, 7, 32, 64, 96, 100, 128, 512, 1000]))
            bt = int(rng.choice([1, 1, 2, 3]))
            ta, tb, tc = (bool(rng.integers(0, 2)) for _ in range(3))
            pa, pb, pc = (int(rng.choice([0, 8])) for _ in range(3))
            A = Guarded(gpu, rng, (bt, k, m) if ta else (bt, m, k), f16, pa)
            B = Guarded(gpu, rng, (bt, n, k) if tb else (bt, k, n), f16, pb, scale=0.1)
            C = Guarded(gpu, rng, (bt, n, m) if tc else (bt, m, n), f16, pc)
            tr = lambda g, t: (TensorLayout(dt.F16, [g.shape[0], g.shape[2], g.shape[1]], [g.strides[0], g.strides[2], g.strides[1]]),
                               g.view().transpose(0, 2, 1)) if t else (g.layout, g.view())
            (al, av), (bl, bv), (cl, cv) = tr(A, ta), tr(B, tb), tr(C, tc)
            if bt > 1 and case % 4 == 0:  # one b for every batch
                bl = TensorLayout(dt.F16, bl.shape, [0] + list(bl.strides[1:]))
                bv = np.broadcast_to(bv[:1], bv.shape)
            alpha, beta = float(rng.choice([1.0, 0.5, -1.25])), float(rng.choice([0.0, 1.0, 0.5]))
            args = ophip.MatMulArgs(cl, C.ptr, beta, al, A.ptr, bl, B.ptr, alpha)
            say("random mat_mul %d: bt=%d m=%d n=%d k=%d t=%d%d%d pads=%d%d%d a=%g b=%g [%s]" % (
                case, bt, m, n, k, ta, tb, tc, pa, pb, pc, alpha, beta, mm.describe(args)))
            ref = cv.copy()
            oracle.mat_mul(ref, beta, av, np.ascontiguousarray(bv) if bv.strides[0] == 0 and bt > 1 else bv, alpha)
            mm.launch(args, None, stream)
            got = C.fetch(stream)
            got = got.transpose(0, 2, 1) if tc else got
            scale = float(np.abs(ref.astype(np.float64)).max()) + 1e-3
            err = np.abs(got.astype(np.float64) - ref.astype(np.float64)).max()
            assert err <= 2e-3 + 4e-3 * scale, (err, scale)
    finally:
        oracle.set_threads(1)


@SWEEPS
def test_random_mat_mul_tile_shapes(gpu, stream, monkeypatch, sweep):
    """Shapes the LDS-tiled MFMA kernels take: multiples of 128 / 256 with K-steps of 32 and 64, one to many
    steps, few tiles with a long K (split K), padded rows, every operand layout, batches.  Every third case
    keeps the 256 x 256 tile, which the library would only choose for much larger outputs."""
    rng = np.random.default_rng(105 + 1000 * sweep)
    mm = ophip.MatMul(gpu)
    oracle.set_threads(8)
    seen = set()
    try:
        for case in range(12):
            big = case % 3 == 0
            if big:
                monkeypatch.setenv("OPHIP_GEMM_TILE", "256")
                mm = ophip.MatMul(gpu)  # the knob is read when an operator is created
                m, n = int(rng.choice([256, 512, 768])), int(rng.choice([256, 512, 1024]))
                k = int(rng.choice([64, 128, 192, 1088, 2048]))
            else:
                monkeypatch.delenv("OPHIP_GEMM_TILE", raising=False)
                mm = ophip.MatMul(gpu)
                m = int(rng.choice([128, 256, 384, 512, 1024]))
                n = int(rng.choice([128, 256, 384, 768, 1024]))
                k = int(rng.choice([32, 64, 96, 192, 1056, 2048]))
            bt = int(rng.choice([1, 1, 2]))
            ta, tb, tc = (bool(rng.integers(0, 2)) for _ in range(3))
            pa, pb, pc = (int(rng.choice([0, 8])) for _ in range(3))
            A = Guarded(gpu, rng, (bt, k, m) if ta else (bt, m, k), f16, pa, scale=0.25)
            B = Guarded(gpu, rng, (bt, n, k) if tb else (bt, k, n), f16, pb, scale=0.25)
            C = Guarded(gpu, rng, (bt, n, m) if tc else (bt, m, n), f16, pc)
            tr = lambda g, t: (TensorLayout(dt.F16, [g.shape[0], g.shape[2], g.shape[1]], [g.strides[0], g.strides[2], g.strides[1]]),
                               g.view().transpose(0, 2, 1)) if t else (g.layout, g.view())
            (al, av), (bl, bv), (cl, cv) = tr(A, ta), tr(B, tb), tr(C, tc)
            alpha, beta = float(rng.choice([1.0, 0.5])), float(rng.choice([0.0, 1.0, 0.5]))
            args = ophip.MatMulArgs(cl, C.ptr, beta, al, A.ptr, bl, B.ptr, alpha)
            what = mm.describe(args)
            seen.add(what.split()[0])
            say("random tile mat_mul %d: bt=%d m=%d n=%d k=%d t=%d%d%d pads=%d%d%d a=%g b=%g [%s]" % (
                case, bt, m, n, k, ta, tb, tc, pa, pb, pc, alpha, beta, what))
            assert what.startswith("tile256" if big else "tile128"), what
            ref = cv.copy()
            oracle.mat_mul(ref, beta, av, bv, alpha)
            mm.launch(args, None, stream)
            got = C.fetch(stream)
            got = got.transpose(0, 2, 1) if tc else got
            scale = float(np.abs(ref.astype(np.float64)).max()) + 1e-3
            err = np.abs(got.astype(np.float64) - ref.astype(np.float64)).max()
            assert err <= 2e-3 + 4e-3 * scale, (err, scale)
    finally:
        oracle.set_threads(1)
    say("tile kernels exercised: %s" % sorted(seen))


@SWEEPS
def test_random_mat_mul_ragged_tile_shapes(gpu, stream, monkeypatch, sweep):
    """More than 64 rows and columns that are no multiples of the 128 tile: the last tiles of the MFMA kernel load
    clamped rows and store only what exists (guard zones around C catch a store past M or N).  Two thirds of the
    cases have M and N in multiples of 8 with every operand layout; the others an odd M with A and C row-major
    (nothing is contiguous along M then).  Some have few tiles and a long K (split K over ragged tiles).  Every
    fourth case keeps the 256 x 256 tile, which the library would only choose for much larger outputs.  Half of
    the cases have a K that is no multiple of the kernel's K-step, some of them odd (rows along K are then
    padded to whole groups of 8, which is what the kernel's 16-byte loads need)."""
    rng = np.random.default_rng(731 + 1000 * sweep)
    mm = ophip.MatMul(gpu)
    oracle.set_threads(8)
    try:
        for case in range(24):
            odd_m = case % 3 == 2
            big = case % 4 == 1
            if big:
                monkeypatch.setenv("OPHIP_GEMM_TILE", "256")
            else:
                monkeypatch.delenv("OPHIP_GEMM_TILE", raising=False)
            mm = ophip.MatMul(gpu)  # the knob is read when an operator is created
            n = 8 * int(rng.integers(9, 90))
            m = 2 * int(rng.integers(33, 350)) + 1 if odd_m else 8 * int(rng.integers(9, 90))
            if case % 2 == 0:
                k = int(rng.choice([64, 192, 1088, 2048]) if big else rng.choice([32, 64, 96, 192, 1056, 2048, 4096]))
            else:
                k = int(rng.choice([72, 100, 136, 509, 1000, 2056, 4095]))
            bt = int(rng.choice([1, 1, 2]))
            ta, tb, tc = (bool(rng.integers(0, 2)) for _ in range(3))
            if odd_m:
                ta = tc = False
            sa, sb, sc = ((bt, k, m) if ta else (bt, m, k)), ((bt, n, k) if tb else (bt, k, n)), ((bt, n, m) if tc else (bt, m, n))
            pa, pb, pc = ((-sh[-1]) % 8 + int(rng.choice([0, 8])) for sh in (sa, sb, sc))
            A = Guarded(gpu, rng, sa, f16, pa, scale=0.25)
            B = Guarded(gpu, rng, sb, f16, pb, scale=0.25)
            C = Guarded(gpu, rng, sc, f16, pc)
            tr = lambda g, t: (TensorLayout(dt.F16, [g.shape[0], g.shape[2], g.shape[1]], [g.strides[0], g.strides[2], g.strides[1]]),
                               g.view().transpose(0, 2, 1)) if t else (g.layout, g.view())
            (al, av), (bl, bv), (cl, cv) = tr(A, ta), tr(B, tb), tr(C, tc)
            alpha, beta = float(rng.choice([1.0, 0.5])), float(rng.choice([0.0, 1.0, 0.5]))
            args = ophip.MatMulArgs(cl, C.ptr, beta, al, A.ptr, bl, B.ptr, alpha)
            what = mm.describe(args)
            say("random ragged mat_mul %d: bt=%d m=%d n=%d k=%d t=%d%d%d pads=%d%d%d a=%g b=%g [%s]" % (
                case, bt, m, n, k, ta, tb, tc, pa, pb, pc, alpha, beta, what))
            assert what.startswith("tile256" if big else "tile128") and "ragged" in what, what
            ref = cv.copy()
            oracle.mat_mul(ref, beta, av, bv, alpha)
            mm.launch(args, None, stream)
            got = C.fetch(stream)
            got = got.transpose(0, 2, 1) if tc else got
            scale = float(np.abs(ref.astype(np.float64)).max()) + 1e-3
            err = np.abs(got.astype(np.float64) - ref.astype(np.float64)).max()
            assert err <= 2e-3 + 4e-3 * scale, (err, scale)
    finally:
        oracle.set_threads(1)


@SWEEPS
def test_random_attention_one_pass(gpu, stream, monkeypatch, sweep):
    """attention on the one-pass kernel (both builds) over random head counts, groupings, row and key counts and row
    paddings, against the f64 formula; nothing outside o and q (which receives the result too) may change."""
    rng = np.random.default_rng(800 + 1000 * sweep)
    monkeypatch.setenv("OPHIP_ATTN_FUSED", "1")
    ops = {}
    for split in ("0", "1"):
        monkeypatch.setenv("OPHIP_ATTN_KEYSPLIT", split)
        ops[split] = ophip.Attention(gpu)
    for case in range(16):
        dh = int(rng.choice([64, 128]))
        nkvh = int(rng.choice([1, 2, 3, 5]))
        nh = nkvh * int(rng.choice([1, 2, 4]))
        seq = int(rng.choice([1, 31, 64, 100, 128, 129, 200, 333]))
        causal = bool(rng.integers(0, 2))
        att = seq + int(rng.choice([0, 0, 1, 63, 64, 130])) if causal else int(rng.choice([1, 17, 64, 65, 200, 384]))
        pq, pk, pv, po = (int(rng.choice([0, 8, 24])) for _ in range(4))
        Q, K, V = Guarded(gpu, rng, (nh, seq, dh), f16, pq), Guarded(gpu, rng, (nkvh, att, dh), f16, pk), Guarded(gpu, rng, (nkvh, att, dh), f16, pv)
        O = Guarded(gpu, rng, (nh, seq, dh), f16, po, fill=0)
        split = "01"[case % 2]
        say("random attention %d: nh=%d nkvh=%d seq=%d att=%d dh=%d causal=%s pads=%d %d %d %d split=%s" % (
            case, nh, nkvh, seq, att, dh, causal, pq, pk, pv, po, split))
        q, k, v = Q.view().copy(), K.view().copy(), V.view().copy()
        args = ophip.AttentionArgs(Q.layout, Q.ptr, K.layout, K.ptr, V.layout, V.ptr, O.layout, O.ptr,
                                   ophip.AttnMask.CAUSAL if causal else ophip.AttnMask.NONE)
        ops[split].launch(args, None, stream)
        got = O.fetch(stream)
        g = nh // nkvh
        kk, vv = np.repeat(k.astype(np.float64), g, axis=0), np.repeat(v.astype(np.float64), g, axis=0)
        s = np.einsum("hsd,had->hsa", q.astype(np.float64), kk) / np.sqrt(dh)
        if causal:
            s = np.where((np.arange(att)[None, :] <= (att - seq + np.arange(seq))[:, None])[None], s, -np.inf)
        pr = np.exp(s - s.max(-1, keepdims=True))
        ref = np.einsum("hsa,had->hsd", pr / pr.sum(-1, keepdims=True), vv)
        assert_close_f16(got, ref, "random attention")
        assert np.array_equal(K.fetch(stream), k) and np.array_equal(V.fetch(stream), v)
        # padded rows still follow each other head after head: heads and tokens fold into one dimension, and the reference
        # then leaves att . v in q
        assert np.array_equal(Q.fetch(stream), got)


def random_view(rng, base):
    """A view of `base` reached by slicing with steps (negative ones too), dropping and permuting axes: every address
    inside `base`, no two elements at one address."""
    idx = []
    for n in base.shape:
        kind = rng.integers(0, 4)
        if kind == 0 or n == 1:
            idx.append(slice(None))
        else:
            a, b = sorted(int(x) for x in rng.integers(0, n + 1, 2))
            if a == b:
                a, b = 0, n
            step = int(rng.choice([1, 1, 2, 3]))
            idx.append(slice(a, b, step) if kind != 3 else slice(b - 1, a - 1 if a > 0 else None, -step))
    v = base[tuple(idx)]
    return v.transpose(list(rng.permutation(v.ndim)))


@SWEEPS
def test_random_rearrange_between_arbitrary_views(gpu, stream, sweep):
    """rearrange between views that numpy can describe and the structured tests do not reach: elements of 1, 2, 4 and 8
    bytes, steps, negative strides, a source broadcast along an axis, bases that are only element-aligned.  numpy's
    own assignment between the same two views is the expected result; everything outside the destination view must
    keep its bytes."""
    rng = np.random.default_rng(211 + 1000 * sweep)
    op = ophip.Rearrange(gpu)
    types = {1: (np.uint8, dt.U8), 2: (np.uint16, dt.U16), 4: (np.uint32, dt.U32), 8: (np.uint64, dt.U64)}
    done = 0
    for case in range(60):
        size = int(rng.choice([1, 2, 2, 4, 8]))
        ntype, code = types[size]
        nd = int(rng.integers(1, 5))
        dst_base = rng.integers(0, 256, [int(rng.integers(1, 10)) for _ in range(nd)] + [size], dtype=np.uint8).view(ntype)[..., 0]
        dst_view = random_view(rng, dst_base)
        # a source of the destination view's shape: a view of another base, some axes broadcast (stride 0)
        src_shape = [1 if (n > 1 and rng.integers(0, 5) == 0) else n for n in dst_view.shape]
        pad = [int(rng.integers(0, 3)) for _ in src_shape]
        src_base = rng.integers(0, 256, [n + p for n, p in zip(src_shape, pad)] + [size], dtype=np.uint8).view(ntype)[..., 0]
        src_view = src_base[tuple(slice(int(rng.integers(0, p + 1)), None) for p in pad)]
        src_view = src_view[tuple(slice(0, n) for n in src_shape)]
        if rng.integers(0, 3) == 0 and src_view.ndim:
            ax = int(rng.integers(0, src_view.ndim))
            src_view = np.flip(src_view, ax)
        src_view = np.broadcast_to(src_view, dst_view.shape)
        if dst_view.size == 0:
            continue
        dd, sd = gpu.from_host(dst_base), gpu.from_host(src_base)
        d_off = dst_view.__array_interface__["data"][0] - dst_base.__array_interface__["data"][0]
        s_off = src_view.__array_interface__["data"][0] - src_base.__array_interface__["data"][0]
        say("random views %d: %d-byte elements, shape %s, dst strides %s, src strides %s" % (case, size, dst_view.shape, dst_view.strides, src_view.strides))
        op.launch(ophip.RearrangeArgs(TensorLayout(code, list(dst_view.shape), list(dst_view.strides)), dd.ptr + d_off,
                                      TensorLayout(code, list(src_view.shape), list(src_view.strides)), sd.ptr + s_off), None, stream)
        want = dst_base.copy()
        want_view = np.lib.stride_tricks.as_strided(want.reshape(-1)[d_off // size:], dst_view.shape, dst_view.strides) if all(s >= 0 for s in dst_view.strides) else None
        if want_view is None:  # negative strides: the same view of the copy, by the same recipe relative to its own base
            want_view = np.ndarray(dst_view.shape, ntype, want.data, d_off, dst_view.strides)
        want_view[...] = src_view
        got = gpu.to_host(dd, ntype, dst_base.size, stream=stream).reshape(dst_base.shape)
        assert np.array_equal(got, want), case
        done += 1
    assert done > 40


def random_source(rng, shape, ntype, make):
    """A view of the given shape over a base of its own: padded, offset, some axes broadcast, one possibly flipped."""
    src_shape = [1 if (n > 1 and rng.integers(0, 5) == 0) else n for n in shape]
    pad = [int(rng.integers(0, 3)) for _ in src_shape]
    base = make([n + p for n, p in zip(src_shape, pad)])
    view = base[tuple(slice(int(rng.integers(0, p + 1)), None) for p in pad)]
    view = view[tuple(slice(0, n) for n in src_shape)]
    if rng.integers(0, 3) == 0 and view.ndim:
        view = np.flip(view, int(rng.integers(0, view.ndim)))
    return base, np.broadcast_to(view, shape)


@SWEEPS
def test_random_add_between_arbitrary_views(gpu, stream, sweep):
    """add with the three operands as unrelated views (steps, negative strides, broadcast a and b, element-aligned
    bases) in f16, f32, i32 and u8; numpy's sum of the same views is the expected result (f16: the f32 sum rounded
    once; integers wrap), and nothing outside c's view may change."""
    rng = np.random.default_rng(223 + 1000 * sweep)
    op = ophip.Add(gpu)
    kinds = [(f16, dt.F16), (f32, dt.F32), (np.int32, dt.I32), (np.uint8, dt.U8)]
    done = 0
    for case in range(48):
        ntype, code = kinds[int(rng.integers(0, len(kinds)))]
        if np.issubdtype(ntype, np.floating):
            make = lambda s: rng.standard_normal(s).astype(f32).astype(ntype)
        else:
            info = np.iinfo(ntype)
            make = lambda s: rng.integers(info.min, info.max, s, dtype=ntype, endpoint=True)
        nd = int(rng.integers(1, 5))
        c_base = make([int(rng.integers(1, 10)) for _ in range(nd)])
        c_view = random_view(rng, c_base)
        if c_view.size == 0:
            continue
        a_base, a_view = random_source(rng, c_view.shape, ntype, make)
        b_base, b_view = random_source(rng, c_view.shape, ntype, make)
        off = lambda v, b: v.__array_interface__["data"][0] - b.__array_interface__["data"][0]
        cd, ad, bd = gpu.from_host(c_base), gpu.from_host(a_base), gpu.from_host(b_base)
        lay = lambda v: TensorLayout(code, list(v.shape), list(v.strides))
        say("random add views %d: %s shape %s, c strides %s, a strides %s, b strides %s" % (case, ntype.__name__, c_view.shape, c_view.strides, a_view.strides, b_view.strides))
        op.launch(ophip.AddArgs(lay(c_view), cd.ptr + off(c_view, c_base), lay(a_view), ad.ptr + off(a_view, a_base), lay(b_view), bd.ptr + off(b_view, b_base)), None, stream)
        want = c_base.copy()
        want_view = np.ndarray(c_view.shape, ntype, want.data, off(c_view, c_base), c_view.strides)
        if ntype is f16:
            want_view[...] = (a_view.astype(f32) + b_view.astype(f32)).astype(f16)
        else:
            with np.errstate(over="ignore"):
                want_view[...] = a_view + b_view
        got = gpu.to_host(cd, ntype, c_base.size, stream=stream).reshape(c_base.shape)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), case
        done += 1
    assert done > 30


@SWEEPS
def test_random_add_rows_between_arbitrary_views(gpu, stream, sweep):
    """add_rows (dst[b, i, :] += src[idx[b, i], :]) with dst, src and idx as unrelated views: steps and negative strides
    in every dimension, the last one included; u32 and u64 indices; f16, f32 and i32 elements.  Expected: numpy on the
    same views, row by row, the sum formed as the operator's type forms it."""
    rng = np.random.default_rng(227 + 1000 * sweep)
    op = ophip.AddRows(gpu)
    kinds = [(f16, dt.F16), (f32, dt.F32), (np.int32, dt.I32)]
    for case in range(32):
        ntype, code = kinds[int(rng.integers(0, len(kinds)))]
        itype, icode = [(np.uint32, dt.U32), (np.uint64, dt.U64)][int(rng.integers(0, 2))]
        if np.issubdtype(ntype, np.floating):
            make = lambda s: rng.standard_normal(s).astype(f32).astype(ntype)
        else:
            make = lambda s: rng.integers(-2 ** 31, 2 ** 31 - 1, s, dtype=ntype, endpoint=True)
        batch, m, n, k = (int(rng.integers(1, 5)), int(rng.integers(1, 7)), int(rng.choice([1, 3, 8, 24, 40])), int(rng.integers(1, 9)))

        def strided(shape, make_):
            """a view of `shape` inside a larger base: a random step and direction per axis"""
            steps = [int(rng.choice([1, 1, 2, 3])) * int(rng.choice([1, 1, -1])) for _ in shape]
            base = make_([abs(s) * d + int(rng.integers(0, 3)) for s, d in zip(steps, shape)])
            return base, base[tuple(slice(None, None, s) for s in steps)][tuple(slice(0, d) for d in shape)]

        dst_base, dst_view = strided((batch, m, n), make)
        src_base, src_view = strided((k, n), make)
        idx_base, idx_view = strided((batch, m), lambda s: rng.integers(0, k, s).astype(itype))
        off = lambda v, b: v.__array_interface__["data"][0] - b.__array_interface__["data"][0]
        dd, sd, idd = gpu.from_host(dst_base), gpu.from_host(src_base), gpu.from_host(idx_base)
        say("random add_rows views %d: %s / %s, dst %s strides %s, src strides %s, idx strides %s"
            % (case, ntype.__name__, itype.__name__, dst_view.shape, dst_view.strides, src_view.strides, idx_view.strides))
        op.launch(ophip.AddRowsArgs(TensorLayout(code, list(dst_view.shape), list(dst_view.strides)), dd.ptr + off(dst_view, dst_base),
                                    TensorLayout(code, list(src_view.shape), list(src_view.strides)), sd.ptr + off(src_view, src_base),
                                    TensorLayout(icode, list(idx_view.shape), list(idx_view.strides)), idd.ptr + off(idx_view, idx_base)), None, stream)
        want = dst_base.copy()
        want_view = np.ndarray(dst_view.shape, ntype, want.data, off(dst_view, dst_base), dst_view.strides)
        rows = src_view[idx_view.astype(np.int64)]  # [batch, m, n]
        if ntype is f16:
            want_view[...] = (dst_view.astype(f32) + rows.astype(f32)).astype(f16)
        else:
            with np.errstate(over="ignore"):
                want_view[...] = dst_view + rows
        got = gpu.to_host(dd, ntype, dst_base.size, stream=stream).reshape(dst_base.shape)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), case


def outer_strided(rng, shape, make):
    """A view of `shape` whose last axis is contiguous and whose other axes run with a random step and direction
    through a larger base."""
    steps = [int(rng.choice([1, 1, 2, 3])) * int(rng.choice([1, 1, -1])) for _ in shape[:-1]] + [1]
    base = make([abs(s) * d + int(rng.integers(0, 2)) for s, d in zip(steps, shape)])
    return base, base[tuple(slice(None, None, s) for s in steps)][tuple(slice(0, d) for d in shape)]


def byte_offset(view, base):
    return view.__array_interface__["data"][0] - base.__array_interface__["data"][0]


def view_layout(view, code=None):
    return TensorLayout(code if code is not None else ophip.NP_DT[view.dtype], list(view.shape), list(view.strides))


@SWEEPS
def test_random_row_operators_on_views_that_step_backwards(gpu, stream, sweep):
    """rms_norm, layer_norm, swiglu, gelu, fused softmax and rope on tensors whose rows (heads, tokens) lie at a step, or
    in descending order, inside a larger buffer: the oracle runs on contiguous copies of the same views; whatever lies
    between the rows must keep its bytes."""
    rng = np.random.default_rng(229 + 1000 * sweep)
    make = lambda s: normal_f16(rng, s)

    def settle(base, view, mem, new_rows, what):
        """device buffer against: the base with `new_rows` in the view's place (within the f16 bar there, equal elsewhere)"""
        got = gpu.to_host(mem, f16, base.size, stream=stream).reshape(base.shape)
        got_view = np.ndarray(view.shape, f16, got.data, byte_offset(view, base), view.strides)
        assert_close_f16(got_view, new_rows, what)
        keep = np.ones(base.shape, bool)
        np.ndarray(view.shape, bool, keep.data, byte_offset(view, base) // 2, tuple(s // 2 for s in view.strides))[...] = False
        assert np.array_equal(got[keep].view(np.uint16), base[keep].view(np.uint16)), what + ": bytes between the rows changed"

    for case in range(10):
        n, d = int(rng.integers(1, 40)), int(rng.choice([8, 24, 256, 1000, 1024, 4096]))
        w, b = rng.uniform(0.5, 1.5, d).astype(f32).astype(f16), rng.uniform(-1, 1, d).astype(f32).astype(f16)
        wd, bd = gpu.from_host(w), gpu.from_host(b)
        xb, xv = outer_strided(rng, (n, d), make)
        yb, yv = outer_strided(rng, (n, d), make)
        xd, yd = gpu.from_host(xb), gpu.from_host(yb)
        say("views %d: rms_norm / layer_norm [%d, %d], x strides %s, y strides %s" % (case, n, d, xv.strides, yv.strides))
        xc = np.ascontiguousarray(xv)
        ophip.RmsNorm(gpu).launch(ophip.RmsNormArgs(view_layout(yv), yd.ptr + byte_offset(yv, yb), view_layout(xv), xd.ptr + byte_offset(xv, xb),
                                                    TensorLayout.of(w), wd, 1e-5), None, stream)
        settle(yb, yv, yd, oracle.rms_norm(np.empty_like(xc), xc, w, 1e-5), "rms_norm on views")
        ophip.LayerNorm(gpu).launch(ophip.LayerNormArgs(view_layout(yv), yd.ptr + byte_offset(yv, yb), view_layout(xv), xd.ptr + byte_offset(xv, xb),
                                                        TensorLayout.of(w), wd, TensorLayout.of(b), bd, 1e-5), None, stream)
        settle(yb, yv, yd, oracle.layer_norm(np.empty_like(xc), xc, w, b, 1e-5), "layer_norm on views")

        gb, gv = outer_strided(rng, (n, d), make)
        gd = gpu.from_host(gb)
        say("views %d: swiglu, gelu [%d, %d], gate strides %s, up strides %s" % (case, n, d, gv.strides, xv.strides))
        ophip.Swiglu(gpu).launch(ophip.SwigluArgs(view_layout(gv), gd.ptr + byte_offset(gv, gb), view_layout(xv), xd.ptr + byte_offset(xv, xb)), None, stream)
        after = oracle.swiglu(np.ascontiguousarray(gv), xc)
        settle(gb, gv, gd, after, "swiglu on views")
        got = gpu.to_host(gd, f16, gb.size, stream=stream).reshape(gb.shape)
        gb2 = got  # what the device holds now is gelu's input
        gv2 = np.ndarray(gv.shape, f16, gb2.data, byte_offset(gv, gb), gv.strides)
        ophip.Gelu(gpu).launch(ophip.GeluArgs(view_layout(gv), gd.ptr + byte_offset(gv, gb)), None, stream)
        settle(gb2, gv2, gd, oracle.gelu(np.ascontiguousarray(gv2)), "gelu on views")

        nh, seq = int(rng.integers(1, 5)), int(rng.integers(1, 9))
        att = seq + int(rng.integers(0, 600))
        ab, av = outer_strided(rng, (nh, seq, att), lambda s: normal_f16(rng, s, std=2.0))
        ad = gpu.from_host(ab)
        say("views %d: softmax [%d, %d, %d] strides %s" % (case, nh, seq, att, av.strides))
        ophip.FusedSoftmax(gpu).launch(ophip.FusedSoftmaxArgs(ophip.AttnMask.CAUSAL, view_layout(av), ad.ptr + byte_offset(av, ab)), None, stream)
        settle(ab, av, ad, oracle.fused_softmax(np.ascontiguousarray(av), causal=True), "softmax on views")

        nt, nh, dh = int(rng.integers(1, 20)), int(rng.integers(1, 6)), int(rng.choice([16, 64, 128]))
        tb, tv = outer_strided(rng, (nt, nh, dh), make)
        pb, pv = outer_strided(rng, (nt, 1), lambda s: rng.integers(0, 5000, s).astype(np.uint32))
        pv = pv[:, 0]
        td, pd = gpu.from_host(tb), gpu.from_host(pb)
        say("views %d: rope [%d, %d, %d] strides %s, pos stride %s" % (case, nt, nh, dh, tv.strides, pv.strides))
        empty = TensorLayout(dt.F16, [0, dh], [2 * dh, 2])
        ophip.Rope(gpu).launch(ophip.RopeArgs(view_layout(tv), td.ptr + byte_offset(tv, tb), view_layout(pv), pd.ptr + byte_offset(pv, pb),
                                              empty, None, empty, None, 1e4), None, stream)
        settle(tb, tv, td, oracle.rope(np.ascontiguousarray(tv), np.ascontiguousarray(pv), 1e4), "rope on views")


@SWEEPS
def test_random_mat_mul_on_views(gpu, stream, sweep):
    """mat_mul whose three operands are unrelated views: each row- or column-major at random (one unit stride, as the
    reference requires, mat_mul/args.rs:160-176), the other axis and the batch axis at a step or in descending order,
    a and b possibly one matrix for every batch.  A layout the library refuses must be refused as StridesNotSupport;
    one it takes must give numpy's product, and leave alone what lies between c's elements."""
    rng = np.random.default_rng(233 + 1000 * sweep)
    op = ophip.MatMul(gpu)
    taken = 0
    for case in range(24):
        bt, m, n, k = int(rng.integers(1, 4)), int(rng.choice([1, 5, 16, 33, 70])), int(rng.choice([8, 24, 130, 256])), int(rng.choice([16, 32, 100, 512]))

        def matrix(batches, rows, cols, std):
            """[batches, rows, cols] with rows or columns contiguous and everything else at a step, maybe backwards"""
            col_major = bool(rng.integers(0, 2))
            inner, outer = (rows, cols) if col_major else (cols, rows)
            base, view = outer_strided(rng, (batches, outer, inner), lambda s: normal_f16(rng, s, std=std))
            return base, (view.transpose(0, 2, 1) if col_major else view)

        cb, cv = matrix(bt, m, n, 1.0)
        ab, av = matrix(bt if rng.integers(0, 4) else 1, m, k, 1.0)
        bb, bv = matrix(bt if rng.integers(0, 4) else 1, k, n, 0.1)
        alpha, beta = float(rng.choice([1.0, 0.5])), float(rng.choice([0.0, 1.0, 0.25]))
        cd, ad, bd = gpu.from_host(cb), gpu.from_host(ab), gpu.from_host(bb)
        args = ophip.MatMulArgs(view_layout(cv), cd.ptr + byte_offset(cv, cb), beta, view_layout(av), ad.ptr + byte_offset(av, ab),
                                view_layout(bv), bd.ptr + byte_offset(bv, bb), alpha)
        say("mat_mul views %d: %dx(%dx%dx%d), c strides %s, a %s strides %s, b %s strides %s, alpha %g beta %g"
            % (case, bt, m, n, k, cv.strides, av.shape, av.strides, bv.shape, bv.strides, alpha, beta))
        try:
            op.launch(args, None, stream)
        except ophip.LaunchError as e:
            assert e.kind == "StridesNotSupport", e
            continue
        taken += 1
        got = gpu.to_host(cd, f16, cb.size, stream=stream).reshape(cb.shape)
        got_view = np.ndarray(cv.shape, f16, got.data, byte_offset(cv, cb), cv.strides)
        ref = alpha * np.matmul(av.astype(np.float64), bv.astype(np.float64)) + (beta * cv.astype(np.float64) if beta != 0 else 0.0)
        err = np.abs(got_view.astype(np.float64) - ref)
        assert (err <= 4e-3 + 1e-2 * np.maximum(np.abs(ref), np.abs(ref).mean())).all(), (case, err.max())
        keep = np.ones(cb.shape, bool)
        np.ndarray(cv.shape, bool, keep.data, byte_offset(cv, cb) // 2, tuple(s // 2 for s in cv.strides))[...] = False
        assert np.array_equal(got[keep].view(np.uint16), cb[keep].view(np.uint16)), "bytes between c's elements changed"
    assert taken >= 6


def attention_in_f64(q, k, v, causal):
    nh, seq, dh = q.shape
    nkvh, att, _ = k.shape
    kk, vv = np.repeat(k.astype(np.float64), nh // nkvh, axis=0), np.repeat(v.astype(np.float64), nh // nkvh, axis=0)
    s = np.einsum("hsd,had->hsa", q.astype(np.float64), kk) / np.sqrt(dh)
    if causal:
        s = np.where((np.arange(att)[None, :] <= (att - seq + np.arange(seq))[:, None])[None], s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    return np.einsum("hsa,had->hsd", p / p.sum(-1, keepdims=True), vv)


def assert_attention_close(got, ref, what):
    """Against the formula in f64: every element within abs 2e-3 or rel 1e-2.  The reference's ErrorCollector outliers
    (abs > f16 eps and rel > 1e-3) are held to one per hundred elements here, not one per thousand: on these small
    tensors the composite of launches rounds scores and probabilities to f16 on the way (as the reference does, and
    as the oracle's composite does in the parity tests), which moves a few elements by a step of f16."""
    a, r = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    err = np.abs(a - r)
    assert ((err <= 2e-3) | (err <= 1e-2 * np.abs(r))).all(), "%s: max abs %g" % (what, err.max())
    outliers = int(((err > 9.765625e-4) & (err / (np.abs(a) + np.abs(r) + 2.2e-16) > 1e-3)).sum())
    assert outliers <= max(2, a.size // 100), "%s: %d / %d outliers" % (what, outliers, a.size)


@SWEEPS
def test_random_attention_kv_cached_on_views(gpu, stream, sweep):
    """attention_kv_cached with q, k, v, o and both caches as unrelated views: head-major or token-major at random,
    heads and tokens at a step or in descending order (the head dimension contiguous, as every backend requires).
    Whatever path the library picks (one pass or the composite of launches): o against the formula in f64, the
    appended cache rows exact, every other byte of the caches and everything between o's elements unchanged."""
    rng = np.random.default_rng(239 + 1000 * sweep)
    op = ophip.AttnKVCached(gpu)
    for case in range(8):
        nkvh = int(rng.choice([1, 2, 4]))
        nh = nkvh * int(rng.choice([1, 2, 4]))
        seq, dh = int(rng.choice([1, 3, 16, 40])), int(rng.choice([64, 128]))
        pos = int(rng.integers(0, 300))
        buf = pos + seq + int(rng.integers(0, 9))
        causal = bool(rng.integers(0, 4))

        def heads(nheads, ntok):
            """[nheads, ntok, dh], stored head-major or token-major, outer axes at a step or backwards"""
            token_major = bool(rng.integers(0, 2))
            base, view = outer_strided(rng, (ntok, nheads, dh) if token_major else (nheads, ntok, dh), lambda s: normal_f16(rng, s))
            return base, (view.transpose(1, 0, 2) if token_major else view)

        (qb, qv), (kb, kv), (vb, vv), (ob, ov) = heads(nh, seq), heads(nkvh, seq), heads(nkvh, seq), heads(nh, seq)
        (kcb, kcv), (vcb, vcv) = heads(nkvh, buf), heads(nkvh, buf)
        dev = {name: gpu.from_host(b) for name, b in (("q", qb), ("k", kb), ("v", vb), ("o", ob), ("kc", kcb), ("vc", vcb))}
        at = lambda name, view, base: dev[name].ptr + byte_offset(view, base)
        args = ophip.AttnKVCachedArgs(view_layout(qv), at("q", qv, qb), view_layout(kv), at("k", kv, kb), view_layout(vv), at("v", vv, vb),
                                      view_layout(ov), at("o", ov, ob), view_layout(kcv), at("kc", kcv, kcb), view_layout(vcv), at("vc", vcv, vcb),
                                      ophip.AttnMask.CAUSAL if causal else ophip.AttnMask.NONE, pos)
        say("attention_kv_cached views %d: nh=%d nkvh=%d seq=%d dh=%d pos=%d buf=%d causal=%s q %s k %s o %s caches %s / %s"
            % (case, nh, nkvh, seq, dh, pos, buf, causal, qv.strides, kv.strides, ov.strides, kcv.strides, vcv.strides))
        if kcv.strides != vcv.strides:
            # the reference addresses the v cache with the k cache's strides (attention_kv_cached/operator.rs:114,156):
            # give both caches one layout, as every caller of the reference has to
            vcb = normal_f16(rng, kcb.shape)
            vcv = np.ndarray(kcv.shape, f16, vcb.data, byte_offset(kcv, kcb), kcv.strides)
            dev["vc"] = gpu.from_host(vcb)
            args.v_cache_layout, args.v_cache_base = view_layout(vcv), dev["vc"].ptr + byte_offset(vcv, vcb)
        op.scheme(args, 2 ** 40)
        op.launch(args, None, stream)
        keys = np.concatenate([kcv[:, :pos], kv], axis=1)
        vals = np.concatenate([vcv[:, :pos], vv], axis=1)
        got_o = gpu.to_host(dev["o"], f16, ob.size, stream=stream).reshape(ob.shape)
        got_view = np.ndarray(ov.shape, f16, got_o.data, byte_offset(ov, ob), ov.strides)
        assert_attention_close(got_view, attention_in_f64(qv, keys, vals, causal), "attention_kv_cached on views, case %d" % case)
        keep = np.ones(ob.shape, bool)
        np.ndarray(ov.shape, bool, keep.data, byte_offset(ov, ob) // 2, tuple(s // 2 for s in ov.strides))[...] = False
        assert np.array_equal(got_o[keep].view(np.uint16), ob[keep].view(np.uint16)), "bytes between o's elements changed"
        for name, base, view, new in (("kc", kcb, kcv, kv), ("vc", vcb, vcv, vv)):
            want = base.copy()
            np.ndarray(view.shape, f16, want.data, byte_offset(view, base), view.strides)[:, pos:pos + seq] = new
            got = gpu.to_host(dev[name], f16, base.size, stream=stream).reshape(base.shape)
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), name


@SWEEPS
def test_random_attention_on_views(gpu, stream, sweep):
    """attention with q, k, v and o as unrelated views (head-major or token-major, heads and tokens at a step or in
    descending order), grouped heads, with and without the causal mask, from a handful of query rows to several
    128-row blocks: o against the formula in f64, everything between o's elements unchanged, k and v untouched."""
    rng = np.random.default_rng(241 + 1000 * sweep)
    op = ophip.Attention(gpu)
    for case in range(8):
        nkvh = int(rng.choice([1, 2, 4]))
        nh = nkvh * int(rng.choice([1, 2, 4]))
        seq, dh = int(rng.choice([1, 5, 16, 70, 200])), int(rng.choice([64, 128]))
        att = seq + int(rng.choice([0, 0, 3, 130]))
        causal = bool(rng.integers(0, 4))

        def heads(nheads, ntok):
            token_major = bool(rng.integers(0, 2))
            base, view = outer_strided(rng, (ntok, nheads, dh) if token_major else (nheads, ntok, dh), lambda s: normal_f16(rng, s))
            return base, (view.transpose(1, 0, 2) if token_major else view)

        (qb, qv), (kb, kv), (vb, vv), (ob, ov) = heads(nh, seq), heads(nkvh, att), heads(nkvh, att), heads(nh, seq)
        dev = {name: gpu.from_host(b) for name, b in (("q", qb), ("k", kb), ("v", vb), ("o", ob))}
        at = lambda name, view, base: dev[name].ptr + byte_offset(view, base)
        args = ophip.AttentionArgs(view_layout(qv), at("q", qv, qb), view_layout(kv), at("k", kv, kb), view_layout(vv), at("v", vv, vb),
                                   view_layout(ov), at("o", ov, ob), ophip.AttnMask.CAUSAL if causal else ophip.AttnMask.NONE)
        say("attention views %d: nh=%d nkvh=%d seq=%d att=%d dh=%d causal=%s q %s k %s v %s o %s"
            % (case, nh, nkvh, seq, att, dh, causal, qv.strides, kv.strides, vv.strides, ov.strides))
        op.scheme(args, 2 ** 40)
        op.launch(args, None, stream)
        got_o = gpu.to_host(dev["o"], f16, ob.size, stream=stream).reshape(ob.shape)
        got_view = np.ndarray(ov.shape, f16, got_o.data, byte_offset(ov, ob), ov.strides)
        assert_attention_close(got_view, attention_in_f64(qv, kv, vv, causal), "attention on views, case %d" % case)
        keep = np.ones(ob.shape, bool)
        np.ndarray(ov.shape, bool, keep.data, byte_offset(ov, ob) // 2, tuple(s // 2 for s in ov.strides))[...] = False
        assert np.array_equal(got_o[keep].view(np.uint16), ob[keep].view(np.uint16)), "bytes between o's elements changed"
        for name, base in (("k", kb), ("v", vb)):
            assert np.array_equal(gpu.to_host(dev[name], f16, base.size, stream=stream).reshape(base.shape).view(np.uint16), base.view(np.uint16)), name


@SWEEPS
def test_random_launches_need_no_more_workspace_than_scheme_reports(gpu, stream, sweep):
    """mat_mul (split K), attention and random_sample launched with a workspace of exactly the size scheme() answered
    and a queue allocator that has nothing to give (an empty StreamMemPool): the launch must not ask for more, and
    must not reach past the workspace (against the host build of the library its end lies against a guard page)."""
    rng = np.random.default_rng(251 + 1000 * sweep)
    pool = ophip.StreamMemPool(gpu, stream)  # no slab was put: every allocation fails
    mm, at, rs = ophip.MatMul(gpu), ophip.Attention(gpu), ophip.RandomSample(gpu)
    lay = TensorLayout.of
    with_workspace = 0
    for case in range(18):
        if case % 3 == 0:
            bt, m = int(rng.choice([1, 1, 4, 32])), int(rng.choice([1, 16, 40, 64, 200]))
            n, k = int(rng.choice([128, 256, 1024])), int(rng.choice([128, 512, 2048, 4096]))
            a, b, c = normal_f16(rng, (bt, m, k)), normal_f16(rng, (bt, k, n), std=0.05), np.zeros((bt, m, n), f16)
            ad, bd, cd = gpu.from_host(a), gpu.from_host(b), gpu.from_host(c)
            args = ophip.MatMulArgs(lay(c), cd, 0.0, lay(a), ad, lay(b), bd, 1.0)
            need = mm.scheme(args, 2 ** 40)
            say("workspace %d: mat_mul %dx(%dx%dx%d), %s, %d bytes" % (case, bt, m, n, k, mm.describe(args), need))
            mm.launch(args, gpu.malloc(need) if need else None, pool)
            got = gpu.to_host(cd, f16, c.size, stream=stream).reshape(c.shape).astype(np.float64)
            ref = a.astype(np.float64) @ b.astype(np.float64)
            assert (np.abs(got - ref) / np.maximum(np.abs(ref), np.abs(ref).mean())).max() <= 1e-2
        elif case % 3 == 1:
            nkvh = int(rng.choice([1, 2, 8]))
            nh, seq, dh = nkvh * int(rng.choice([1, 4])), int(rng.choice([1, 16, 100, 300])), int(rng.choice([64, 128]))
            att = seq + int(rng.choice([0, 50, 700]))
            q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, att, dh)), normal_f16(rng, (nkvh, att, dh))
            qd, kd, vd, od = gpu.from_host(q), gpu.from_host(k), gpu.from_host(v), gpu.malloc(q.nbytes)
            args = ophip.AttentionArgs(lay(q), qd, lay(k), kd, lay(v), vd, lay(q), od, ophip.AttnMask.CAUSAL)
            need = at.scheme(args, 2 ** 40)
            say("workspace %d: attention nh=%d nkvh=%d seq=%d att=%d dh=%d, %d bytes" % (case, nh, nkvh, seq, att, dh, need))
            at.launch(args, gpu.malloc(need) if need else None, pool)
            got = gpu.to_host(od, f16, q.size, stream=stream).reshape(q.shape)
            assert_attention_close(got, attention_in_f64(q, k, v, True), "attention with an exact workspace")
        else:
            n = int(rng.choice([1000, 32000, 50257, 128256]))
            logits = normal_f16(rng, (n,), std=3.0)
            ld, kvd = gpu.from_host(logits), gpu.malloc(8)
            args = ophip.RandomSampleArgs.layout(dt.F16, n)
            args.kv_pair_base, args.logits_base = kvd, ld
            args.config = ophip.SampleArgs(float(rng.choice([0.7, 1.0])), float(rng.choice([0.5, 0.9, 1.0])), int(rng.choice([1, 50, 300, 5000, 2 ** 62])))
            args.seed = float(rng.random())
            need = rs.scheme(args, 2 ** 40)
            say("workspace %d: random_sample n=%d, %d bytes" % (case, n, need))
            rs.launch(args, gpu.malloc(need) if need else None, pool)
            kv = gpu.to_host(kvd, np.uint32, 2, stream=stream)
            assert int(kv[0]) < n
        with_workspace += need > 0
    assert with_workspace >= 8


@SWEEPS
def test_random_and_mostly_invalid_arguments_come_back_as_status_codes(gpu, stream, sweep):
    """Layouts drawn at random (ranks, types, zero, huge and dynamic extents, zero, negative, misaligned and dynamic
    strides; every so often a plausible contiguous tensor with one entry disturbed) into scheme and launch of every
    operator, all bases null: each call ends in a status code (a launch in ArgsNotSupport at the latest), never in a
    kernel and never in a crash of the host side."""
    rng = np.random.default_rng(257 + 1000 * sweep)
    types = [dt.F16, dt.F32, dt.F64, dt.BF16, dt.U8, dt.U32, dt.U64, dt.I32, dt.BOOL, dt.KVPAIR]
    extents = [0, 1, 2, 3, 7, 8, 16, 64, 128, 4096, 2 ** 31, 2 ** 40, None]
    steps = [0, 1, 2, 4, 8, -2, -8, 6, 256, 8192, 2 ** 33, -(2 ** 33), None]
    small = [1, 2, 3, 8, 16, 64]

    def lay(rank, typ=dt.F16):
        nd = rank if rng.integers(0, 8) else int(rng.integers(0, 5))
        typ = types[int(rng.integers(0, len(types)))] if rng.integers(0, 6) == 0 else typ
        if rng.integers(0, 2):  # contiguous, one entry disturbed now and then
            shape = [int(rng.choice(small)) for _ in range(nd)]
            strides, m = [], ophip.dtype_nbytes(typ)
            for n in reversed(shape):
                strides.insert(0, m)
                m *= n
            if nd and rng.integers(0, 2):
                i = int(rng.integers(0, nd))
                if rng.integers(0, 2):
                    shape[i] = extents[int(rng.integers(0, len(extents)))]
                else:
                    strides[i] = steps[int(rng.integers(0, len(steps)))]
            return TensorLayout(typ, shape, strides)
        return TensorLayout(typ, [extents[int(rng.integers(0, len(extents)))] for _ in range(nd)], [steps[int(rng.integers(0, len(steps)))] for _ in range(nd)])

    same = lambda make: make(int(rng.integers(0, 5)))
    ops = [
        (ophip.RmsNorm(gpu), lambda: ophip.RmsNormArgs(lay(2), None, lay(2), None, lay(1), None, 1e-5)),
        (ophip.Rope(gpu), lambda: ophip.RopeArgs(lay(3), None, lay(1, dt.U32), None, lay(2), None, lay(2), None, 1e4)),
        (ophip.FusedSoftmax(gpu), lambda: ophip.FusedSoftmaxArgs(int(rng.integers(0, 4)), lay(3), None)),
        (ophip.Rearrange(gpu), lambda: same(lambda n: ophip.RearrangeArgs(lay(n), None, lay(n), None))),
        (ophip.Swiglu(gpu), lambda: ophip.SwigluArgs(lay(2), None, lay(2), None)),
        (ophip.MatMul(gpu), lambda: same(lambda n: ophip.MatMulArgs(lay(2 + n % 2), None, 0.5, lay(2 + n % 2), None, lay(2 + n % 2), None, 1.0))),
        (ophip.Attention(gpu), lambda: ophip.AttentionArgs(lay(3), None, lay(3), None, lay(3), None, lay(3), None, int(rng.integers(0, 3)))),
        (ophip.AttnKVCached(gpu), lambda: ophip.AttnKVCachedArgs(lay(3), None, lay(3), None, lay(3), None, lay(3), None, lay(3), None, lay(3), None,
                                                                 int(rng.integers(0, 3)), [0, 5, 2 ** 40, None][int(rng.integers(0, 4))])),
        (ophip.LayerNorm(gpu), lambda: ophip.LayerNormArgs(lay(2), None, lay(2), None, lay(1), None, lay(1), None, 1e-5)),
        (ophip.Gelu(gpu), lambda: ophip.GeluArgs(lay(2), None)),
        (ophip.Add(gpu), lambda: same(lambda n: ophip.AddArgs(lay(n), None, lay(n), None, lay(n), None))),
        (ophip.AddRows(gpu), lambda: ophip.AddRowsArgs(lay(3), None, lay(2), None, lay(2, dt.U32), None)),
    ]
    outcomes = set()
    for it in range(1800):
        op, make = ops[it % len(ops)]
        small[:] = [int(rng.choice([1, 2, 8, 16, 64]))] if rng.integers(0, 4) else [1, 2, 3, 8, 16, 64]
        args = make()
        for verb in ("scheme", "launch"):
            try:
                op.scheme(args, [0, 1 << 20, 2 ** 40][int(rng.integers(0, 3))]) if verb == "scheme" else op.launch(args, None, stream)
                outcomes.add("ok")
            except (ophip.SchemeError, ophip.LaunchError) as e:
                outcomes.add(e.kind)
    stream.synchronize()
    assert len(outcomes) >= 6, outcomes  # the draws reach well past the first check
