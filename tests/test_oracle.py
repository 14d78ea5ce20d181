"""Pins the CPU oracle (oracle/oracle.c) without running the reference.

The reference's repository holds exactly one known-answer test for this path
(rearrange/args.rs:242-304, both layouts); everything else the oracle computes
is pinned here by closed forms, invariants, special cases and brute force chosen
so that a dropped term, a wrong index or a swapped operand fails.
"""
import math

import numpy as np
import pytest

import oracle

f16, f32, f64 = np.float16, np.float32, np.float64


def ulp16(x):
    x = np.abs(np.asarray(x, dtype=f64))
    e = np.floor(np.log2(np.maximum(x, 2.0 ** -14)))
    return 2.0 ** (e - 10)


# ------------------------------------------------------------------ f16 ----

def test_f16_conversions_match_ieee():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(f16).astype(f32)
    got = np.array([oracle.f16_bits_to_f32(int(b)) for b in bits], dtype=f32)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all()
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(20000) * rng.choice([1e-8, 1e-6, 1e-4, 1, 300, 7e4], 20000)).astype(f32)
    fin = want[np.isfinite(want)].astype(f64)
    fin.sort()
    mid = ((fin[:-1] + fin[1:]) / 2).astype(f32)  # exact ties between neighbouring f16 values
    x = np.concatenate([x, mid, np.array([0.0, -0.0, np.inf, -np.inf, 65504, 65520, 65519.99, 2.0 ** -25], f32)])
    with np.errstate(over="ignore"):
        want16 = x.astype(f16).view(np.uint16)
    got16 = np.array([oracle.f32_to_f16_bits(v) for v in x], dtype=np.uint16)
    assert (got16 == want16).all()


# ------------------------------------------------------------- rms_norm ----

def rms_ref64(x, w, eps):
    x = x.astype(f64)
    return x / np.sqrt((x * x).mean(axis=1, keepdims=True) + eps) * w.astype(f64)


@pytest.mark.parametrize("eps", [1e-5, 1.0])
def test_rms_norm_f64_closed_form(eps):
    rng = np.random.default_rng(0)
    x, w = rng.standard_normal((5, 96)), rng.uniform(0.5, 1.5, 96)
    y = oracle.rms_norm(np.empty_like(x), x, w, eps)
    np.testing.assert_allclose(y, rms_ref64(x, w, f64(f32(eps))), rtol=1e-13)


def test_rms_norm_f16_against_closed_form_and_order():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((7, 512)).astype(f16)
    w = rng.uniform(0.5, 1.5, 512).astype(f16)
    y = oracle.rms_norm(np.empty_like(x), x, w, 1e-5)
    ref = rms_ref64(x, w, 1e-5)
    assert (np.abs(y.astype(f64) - ref) <= 0.5 * ulp16(ref) + 1e-4 * np.abs(ref)).all()
    # rounding points: sequential f32 sum, k = 1/sqrt, (k*w)*x left to right, one RNE to f16
    xf, wf = x.astype(f32), w.astype(f32)
    for i in range(x.shape[0]):
        s = f32(0)
        for v in xf[i]:
            s = f32(s + f32(v * v))
        k = f32(1) / np.sqrt(f32(s / f32(512) + f32(1e-5)))
        want = ((k * wf).astype(f32) * xf[i]).astype(f16)
        assert np.array_equal(want.view(np.uint16), y[i].view(np.uint16))


def test_rms_norm_special_cases():
    # constant row: y = w * c / sqrt(c^2 + eps)
    x = np.full((1, 256), 2.0, f32)
    w = np.linspace(0.5, 1.5, 256).astype(f32)
    y = oracle.rms_norm(np.empty_like(x), x, w, 1.0)
    np.testing.assert_allclose(y[0], w * 2.0 / math.sqrt(5.0), rtol=3e-7)
    # d = 1
    x1 = np.array([[3.0], [-4.0]], f64)
    y1 = oracle.rms_norm(np.empty_like(x1), x1, np.array([2.0]), 0.5)
    np.testing.assert_allclose(y1[:, 0], [6 / math.sqrt(9.5), -8 / math.sqrt(16.5)], rtol=1e-15)
    # scaling x by 2 with eps = 0 leaves y bit-identical (power-of-two scaling commutes with rounding)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3, 128)).astype(f16)
    w = rng.uniform(0.5, 1.5, 128).astype(f32)
    a = oracle.rms_norm(np.empty_like(x), x, w, 0.0)
    b = oracle.rms_norm(np.empty_like(x), (x * f16(2)).astype(f16), w, 0.0)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_rms_norm_strided_layout_equals_contiguous():
    rng = np.random.default_rng(4)
    big = rng.standard_normal((6, 200)).astype(f16)
    xv = big[::2, 10:138]
    w = rng.uniform(0.5, 1.5, 128).astype(f16)
    out = np.zeros((3, 300), f16)
    yv = out[:, 50:178]
    oracle.rms_norm(yv, xv, w, 1e-5)
    ref = oracle.rms_norm(np.empty((3, 128), f16), np.ascontiguousarray(xv), w, 1e-5)
    assert np.array_equal(yv, ref)
    assert (out[:, :50] == 0).all() and (out[:, 178:] == 0).all()


def test_rms_norm_unsupported_pair():
    with pytest.raises(oracle.OracleError) as e:
        oracle.rms_norm(np.zeros((1, 4), f32), np.zeros((1, 4), f32), np.zeros(4, f16), 1e-5)
    assert e.value.kind == "TypeNotSupport"


# ----------------------------------------------------------------- rope ----

def rope_ref64(t, pos, theta):
    nt, nh, dh = t.shape
    H = dh // 2
    k = np.arange(H)
    ang = pos.astype(f64)[:, None] / (f64(theta) ** (k / H))[None, :]  # [nt, H]
    s, c = np.sin(ang)[:, None, :], np.cos(ang)[:, None, :]
    a, b = t[..., 0::2].astype(f64), t[..., 1::2].astype(f64)
    out = np.empty(t.shape, f64)
    out[..., 0::2] = a * c - b * s
    out[..., 1::2] = a * s + b * c
    return out


def test_rope_pos_zero_is_identity():
    rng = np.random.default_rng(0)
    t = rng.standard_normal((4, 3, 16)).astype(f16)
    out = oracle.rope(t.copy(), np.zeros(4, np.uint32), 1e4)
    assert np.array_equal(out.view(np.uint16), t.view(np.uint16))


def test_rope_f64_closed_form_pairing_and_exponent():
    rng = np.random.default_rng(1)
    t = rng.standard_normal((7, 5, 12))
    pos = np.array([0, 1, 2, 3, 7, 8, 1], np.uint64)
    out = oracle.rope(t.copy(), pos, 1e4)
    np.testing.assert_allclose(out, rope_ref64(t, pos, 1e4), rtol=1e-10, atol=1e-12)


def test_rope_f16_against_closed_form():
    rng = np.random.default_rng(2)
    t = rng.standard_normal((9, 4, 64)).astype(f16)
    pos = np.array([0, 1, 2, 3, 7, 8, 1, 300, 511], np.uint32)
    out = oracle.rope(t.copy(), pos, 1e4)
    ref = rope_ref64(t, pos, 1e4)
    # f32 angle error grows with pos (ang * 2^-24 relative), then one f16 rounding
    tol = 0.5 * ulp16(ref) + 2e-4
    assert (np.abs(out.astype(f64) - ref) <= tol).all()
    # u64 positions give the same bytes
    out64 = oracle.rope(t.copy(), pos.astype(np.uint64), 1e4)
    assert np.array_equal(out, out64)


def test_rope_first_pair_rotates_by_pos_and_keeps_norm():
    t = np.zeros((3, 1, 8), f32)
    t[..., 0::2] = 1.0  # every pair is (1, 0)
    pos = np.array([1, 2, 100], np.uint32)
    out = oracle.rope(t.copy(), pos, 1e4)
    np.testing.assert_allclose(out[:, 0, 0], np.cos(pos.astype(f64)), atol=1e-6)
    np.testing.assert_allclose(out[:, 0, 1], np.sin(pos.astype(f64)), atol=1e-6)
    np.testing.assert_allclose(out[..., 0::2] ** 2 + out[..., 1::2] ** 2, 1.0, atol=1e-6)


def test_rope_strided_heads_inside_a_wider_buffer():
    rng = np.random.default_rng(5)
    buf = rng.standard_normal((6, 3 * 4 * 16)).astype(f16)  # [tokens, q|k|v]
    q = buf[:, : 4 * 16].reshape(6, 4, 16)  # a view: token stride covers q, k and v
    assert q.base is not None
    before = buf.copy()
    pos = np.arange(6, dtype=np.uint32) + 5
    oracle.rope(q, pos, 1e4)
    ref = oracle.rope(np.ascontiguousarray(before[:, :64]).reshape(6, 4, 16), pos, 1e4)
    assert np.array_equal(buf[:, :64].reshape(6, 4, 16), ref)
    assert np.array_equal(buf[:, 64:], before[:, 64:])


def test_rope_rejects_strided_last_dim():
    t = np.zeros((2, 2, 16), f16)[..., ::2]
    with pytest.raises(oracle.OracleError) as e:
        oracle.rope(t, np.zeros(2, np.uint32), 1e4)
    assert e.value.kind == "StridesNotSupport"


# -------------------------------------------------------- fused softmax ----

def softmax_ref64(att, causal):
    nh, seq, al = att.shape
    out = np.zeros(att.shape, f64)
    for r in range(seq):
        m = al - seq + r + 1 if causal else al
        x = att[:, r, :m].astype(f64)
        e = np.exp(x - x.max(axis=1, keepdims=True))
        out[:, r, :m] = e / e.sum(axis=1, keepdims=True)
    return out


@pytest.mark.parametrize("seq,al", [(1, 511), (7, 511), (7, 64), (5, 5)])
def test_softmax_causal_structure_and_closed_form(seq, al):
    rng = np.random.default_rng(0)
    att = (rng.standard_normal((3, seq, al)) * 2).astype(f16)
    out = oracle.fused_softmax(att.copy(), causal=True)
    bits = out.view(np.uint16)
    for r in range(seq):
        m = al - seq + r + 1
        assert (bits[:, r, m:] == 0).all()  # exactly +0, not -0
        assert (out[:, r, :m].astype(f64).sum(axis=1) > 0.99).all()
    ref = softmax_ref64(att, True)
    assert (np.abs(out.astype(f64) - ref) <= 1.5 * ulp16(ref) + 1e-7).all()
    np.testing.assert_allclose(out.astype(f64).sum(axis=2), 1.0, atol=al * 2.0 ** -12)


def test_softmax_no_mask_and_single_column():
    rng = np.random.default_rng(1)
    att = (rng.standard_normal((2, 3, 40)) * 2).astype(f16)
    out = oracle.fused_softmax(att.copy(), causal=False)
    assert (np.abs(out.astype(f64) - softmax_ref64(att, False)) <= 1.5 * ulp16(out)).all()
    one = oracle.fused_softmax(np.array([[[3.5, 9.0, -2.0]]], f16), causal=True)  # seq 1 keeps all 3
    assert one[0, 0].astype(f64).sum() == pytest.approx(1.0, abs=2e-3)
    sq = oracle.fused_softmax(np.array([[[-7.0, 1.0], [2.0, 2.0]]], f16), causal=True)
    assert sq.view(np.uint16)[0, 0].tolist() == [0x3C00, 0]  # row 0 keeps one column: exactly 1.0
    assert sq.view(np.uint16)[0, 1].tolist() == [0x3800, 0x3800]  # equal logits: exactly 0.5 each


def test_softmax_shift_invariance_and_double_rounding():
    rng = np.random.default_rng(2)
    x = (rng.integers(-32, 32, (2, 4, 24)) / 8.0).astype(f16)  # multiples of 1/8: +2 is exact
    a = oracle.fused_softmax(x.copy(), causal=True)
    b = oracle.fused_softmax((x + f16(2)).astype(f16), causal=True)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    # the value scaled is the f16-rounded exponential, the sum uses the unrounded one
    row = np.array([[[0.0, -1.0, -2.5]]], f16)
    out = oracle.fused_softmax(row.copy(), causal=False)[0, 0]
    e = np.exp((row[0, 0].astype(f32) - f32(0)).astype(f32)).astype(f32)
    s = f32(0)
    for v in e:
        s = f32(s + v)
    want = (e.astype(f16).astype(f32) * (f32(1) / s)).astype(f16)
    assert np.abs(out.astype(f64) - want.astype(f64)).max() <= float(ulp16(want).max())  # libm expf vs numpy exp


@pytest.mark.parametrize("dtype", [f32, f64])
def test_softmax_f32_and_f64_closed_form(dtype):
    """fuesd_softmax/common_cpu/mod.rs:147-193: the same algorithm in the element's own arithmetic."""
    rng = np.random.default_rng(4)
    eps = float(np.finfo(dtype).eps)
    for seq, al in [(1, 37), (6, 6), (5, 64)]:
        att = (rng.standard_normal((2, seq, al)) * 2).astype(dtype)
        out = oracle.fused_softmax(att.copy(), causal=True)
        ref = softmax_ref64(att, True)
        for r in range(seq):
            m = al - seq + r + 1
            assert (out[:, r, m:] == 0).all() and not np.signbit(out[:, r, m:]).any()  # exactly +0
        # exp of a difference of magnitude <= ~16: a few ulp from the argument, then sum and product
        assert (np.abs(out.astype(f64) - ref) <= 24 * eps * ref + 1e-300).all()
        np.testing.assert_allclose(out.astype(f64).sum(axis=2), 1.0, atol=al * eps)
    sq = oracle.fused_softmax(np.array([[[-7.0, 1.0], [2.0, 2.0]]], dtype), causal=True)
    assert sq[0, 0].tolist() == [1.0, 0.0] and sq[0, 1].tolist() == [0.5, 0.5]
    nomask = oracle.fused_softmax(np.array([[[1.0, 1.0, 1.0, 1.0]]], dtype), causal=False)
    assert nomask[0, 0].tolist() == [0.25] * 4
    # the scale is the rounded reciprocal of the sum, not a division: 1 / 3 rounds down in f32 and in f64, and
    # 3 equal logits give exactly that rounded reciprocal
    three = oracle.fused_softmax(np.array([[[0.5, 0.5, 0.5]]], dtype), causal=False)
    assert three[0, 0, 0] == dtype(1) / dtype(3)
    x = (rng.integers(-32, 32, (2, 4, 24)) / 8.0).astype(dtype)  # multiples of 1/8: + 2 is exact
    assert np.array_equal(oracle.fused_softmax(x.copy(), causal=True), oracle.fused_softmax(x + dtype(2), causal=True))


def test_softmax_strided_rows():
    rng = np.random.default_rng(3)
    big = (rng.standard_normal((2, 6, 48)) * 2).astype(f16)
    view = big[:, ::2, :32]
    before = big.copy()
    oracle.fused_softmax(view, causal=True)
    ref = oracle.fused_softmax(np.ascontiguousarray(before[:, ::2, :32]), causal=True)
    assert np.array_equal(big[:, ::2, :32], ref)
    assert np.array_equal(big[:, 1::2], before[:, 1::2]) and np.array_equal(big[:, :, 32:], before[:, :, 32:])


def test_softmax_row_without_columns_is_an_error():
    with pytest.raises(oracle.OracleError):
        oracle.fused_softmax(np.zeros((1, 4, 2), f16), causal=True)


# ------------------------------------------------------------ rearrange ----

def test_rearrange_scheme_reference_known_answers():
    """rearrange/args.rs:242-304 (test_scheme), both layouts, verbatim expectations."""
    s = oracle.rearrange_scheme([4, 3, 2, 1, 2, 3, 4], [288, 96, 48, 48, 24, 8, 2], [576, 192, 96, 48, 8, 16, 2], 2)
    nd = (len(s) - 2) // 3
    assert nd == 3 and s[0] == 8 and s[1] == 24 * 2 * 3
    assert s[2:2 + nd] == [6, 3, 1]
    assert s[2 + nd:2 + 2 * nd] == [48, 24, 8]
    assert s[2 + 2 * nd:] == [96, 8, 16]
    assert [s[1 + i] // s[2 + i] for i in range(nd)] == [24, 2, 3]
    st = [33554432 * 2, 16777216 * 2, 524288 * 2, 128 * 2, 2]
    s2 = oracle.rearrange_scheme([32, 2, 32, 456, 128], st, st, 2)
    assert s2 == [116736, 2048, 1, 1048576, 1048576]
    s3 = oracle.rearrange_distribute_unit(s2, [32 * (1 << n) for n in range(5, -1, -1)])
    assert s3 == [1024, 116736 // 1024 * 2048, 116736 // 1024, 1, 1048576, 1024, 1048576, 1024]


def test_rearrange_scheme_transpose_case_and_errors():
    assert oracle.rearrange_scheme([32, 512, 128], [256, 8192, 2], [131072, 256, 2], 2) == \
        [256, 16384, 32, 1, 8192, 256, 256, 131072]
    with pytest.raises(oracle.OracleError) as e:
        oracle.rearrange_scheme([2, 3], [0, 4], [12, 4], 4)
    assert e.value.kind == "ShapeNotSupport"
    with pytest.raises(oracle.OracleError) as e:
        oracle.rearrange_scheme([2, 3], [12, 4], [12, 4], 4, src_shape=[2, 4])
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(oracle.OracleError) as e:
        oracle.rearrange_scheme([oracle.DYN_USIZE, 3], [12, 4], [12, 4], 4, src_shape=[oracle.DYN_USIZE, 3])
    assert e.value.kind == "DynamicNotSupport"


def random_views(rng, dtype):
    nd = int(rng.integers(1, 5))
    shape = [int(rng.integers(1, 7)) for _ in range(nd)]
    src_full = rng.integers(0, 2 ** 8 * dtype().itemsize, size=[2 * s + 1 for s in shape]).astype(dtype)
    dst_full = np.zeros([2 * s + 2 for s in shape], dtype)

    def view(full):
        idx = []
        for s in shape:
            step = int(rng.choice([1, 2, -1, -2]))
            start = int(rng.integers(0, 2))
            if step > 0:
                idx.append(slice(start, start + step * s, step))
            else:
                hi = start + (-step) * (s - 1)
                idx.append(slice(hi, None if hi + step * s < 0 else hi + step * s, step))
        v = full[tuple(idx)]
        assert list(v.shape) == shape
        return v.transpose(rng.permutation(nd))

    sv, dv = view(src_full), view(dst_full)
    return src_full, dst_full, sv, dv


def test_rearrange_matches_numpy_strided_copy():
    rng = np.random.default_rng(0)
    done = 0
    for _ in range(400):
        dtype = [np.uint8, np.uint16, np.uint32, np.uint64][int(rng.integers(0, 4))]
        src_full, dst_full, sv, dv = random_views(rng, dtype)
        if sv.shape != dv.shape:
            continue
        want_full = dst_full.copy()
        want_view = np.lib.stride_tricks.as_strided(
            want_full.ravel()[(dv.__array_interface__["data"][0] - dst_full.__array_interface__["data"][0])
                              // dst_full.itemsize:], dv.shape, dv.strides)
        want_view[...] = sv
        oracle.rearrange(dv, sv)
        assert np.array_equal(dst_full, want_full)
        done += 1
    assert done > 50


def test_rearrange_broadcast_source_and_single_unit():
    src = np.arange(8, dtype=np.uint32)
    dst = np.zeros((5, 8), np.uint32)
    sv = np.lib.stride_tricks.as_strided(src, (5, 8), (0, 4))  # zero source stride = broadcast
    oracle.rearrange(dst, sv)
    assert (dst == src[None, :]).all()
    a, b = np.arange(24, dtype=np.uint16).reshape(2, 3, 4), np.zeros((2, 3, 4), np.uint16)
    oracle.rearrange(b, a)  # fully contiguous: count == 1, one memcpy
    assert np.array_equal(a, b)


# --------------------------------------------------------------- swiglu ----

def test_swiglu_closed_form_and_special_cases():
    rng = np.random.default_rng(0)
    g = (rng.standard_normal((4, 33)) * 3).astype(f16)
    u = rng.standard_normal((4, 33)).astype(f16)
    out = oracle.swiglu(g.copy(), u)
    a, b = g.astype(f64), u.astype(f64)
    ref = a / (1 + np.exp(-a)) * b
    assert (np.abs(out.astype(f64) - ref) <= 0.5 * ulp16(ref) + 1e-6 * np.abs(ref) + 1e-9).all()
    z = oracle.swiglu(np.zeros((1, 4), f16), np.array([[1, -1, 2, 0.5]], f16))
    assert (z == 0).all()
    silu = oracle.swiglu(np.array([[1.0, -1.0, 4.0]], f32), np.ones((1, 3), f32))
    np.testing.assert_allclose(silu[0], [1 / (1 + math.exp(-1)), -1 / (1 + math.e), 4 / (1 + math.exp(-4))], rtol=2e-7)
    sat = oracle.swiglu(np.array([[30.0, -30.0, -100.0]], f16), np.array([[2.0, 2.0, 2.0]], f16))
    assert sat[0, 0] == f16(60.0) and abs(float(sat[0, 1])) < 1e-10 and sat[0, 2] == 0
    # gate and up as the two halves of one wider buffer (independent row strides)
    buf = rng.standard_normal((3, 40)).astype(f16)
    before = buf.copy()
    oracle.swiglu(buf[:, :20], buf[:, 20:])
    assert np.array_equal(buf[:, :20], oracle.swiglu(before[:, :20].copy(), before[:, 20:].copy()))
    assert np.array_equal(buf[:, 20:], before[:, 20:])


# -------------------------------------------------------- random_sample ----

def test_argmax_keeps_the_last_maximum():
    rng = np.random.default_rng(0)
    for n in [1, 2, 17, 1000]:
        x = rng.integers(-5, 5, n).astype(f16)  # heavy ties
        idx, val = oracle.argmax(x)
        assert idx == n - 1 - int(np.argmax(x[::-1]))
        assert val == int(x.view(np.uint16)[idx])
    assert oracle.argmax(np.full(9, 2.5, f32))[0] == 8
    assert oracle.argmax(np.array([0.0, -0.0, 0.0, -0.0], f16))[0] == 3  # -0 == +0: later wins
    x = np.array([1.0, 7.0, 3.0, 7.0, 2.0], f32)
    idx, val = oracle.argmax(x)
    assert idx == 3 and val == int(np.array([7.0], f32).view(np.uint32)[0])


def test_argmax_nan_restarts_the_scan():
    nan = float("nan")
    assert oracle.argmax(np.array([1.0, nan, 0.5], f32))[0] == 2  # the scan restarts after the NaN
    assert oracle.argmax(np.array([1.0, nan, 0.5, 0.75, 0.1], f16))[0] == 3
    idx, val = oracle.argmax(np.array([1.0, 2.0, nan], f32))
    assert idx == 2 and math.isnan(np.array([val], np.uint32).view(f32)[0])


def sample_brute(x, t, top_p, top_k, seed):
    n = len(x)
    v = x.astype(f32)
    order = np.lexsort((np.arange(n), -v.astype(f64)))
    sv = v[order]
    cum = np.empty(n, f32)
    cum[0] = 1
    for i in range(1, n):
        cum[i] = f32(cum[i - 1] + f32(math.exp(float(f32(f32(sv[i] - sv[0]) / f32(t))))))
    pk = cum[min(top_k, n) - 1]
    pp = f32(cum[-1] * f32(top_p))
    lim = f32(f32(seed) * min(pk, pp))
    i = int(np.argmax(cum >= lim))
    margin = np.min(np.abs(cum.astype(f64) - float(lim)) / max(float(lim), 1e-30))
    return int(order[i]), cum[i], margin, set(order[: min(top_k, n)].tolist())


@pytest.mark.parametrize("dtype", [f16, f32])
def test_random_sample_matches_brute_force(dtype):
    rng = np.random.default_rng(0)
    checked = 0
    for _ in range(300):
        n = int(rng.integers(1, 60))
        x = (rng.standard_normal(n) * 2).astype(dtype)
        if rng.random() < 0.3:
            x = np.round(x).astype(dtype)  # ties
        t = float(rng.uniform(0.3, 2.0))
        top_p = float(rng.uniform(0.1, 1.0))
        top_k = int(rng.integers(2, 70))
        seed = float(rng.uniform(0, 1))
        idx, val = oracle.random_sample(x, t, top_p, top_k, seed)
        bidx, bcum, margin, topset = sample_brute(x, t, top_p, top_k, seed)
        assert idx in topset
        if margin > 1e-5:  # away from a rounding-distance tie between the draw and a running sum
            assert idx == bidx
            got = np.array([val], np.uint32).view(f32)[0] if dtype is f32 else \
                np.array([val & 0xFFFF], np.uint16).view(f16)[0]
            assert abs(float(got) - float(bcum)) <= (float(ulp16(bcum)) if dtype is f16 else 1e-5 * float(bcum))
            checked += 1
    assert checked > 200


def test_random_sample_invariants():
    rng = np.random.default_rng(1)
    x = np.round(rng.standard_normal(500) * 3).astype(f16)
    top = float(x.max())
    idx0, v0 = oracle.random_sample(x, 0.8, 0.9, 50, 0.0)
    assert idx0 == int(np.argmax(x)) and float(x[idx0]) == top  # seed 0: first (smallest index) maximum
    assert (v0 & 0xFFFF) == 0x3C00  # its running sum is exactly 1
    order = np.lexsort((np.arange(500), -x.astype(f64)))
    rank = {int(o): i for i, o in enumerate(order)}
    last = -1
    for s in np.linspace(0, 1, 41):
        idx, _ = oracle.random_sample(x, 0.8, 0.9, 50, float(s))
        assert rank[idx] >= last and rank[idx] < 50
        last = rank[idx]
    # seed 1, top_p 1, small top_k: the k-th entry of the order
    idx, _ = oracle.random_sample(x, 0.8, 1.0, 7, 1.0)
    assert idx == int(order[6])
    # temperature 0 or top_k 1 means argmax (last maximum)
    assert oracle.random_sample(x, 0.0, 0.9, 50, 0.3)[0] == oracle.argmax(x)[0]
    assert oracle.random_sample(x, 0.8, 0.9, 1, 0.3)[0] == oracle.argmax(x)[0]


# -------------------------------------------------------------- mat_mul ----

def lay(arr):
    return (arr.shape, arr.strides)


def test_mat_mul_layout_hand_cases():
    c = np.zeros((5, 7), f16)
    a = np.zeros((5, 3), f16)
    b = np.zeros((3, 7), f16)
    L = oracle.mat_mul_layout(2, lay(c), lay(a), lay(b)).as_dict()
    # row-major C: transpose everything and swap A and B
    assert L == dict(ab_swap=1, a_trans=0, b_trans=0, batch=1, m=7, n=5, k=3, c_stride=0, c_ld=7,
                     a_stride=0, a_ld=7, b_stride=0, b_ld=3)
    L = oracle.mat_mul_layout(2, lay(c.T.copy().T), lay(a), lay(b)).as_dict()  # column-major C
    assert (L["ab_swap"], L["m"], L["n"], L["k"], L["c_ld"]) == (0, 5, 7, 3, 5)
    assert (L["a_trans"], L["a_ld"], L["b_trans"], L["b_ld"]) == (1, 3, 1, 7)
    # each operand may be given transposed
    L = oracle.mat_mul_layout(2, lay(c), lay(np.zeros((3, 5), f16).T), lay(np.zeros((7, 3), f16).T)).as_dict()
    assert (L["ab_swap"], L["a_trans"], L["a_ld"], L["b_trans"], L["b_ld"]) == (1, 1, 3, 1, 5)
    # batches: a broadcast operand gets stride 0
    L = oracle.mat_mul_layout(2, lay(np.zeros((4, 5, 7), f16)), lay(np.zeros((4, 5, 3), f16)),
                              lay(np.zeros((1, 3, 7), f16))).as_dict()
    assert (L["batch"], L["c_stride"], L["a_stride"], L["b_stride"]) == (4, 35, 0, 15)  # after the swap a <- B
    for bad, kind in [
        ((lay(np.zeros((5, 7), f16)), lay(np.zeros((5, 4), f16)), lay(b)), "ShapeMismatch"),
        ((lay(np.zeros((5, 14), f16)[:, ::2].T[::1].T[::2]), lay(np.zeros((3, 3), f16)), lay(b)), "StridesNotSupport"),
        ((lay(np.zeros(7, f16)), lay(a), lay(b)), "RankNotSupport"),
        ((lay(np.zeros((1, 1, 5, 7), f16)), lay(a), lay(b)), "ShapeNotSupport"),
        ((lay(np.zeros((2, 5, 7), f16)), lay(np.zeros((3, 5, 3), f16)), lay(b)), "ShapeMismatch"),
    ]:
        with pytest.raises(oracle.OracleError) as e:
            oracle.mat_mul_layout(2, *bad)
        assert e.value.kind == kind, (kind, e.value.kind)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("tc", [False, True])
def test_mat_mul_against_numpy(ta, tb, tc):
    rng = np.random.default_rng(0)
    bt, m, n, k = 3, 9, 11, 40
    a = rng.standard_normal((bt, k, m) if ta else (bt, m, k)).astype(f16)
    b = rng.standard_normal((1, n, k) if tb else (1, k, n)).astype(f16)  # broadcast batch
    c = rng.standard_normal((bt, n, m) if tc else (bt, m, n)).astype(f16)
    av = a.transpose(0, 2, 1) if ta else a
    bv = b.transpose(0, 2, 1) if tb else b
    cv = c.transpose(0, 2, 1) if tc else c
    c0 = cv.astype(f64).copy()
    oracle.mat_mul(cv, 1.0, av, bv, 0.5)
    ref = 0.5 * av.astype(f64) @ bv.astype(f64) + c0
    assert (np.abs(cv.astype(f64) - ref) <= 0.5 * ulp16(ref) + 1e-5 * np.abs(ref) + 1e-5).all()


def test_mat_mul_beta_zero_ignores_c_and_scalars_are_rounded_to_f16():
    a = np.ones((1, 2047), f16)
    b = np.ones((2047, 1), f16)
    c = np.array([[np.nan]], f16)
    oracle.mat_mul(c, 0.0, a, b, 0.1)
    # alpha is first rounded to f16 (0.0999755859375): 2047 * alpha' = 204.65 -> 204.625; with 0.1 it would be 204.75
    assert float(c[0, 0]) == 204.625
    c32 = np.array([[np.nan]], f32)
    oracle.mat_mul(c32, 0.0, a.astype(f32), b.astype(f32), 0.1)
    assert float(c32[0, 0]) == pytest.approx(204.7, rel=1e-6)
    c = np.array([[2.0]], f16)
    oracle.mat_mul(c, 0.5, a[:, :4], b[:4], 1.0)
    assert float(c[0, 0]) == 5.0


def test_threads_do_not_change_results():
    rng = np.random.default_rng(0)
    att = (rng.standard_normal((4, 16, 64)) * 2).astype(f16)
    a = rng.standard_normal((64, 96)).astype(f16)
    b = rng.standard_normal((96, 300)).astype(f16)
    oracle.set_threads(1)
    s1 = oracle.fused_softmax(att.copy())
    m1 = oracle.mat_mul(np.zeros((64, 300), f16), 0.0, a, b, 1.0)
    oracle.set_threads(4)
    s4 = oracle.fused_softmax(att.copy())
    m4 = oracle.mat_mul(np.zeros((64, 300), f16), 0.0, a, b, 1.0)
    oracle.set_threads(1)
    assert np.array_equal(s1, s4) and np.array_equal(m1, m4)
