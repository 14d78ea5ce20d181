"""Pins for the oracle's layer_norm, gelu, add and add_rows: closed forms in f64, special cases
whose answer is known exactly, and an explicit numpy-f32 replay of every rounding point."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_f16, normal_f16

f16, f32 = np.float16, np.float32


# ------------------------------------------------------------ layer_norm ----

def layer_norm_f64(x, s, b, eps):
    x64 = x.astype(np.float64)
    e = x64.mean(1, keepdims=True)
    std = np.sqrt((x64 ** 2).mean(1, keepdims=True) - e ** 2)
    return (x64 - e) * (s.astype(np.float64) / (std + eps)) + b.astype(np.float64)


@pytest.mark.parametrize("wdt", [f16, f32])
def test_layer_norm_f64_closed_form(wdt):
    rng = np.random.default_rng(1)
    x = normal_f16(rng, (9, 768), std=2.0) + f16(0.5)
    s, b = rng.uniform(0.5, 1.5, 768).astype(wdt), rng.uniform(-1, 1, 768).astype(wdt)
    for eps in (1e-5, 0.5):  # epsilon is added to the standard deviation, not the variance
        y = oracle.layer_norm(np.empty_like(x), x, s, b, eps)
        assert_close_f16(y, layer_norm_f64(x, s, b, eps), "layer_norm vs f64 eps=%g" % eps)
    wrong = (x.astype(np.float64) - x.astype(np.float64).mean(1, keepdims=True)) / np.sqrt(
        x.astype(np.float64).var(1, keepdims=True) + 0.5) * s + b
    assert np.abs(oracle.layer_norm(np.empty_like(x), x, s, b, 0.5).astype(np.float64) - wrong).max() > 0.05


def test_layer_norm_constant_row_returns_bias_and_unit_scale_centres():
    d = 256
    x = np.full((3, d), 1.5, f16)
    s, b = np.full(d, 2.0, f32), np.linspace(-1, 1, d).astype(f32)
    y = oracle.layer_norm(np.empty_like(x), x, s, b, 1e-5)  # sums of 1.5 are exact: x - e == 0
    assert np.array_equal(y, np.broadcast_to(b.astype(f16), (3, d)))
    rng = np.random.default_rng(2)
    x = rng.standard_normal((4, 512)).astype(f32)
    y = oracle.layer_norm(np.empty_like(x), x, np.ones(512, f32), np.zeros(512, f32), 0.0)
    assert np.abs(y.mean(1)).max() < 1e-6 and np.abs(y.std(1) - 1).max() < 1e-5


def test_layer_norm_replay_of_rounding_points_in_numpy_f32():
    rng = np.random.default_rng(3)
    x = normal_f16(rng, (2, 100))
    s, b = rng.uniform(0.5, 1.5, 100).astype(f32), rng.uniform(-1, 1, 100).astype(f32)
    y = oracle.layer_norm(np.empty_like(x), x, s, b, 1e-5)
    for i in range(2):
        sm, sm2 = f32(0), f32(0)
        for v in x[i].astype(f32):
            sm = f32(sm + v)
            sm2 = f32(sm2 + f32(v * v))
        e, e2 = f32(sm / f32(100)), f32(sm2 / f32(100))
        k = f32(f32(1) / f32(np.sqrt(f32(e2 - f32(e * e))) + f32(1e-5)))
        # fma: exact product and sum in f64 (24-bit x 24-bit products are exact), one rounding to f32
        want = ((x[i].astype(f32) - e).astype(np.float64) * (s * k).astype(f32).astype(np.float64)
                + b.astype(np.float64)).astype(f32).astype(f16)
        assert np.array_equal(y[i], want)


# ------------------------------------------------------------------ gelu ----

def test_gelu_closed_form_and_special_values():
    rng = np.random.default_rng(4)
    x = normal_f16(rng, (7, 333), std=3.0)
    y = oracle.gelu(x.copy())
    x64 = x.astype(np.float64)
    ref = 0.5 * x64 * (1 + np.tanh(np.sqrt(2 / np.pi) * (x64 + 0.044715 * x64 ** 3)))
    assert_close_f16(y, ref, "gelu vs f64")
    z = oracle.gelu(np.array([[0.0, -0.0, 20.0, -20.0, 1.0]], f32))
    assert z[0, 0] == 0 and z[0, 2] == 20.0 and z[0, 3] == 0 and np.signbit(z[0, 3])
    assert abs(z[0, 4] - 0.8411919906082768) < 1e-6   # tanh-form gelu(1)
    xs = rng.standard_normal((1, 1000)).astype(f32)
    odd = oracle.gelu(xs.copy()) - oracle.gelu(-xs)     # gelu(x) - gelu(-x) = x
    assert np.abs(odd - xs).max() < 1e-6


# ------------------------------------------------------------------- add ----

@pytest.mark.parametrize("dtype", [f16, f32])
def test_add_matches_numpy_on_strided_and_broadcast_views(dtype):
    rng = np.random.default_rng(5)
    a = rng.standard_normal((6, 5, 8)).astype(f32).astype(dtype)
    b = rng.standard_normal((8, 6)).astype(f32).astype(dtype)
    av = a.transpose(1, 0, 2)                                         # [5, 6, 8] permuted
    bv = np.lib.stride_tricks.as_strided(b, (5, 6, 8), (0, b.strides[1], b.strides[0]))  # broadcast over dim 0
    c = np.zeros((5, 8, 6), dtype).transpose(0, 2, 1)
    oracle.add(c, av, bv)
    assert np.array_equal(c, (av.astype(f32) + bv.astype(f32)).astype(dtype))  # f16 + f16 is exact in f32
    assert np.array_equal(oracle.add(np.zeros((), dtype), np.array(1.5, dtype), np.array(2.0, dtype)), dtype(3.5))


def test_add_errors_in_reference_order():
    z = lambda *s: np.zeros(s, f16)
    for args, kind in (((z(2, 3), z(2, 3), np.zeros((2, 3), f32)), "TypeMismatch"),
                       ((z(2, 3), z(6), z(2, 3)), "RankMismatch"),
                       ((z(2, 3), z(2, 4), z(2, 3)), "ShapeMismatch"),
                       ((np.lib.stride_tricks.as_strided(z(3), (2, 3), (0, 2)), z(2, 3), z(2, 3)), "ShapeNotSupport")):
        with pytest.raises(oracle.OracleError) as e:
            oracle.add(*args)
        assert e.value.kind == kind


# -------------------------------------------------------------- add_rows ----

@pytest.mark.parametrize("idt", [np.uint32, np.uint64])
def test_add_rows_matches_numpy_fancy_indexing(idt):
    rng = np.random.default_rng(6)
    batch, m, n, k = 3, 10, 40, 7
    dst, src = normal_f16(rng, (batch, m, n)), normal_f16(rng, (k, n))
    idx = rng.integers(0, k, (batch, m)).astype(idt)
    idx[0, 0], idx[0, 1], idx[1, 0] = 0, k - 1, k - 1        # boundaries and repeats
    want = (dst.astype(f32) + src[idx.astype(np.int64)].astype(f32)).astype(f16)
    assert np.array_equal(oracle.add_rows(dst, src, idx), want)
    bad = idx.copy()
    bad[2, 3] = k
    with pytest.raises(oracle.OracleError):
        oracle.add_rows(dst, src, bad)
