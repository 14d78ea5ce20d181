"""Shared helpers for the parity tests: synthetic inputs and the comparison bars."""
import numpy as np

F16_EPS = 9.765625e-4  # f16::EPSILON, the abs threshold of the reference's device tests


def normal_f16(rng, shape, std=1.0):
    """One f32 draw rounded once to f16 (RNE); the same bytes feed the oracle and the GPU."""
    return (rng.standard_normal(shape).astype(np.float32) * np.float32(std)).astype(np.float16)


def margins_f16(ans, ref):
    """What the bars below are measured on, as numbers: the largest absolute error, the largest relative error among the
    elements whose absolute error exceeds f16 eps (relative errors of values near zero say nothing), and the count of
    outliers by the reference crate's ErrorCollector rule (common/mod.rs:69-117)."""
    a = np.asarray(ans, dtype=np.float64).ravel()
    r = np.asarray(ref, dtype=np.float64).ravel()
    ok = ~np.isnan(r)
    a, r = a[ok], r[ok]
    err = np.abs(a - r)
    rel = err / np.maximum(np.abs(r), 1e-300)
    rel2 = err / (np.abs(a) + np.abs(r) + np.finfo(np.float64).eps)
    big = err > F16_EPS
    return {"max_abs": float(err.max()) if err.size else 0.0, "max_rel": float(rel[big].max()) if big.any() else 0.0,
            "outliers": int((big & (rel2 > 1e-3)).sum()), "elements": int(a.size)}


def assert_close_f16(ans, ref, what="", abs_tol=2e-3, rel_tol=1e-2):
    """The bar for f16 outputs: every element within max-abs 2e-3 or relative 1e-2
    of the oracle, plus the reference crate's own rule (common/mod.rs:69-117):
    at most 0.1 % of elements with abs > f16 eps AND rel > 1e-3."""
    a = np.asarray(ans, dtype=np.float64).ravel()
    r = np.asarray(ref, dtype=np.float64).ravel()
    assert a.shape == r.shape, (a.shape, r.shape)
    assert np.array_equal(np.isnan(a), np.isnan(r)), "%s: NaN pattern differs" % what
    ok = ~np.isnan(r)
    a, r = a[ok], r[ok]
    err = np.abs(a - r)
    rel = err / np.maximum(np.abs(r), 1e-300)
    bad = (err > abs_tol) & (rel > rel_tol)
    assert not bad.any(), "%s: %d elements beyond abs %g / rel %g (max abs %g, at ref %g)" % (
        what, bad.sum(), abs_tol, rel_tol, err.max(), r[np.argmax(err)])
    rel2 = err / (np.abs(a) + np.abs(r) + np.finfo(np.float64).eps)
    outliers = ((err > F16_EPS) & (rel2 > 1e-3)).sum()
    assert outliers * 1000 <= a.size, "%s: %d / %d outliers by the reference's ErrorCollector rule" % (
        what, outliers, a.size)
    return err.max() if err.size else 0.0


def strided_view(buf, dtype, shape, strides, offset=0):
    """A numpy view over a byte buffer with explicit byte strides."""
    return np.lib.stride_tricks.as_strided(
        np.frombuffer(buf, dtype=dtype, count=1, offset=offset), shape=shape, strides=strides, writeable=True)
