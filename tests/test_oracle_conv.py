"""The oracle's conv composite against a direct f64 cross-correlation."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_f16, normal_f16

f16 = np.float16


def conv_f64(x, w, b, strides, dilations):
    n, c, h, wd_ = x.shape
    m, _, hk, wk = w.shape
    (hs, ws), (hd, wd) = strides, dilations
    hy, wy = (h - ((hk - 1) * hd + 1)) // hs + 1, (wd_ - ((wk - 1) * wd + 1)) // ws + 1
    y = np.zeros((n, m, hy, wy))
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    for i in range(hy):
        for j in range(wy):
            patch = x64[:, :, i * hs:i * hs + (hk - 1) * hd + 1:hd, j * ws:j * ws + (wk - 1) * wd + 1:wd]
            y[:, :, i, j] = np.einsum("nckl,mckl->nm", patch, w64)
    return y + b.astype(np.float64)[None, :, None, None]


@pytest.mark.parametrize("n,c,h,w,m,hk,wk,strides,dilations", [(2, 3, 8, 8, 4, 3, 3, (1, 1), (1, 1)),
                                                               (1, 3, 28, 28, 8, 14, 14, (14, 14), (1, 1)),
                                                               (2, 2, 9, 11, 3, 2, 3, (1, 2), (2, 1)),
                                                               (1, 1, 5, 5, 1, 5, 5, (1, 1), (1, 1))])
def test_conv_matches_direct_correlation(n, c, h, w, m, hk, wk, strides, dilations):
    rng = np.random.default_rng(n + c + h + m)
    x, wt, b = normal_f16(rng, (n, c, h, w)), normal_f16(rng, (m, c, hk, wk), 0.2), normal_f16(rng, (m,))
    ref = conv_f64(x, wt, b, strides, dilations)
    y = np.full(ref.shape, np.nan, f16)  # overwritten by the bias first: NaN must not survive
    oracle.conv(y, x, wt, b, strides, dilations)
    assert_close_f16(y, ref, "conv vs f64", abs_tol=4e-3)


def test_conv_errors():
    z = lambda *s: np.zeros(s, f16)
    with pytest.raises(oracle.OracleError) as e:
        oracle.conv(z(1, 1, 2, 2), z(1, 1, 4, 4), z(1, 1, 3, 3), z(1), pads=(1, 0, 0, 0))
    assert e.value.kind == "ArgsNotSupport"
    with pytest.raises(oracle.OracleError) as e:
        oracle.conv(z(1, 1, 2, 2), z(1, 1, 6, 6), z(1, 1, 3, 3), z(1), strides=(2, 2))
    assert e.value.kind == "StridesNotSupport"
