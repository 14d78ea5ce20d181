"""conv (the im2col composite) on the HIP backend against the oracle's composite and a direct
f64 correlation, through the C ABI.  Shapes: small kernels, a ViT-style 14 x 14 patch embedding
(stride = kernel size), dilation and unequal strides."""
import numpy as np
import pytest

import ophip
import oracle
from helpers import assert_close_f16, normal_f16
from ophip import TensorLayout, dt
from test_oracle_conv import conv_f64

pytestmark = pytest.mark.gpu

f16 = np.float16


@pytest.mark.parametrize("n,c,h,w,m,hk,wk,strides,dilations", [(2, 3, 8, 8, 4, 3, 3, (1, 1), (1, 1)),
                                                               (2, 3, 224, 224, 64, 14, 14, (14, 14), (1, 1)),
                                                               (2, 2, 9, 11, 3, 2, 3, (1, 2), (2, 1)),
                                                               (1, 16, 32, 32, 32, 3, 3, (1, 1), (1, 1))])
def test_conv(gpu, stream, n, c, h, w, m, hk, wk, strides, dilations):
    rng = np.random.default_rng(n + c + h + m)
    x, wt, b = normal_f16(rng, (n, c, h, w)), normal_f16(rng, (m, c, hk, wk), 0.1), normal_f16(rng, (m,))
    ref64 = conv_f64(x, wt, b, strides, dilations)
    y = np.full(ref64.shape, np.nan, f16)
    xd, wd, bd, yd = (gpu.from_host(a) for a in (x, wt, b, y))
    lay = TensorLayout.of
    op = ophip.Conv(gpu)
    args = ophip.ConvArgs(lay(y), yd, lay(x), xd, lay(wt), wd, lay(b), bd, strides, dilations)
    need = op.scheme(args, 2 ** 40)
    assert need == n * c * hk * wk * y.shape[2] * y.shape[3] * 2
    assert op.scheme(args, need - 1) == 0
    print("conv n=%d c=%d %dx%d m=%d k=%dx%d" % (n, c, h, w, m, hk, wk), flush=True)
    ws = gpu.malloc(need + 4096)
    for workspace in (None, ws):
        gpu.memset(yd, 0xFF)
        op.launch(args, workspace, stream)
        out = gpu.to_host(yd, f16, y.size, stream=stream).reshape(y.shape)
        assert_close_f16(out, oracle.conv(y.copy(), x, wt, b, strides, dilations), "conv vs oracle", abs_tol=4e-3)
        assert_close_f16(out, ref64, "conv vs f64", abs_tol=4e-3)


def test_conv_errors(gpu, stream):
    op = ophip.Conv(gpu)
    c = lambda *s: TensorLayout.new_contiguous(dt.F16, list(s))
    base = dict(y_layout=c(1, 1, 2, 2), y_base=None, x_layout=c(1, 1, 4, 4), x_base=None, w_layout=c(1, 1, 3, 3),
                w_base=None, b_layout=c(1), b_base=None)
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.ConvArgs(**base, pads=(0, 1, 0, 0)), 0)
    assert e.value.kind == "ArgsNotSupport"
    with pytest.raises(ophip.LaunchError) as e:
        op.launch(ophip.ConvArgs(**dict(base, x_layout=c(1, 1, 6, 6)), strides=(2, 2)), None, stream)
    assert e.value.kind == "StridesNotSupport"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.ConvArgs(**dict(base, w_layout=c(1, 2, 3, 3))), 0)
    assert e.value.kind == "ShapeMismatch"
    with pytest.raises(ophip.SchemeError) as e:
        op.scheme(ophip.ConvArgs(**dict(base, b_layout=c(1, 1))), 0)
    assert e.value.kind == "RankNotSupport"
    dyn = lambda *s: TensorLayout(dt.F16, [None] + list(s), [None] * 4)
    assert op.scheme(ophip.ConvArgs(**dict(base, x_layout=dyn(1, 4, 4))), 2 ** 40) == 72  # n known from y
    assert op.scheme(ophip.ConvArgs(**dict(base, x_layout=dyn(1, 4, 4), y_layout=dyn(1, 2, 2))), 2 ** 40) == 0
