"""Committed fixtures (tests/golden/): the reference's own known answers as data, and small
seeded vectors with the oracle's outputs.  On the CPU they pin the oracle (and the host-side
planners); on the GPU the HIP backend must reproduce them through the C ABI - exactly where the
operator is integer / byte / single-rounding work, within the f16 bar elsewhere."""
import json
import os

import numpy as np
import pytest

import ophip
import oracle
from helpers import assert_close_f16
from ophip import TensorLayout, dt

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))
VEC = json.load(open(os.path.join(HERE, "golden", "vectors.json")))

f16, f32 = np.float16, np.float32


def arr(hexstr, dtype, shape=None):
    a = np.frombuffer(bytes.fromhex(hexstr), dtype=dtype).copy()
    return a.reshape(shape) if shape is not None else a


# ------------------------------------------------------------------ CPU ----

def test_reference_rearrange_known_answers_oracle_and_host_planner():
    k0, k1 = KATS["rearrange_scheme"]
    for plan in (lambda k: oracle.rearrange_scheme(k["shape"], k["dst_strides"], k["src_strides"], k["elem_size"]),
                 lambda k: ophip.Rearrange.plan(ophip.RearrangeArgs(
                     TensorLayout(dt.F16, k["shape"], k["dst_strides"]), None,
                     TensorLayout(dt.F16, k["shape"], k["src_strides"]), None))):
        s = plan(k0)
        e = k0["expect"]
        nd = (len(s) - 2) // 3
        assert nd == e["ndim"] and s[0] == e["unit"] and s[1] == e["count"]
        assert s[2:2 + nd] == e["idx_strides"] and s[2 + nd:2 + 2 * nd] == e["dst_strides"]
        assert s[2 + 2 * nd:] == e["src_strides"]
        assert [s[1 + i] // s[2 + i] for i in range(nd)] == e["shape"]
        assert plan(k1) == k1["expect_vector"]
    assert oracle.rearrange_distribute_unit(k1["expect_vector"], k1["distribute_unit_candidates"]) == \
        k1["expect_distributed"]


def test_oracle_reproduces_the_committed_vectors():
    v = VEC["rms_norm"]
    x, w = arr(v["x"], f16, v["shape"]), arr(v["w"], f16)
    assert oracle.rms_norm(np.empty_like(x), x, w, v["epsilon"]).tobytes().hex() == v["y"]
    v = VEC["rope"]
    assert oracle.rope(arr(v["t"], f16, v["shape"]), arr(v["pos"], np.uint32), v["theta"]).tobytes().hex() == v["out"]
    v = VEC["fused_softmax"]
    assert oracle.fused_softmax(arr(v["att"], f16, v["shape"]), True).tobytes().hex() == v["causal"]
    assert oracle.fused_softmax(arr(v["att"], f16, v["shape"]), False).tobytes().hex() == v["none"]
    v = VEC["swiglu"]
    assert oracle.swiglu(arr(v["gate"], f16, v["shape"]), arr(v["up"], f16, v["shape"])).tobytes().hex() == v["out"]
    v = VEC["rearrange"]
    dst = np.zeros((3, 2, 4), np.uint16)
    oracle.rearrange(dst.transpose(1, 0, 2), arr(v["src"], np.uint16, v["shape"]))
    assert dst.tobytes().hex() == v["dst_as_3_2_4"]
    for c in VEC["argmax"]:
        assert oracle.argmax(arr(c["logits"], f16)) == (c["idx"], c["val_bits"]), c["name"]
    for c in VEC["random_sample"]:
        got = oracle.random_sample(arr(c["logits"], f16), c["temperature"], c["top_p"], c["top_k"], c["seed"])
        assert got == (c["idx"], c["val_bits"])
    v = VEC["mat_mul"]
    out = oracle.mat_mul(arr(v["c"], f16, (v["m"], v["n"])), v["beta"], arr(v["a"], f16, (v["m"], v["k"])),
                         arr(v["b"], f16, (v["k"], v["n"])), v["alpha"])
    assert out.tobytes().hex() == v["out"]
    v = VEC["layer_norm"]
    x = arr(v["x"], f16, v["shape"])
    assert oracle.layer_norm(np.empty_like(x), x, arr(v["scale_f32"], f32), arr(v["bias_f32"], f32),
                             v["epsilon"]).tobytes().hex() == v["y"]
    v = VEC["gelu"]
    assert oracle.gelu(arr(v["x"], f16, v["shape"])).tobytes().hex() == v["out"]
    v = VEC["add"]
    a = arr(v["a"], f16, v["shape"])
    assert oracle.add(np.zeros_like(a), a, arr(v["b"], f16, v["shape"])).tobytes().hex() == v["c"]
    v = VEC["add_rows"]
    assert oracle.add_rows(arr(v["dst"], f16, v["dst_shape"]), arr(v["src"], f16, v["src_shape"]),
                           arr(v["idx"], np.uint32, (2, 2))).tobytes().hex() == v["out"]
    v = VEC["attention"]
    q = arr(v["q"], f16, (v["nh"], v["seq"], v["dh"]))
    kv = (v["nkvh"], v["att"], v["dh"])
    assert oracle.attention(q, arr(v["k"], f16, kv), arr(v["v"], f16, kv), np.zeros_like(q)).tobytes().hex() == v["o"]


# ------------------------------------------------------------------ GPU ----

def _dev(gpu, a):
    return gpu.from_host(np.ascontiguousarray(a))


def _back(gpu, stream, mem, like):
    return gpu.to_host(mem, like.dtype, like.size, stream=stream).reshape(like.shape)


@pytest.mark.gpu
def test_hip_backend_reproduces_the_committed_vectors(gpu, stream):
    lay = TensorLayout.of
    print("golden vectors on the GPU", flush=True)
    v = VEC["rms_norm"]
    x, w, y = arr(v["x"], f16, v["shape"]), arr(v["w"], f16), arr(v["y"], f16, v["shape"])
    xd, wd, yd = _dev(gpu, x), _dev(gpu, w), gpu.malloc(x.nbytes)
    ophip.RmsNorm(gpu).launch(ophip.RmsNormArgs(lay(x), yd, lay(x), xd, lay(w), wd, v["epsilon"]), None, stream)
    assert_close_f16(_back(gpu, stream, yd, y), y, "golden rms_norm")

    v = VEC["rope"]
    t, pos, out = arr(v["t"], f16, v["shape"]), arr(v["pos"], np.uint32), arr(v["out"], f16, v["shape"])
    td, pd = _dev(gpu, t), _dev(gpu, pos)
    empty = TensorLayout(dt.F16, [0, 8], [16, 2])
    ophip.Rope(gpu).launch(ophip.RopeArgs(lay(t), td, lay(pos), pd, empty, None, empty, None, v["theta"]), None, stream)
    assert_close_f16(_back(gpu, stream, td, t), out, "golden rope")

    v = VEC["fused_softmax"]
    for mask, key in ((ophip.AttnMask.CAUSAL, "causal"), (ophip.AttnMask.NONE, "none")):
        att, want = arr(v["att"], f16, v["shape"]), arr(v[key], f16, v["shape"])
        ad = _dev(gpu, att)
        ophip.FusedSoftmax(gpu).launch(ophip.FusedSoftmaxArgs(mask, lay(att), ad), None, stream)
        got = _back(gpu, stream, ad, att)
        assert_close_f16(got, want, "golden softmax " + key)
        assert np.array_equal(got == 0, want == 0)  # the masked tail is exactly zero

    v = VEC["swiglu"]
    g, u, want = arr(v["gate"], f16, v["shape"]), arr(v["up"], f16, v["shape"]), arr(v["out"], f16, v["shape"])
    gd, ud = _dev(gpu, g), _dev(gpu, u)
    ophip.Swiglu(gpu).launch(ophip.SwigluArgs(lay(g), gd, lay(u), ud), None, stream)
    assert_close_f16(_back(gpu, stream, gd, g), want, "golden swiglu")

    v = VEC["rearrange"]
    src, want = arr(v["src"], np.uint16, v["shape"]), arr(v["dst_as_3_2_4"], np.uint16, (3, 2, 4))
    sd, dd = _dev(gpu, src), gpu.malloc(src.nbytes)
    ophip.Rearrange(gpu).launch(ophip.RearrangeArgs(lay(want.transpose(1, 0, 2)), dd, lay(src), sd), None, stream)
    assert np.array_equal(_back(gpu, stream, dd, want), want)

    rs = ophip.RandomSample(gpu)
    kvd = gpu.malloc(8)
    for c in VEC["argmax"] + VEC["random_sample"]:
        lg = arr(c["logits"], f16)
        ld = _dev(gpu, lg)
        a = ophip.RandomSampleArgs.layout(dt.F16, lg.size)
        a.kv_pair_base, a.logits_base = kvd, ld
        if "seed" in c:
            a.config, a.seed = ophip.SampleArgs(c["temperature"], c["top_p"], c["top_k"]), c["seed"]
        else:
            a.config, a.seed = ophip.SampleArgs.argmax(), 0.0
        rs.launch(a, None, stream)
        idx, val = gpu.to_host(kvd, np.uint32, 2, stream=stream)
        assert int(idx) == c["idx"], c
        if "seed" not in c:
            assert int(val) == c["val_bits"], c

    v = VEC["mat_mul"]
    a_, b_, c_ = arr(v["a"], f16, (v["m"], v["k"])), arr(v["b"], f16, (v["k"], v["n"])), arr(v["c"], f16, (v["m"], v["n"]))
    ad, bd, cd = _dev(gpu, a_), _dev(gpu, b_), _dev(gpu, c_)
    ophip.MatMul(gpu).launch(ophip.MatMulArgs(lay(c_), cd, v["beta"], lay(a_), ad, lay(b_), bd, v["alpha"]), None, stream)
    assert_close_f16(_back(gpu, stream, cd, c_), arr(v["out"], f16, c_.shape), "golden mat_mul")

    v = VEC["layer_norm"]
    x, s, b = arr(v["x"], f16, v["shape"]), arr(v["scale_f32"], f32), arr(v["bias_f32"], f32)
    xd, sd, bd, yd = _dev(gpu, x), _dev(gpu, s), _dev(gpu, b), gpu.malloc(x.nbytes)
    ophip.LayerNorm(gpu).launch(ophip.LayerNormArgs(lay(x), yd, lay(x), xd, lay(s), sd, lay(b), bd, v["epsilon"]), None,
                                stream)
    assert_close_f16(_back(gpu, stream, yd, x), arr(v["y"], f16, v["shape"]), "golden layer_norm")

    v = VEC["gelu"]
    x = arr(v["x"], f16, v["shape"])
    xd = _dev(gpu, x)
    ophip.Gelu(gpu).launch(ophip.GeluArgs(lay(x), xd), None, stream)
    assert_close_f16(_back(gpu, stream, xd, x), arr(v["out"], f16, v["shape"]), "golden gelu")

    v = VEC["add"]
    a_, b_ = arr(v["a"], f16, v["shape"]), arr(v["b"], f16, v["shape"])
    ad, bd, cd = _dev(gpu, a_), _dev(gpu, b_), gpu.malloc(a_.nbytes)
    ophip.Add(gpu).launch(ophip.AddArgs(lay(a_), cd, lay(a_), ad, lay(b_), bd), None, stream)
    assert _back(gpu, stream, cd, a_).tobytes().hex() == v["c"]

    v = VEC["add_rows"]
    d_, s_, i_ = arr(v["dst"], f16, v["dst_shape"]), arr(v["src"], f16, v["src_shape"]), arr(v["idx"], np.uint32, (2, 2))
    dd, sd, idd = _dev(gpu, d_), _dev(gpu, s_), _dev(gpu, i_)
    ophip.AddRows(gpu).launch(ophip.AddRowsArgs(lay(d_), dd, lay(s_), sd, lay(i_), idd), None, stream)
    assert _back(gpu, stream, dd, d_).tobytes().hex() == v["out"]

    v = VEC["attention"]
    q = arr(v["q"], f16, (v["nh"], v["seq"], v["dh"]))
    kv = (v["nkvh"], v["att"], v["dh"])
    k_, v_ = arr(v["k"], f16, kv), arr(v["v"], f16, kv)
    qd, kd, vd, od = _dev(gpu, q), _dev(gpu, k_), _dev(gpu, v_), gpu.malloc(q.nbytes)
    ophip.Attention(gpu).launch(ophip.AttentionArgs(lay(q), qd, lay(k_), kd, lay(v_), vd, lay(q), od,
                                                    ophip.AttnMask.CAUSAL), None, stream)
    assert_close_f16(_back(gpu, stream, od, q), arr(v["o"], f16, q.shape), "golden attention")
