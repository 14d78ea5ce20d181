"""The oracle's attention composites against what the mathematics fixes: an f64
softmax(q k^T / sqrt(dh)) v with grouped kv heads and the causal rule of the crate's
fused softmax (row r of seq keeps att - seq + r + 1 columns)."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_f16, normal_f16

f16 = np.float16


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


@pytest.mark.parametrize("nh,nkvh,seq,att,dh,causal", [(32, 4, 7, 127, 64, True), (8, 8, 5, 5, 32, True),
                                                       (6, 2, 3, 40, 16, False), (4, 1, 1, 33, 8, True)])
def test_attention_matches_f64_closed_form(nh, nkvh, seq, att, dh, causal):
    rng = np.random.default_rng(nh * 1000 + att)
    q, k, v = (rng.random(s).astype(f16) for s in ((nh, seq, dh), (nkvh, att, dh), (nkvh, att, dh)))
    q0, o = q.copy(), np.zeros((nh, seq, dh), f16)
    oracle.attention(q, k, v, o, causal=causal)
    assert_close_f16(o, attention_f64(q0, k, v, causal), "attention vs f64")
    assert np.array_equal(q, o)  # contiguous q merges heads and tokens: the reference overwrites it


def test_attention_head_grouping_is_big_endian():
    """q head h reads kv head h // (nh / nkvh): make kv head 1 all-zero values and check exactly
    the second half of the q heads returns zeros."""
    rng = np.random.default_rng(3)
    nh, nkvh, seq, att, dh = 4, 2, 2, 6, 8
    q, k, v = (rng.random(s).astype(f16) for s in ((nh, seq, dh), (nkvh, att, dh), (nkvh, att, dh)))
    v[1] = 0
    o = np.ones((nh, seq, dh), f16)
    oracle.attention(q, k, v, o)
    assert (o[2:] == 0).all() and (o[:2] != 0).any()


def test_attention_strided_q_is_staged_and_left_alone():
    """q as the [token, head, dh] slice of a fused QKV buffer does not merge: the composite copies
    it (attention/operator.rs:194-210) and q keeps its values."""
    rng = np.random.default_rng(4)
    nh, seq, dh, att = 8, 6, 16, 20
    qkv = normal_f16(rng, (seq, 3 * nh * dh))
    q = qkv[:, :nh * dh].reshape(seq, nh, dh).transpose(1, 0, 2)
    k, v = normal_f16(rng, (nh, att, dh)), normal_f16(rng, (nh, att, dh))
    before = qkv.copy()
    obuf = np.zeros((seq, nh * dh), f16)
    o = obuf.reshape(seq, nh, dh).transpose(1, 0, 2)
    oracle.attention(q, k, v, o)
    assert np.array_equal(qkv, before)
    assert_close_f16(o, attention_f64(q, k, v, True), "strided attention vs f64")


def test_attention_kv_cached_appends_then_attends():
    rng = np.random.default_rng(5)
    nh, nkvh, seq, dh, buf, pos = 8, 2, 3, 16, 32, 9
    q, k, v = normal_f16(rng, (nh, seq, dh)), normal_f16(rng, (nkvh, seq, dh)), normal_f16(rng, (nkvh, seq, dh))
    kc, vc = normal_f16(rng, (nkvh, buf, dh)), normal_f16(rng, (nkvh, buf, dh))
    kc0, vc0, q0 = kc.copy(), vc.copy(), q.copy()
    o = np.zeros_like(q)
    oracle.attention_kv_cached(q, k, v, o, kc, vc, pos)
    assert np.array_equal(kc[:, pos:pos + seq], k) and np.array_equal(vc[:, pos:pos + seq], v)
    keep = np.ones(buf, bool)
    keep[pos:pos + seq] = False
    assert np.array_equal(kc[:, keep], kc0[:, keep]) and np.array_equal(vc[:, keep], vc0[:, keep])
    assert_close_f16(o, attention_f64(q0, kc[:, :pos + seq], vc[:, :pos + seq], True), "kv cached vs f64")
    with pytest.raises(oracle.OracleError) as e:
        oracle.attention_kv_cached(q, k, v, o, kc, vc, buf - seq + 1)
    assert e.value.kind == "ShapeMismatch"
