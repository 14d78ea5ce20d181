#!/usr/bin/env python3
"""Writes tests/golden/vectors.json: small seeded inputs and the CPU oracle's outputs for every
operator, as hex strings of the raw little-endian bytes.  The vectors pin the oracle against
drift (tests/test_golden.py, CPU) and give the HIP backend fixed known answers (GPU).  They are
regenerated only on purpose:  python tests/golden/make_vectors.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

f16, f32 = np.float16, np.float32


def hx(a):
    return np.ascontiguousarray(a).tobytes().hex()


def nf16(rng, shape, std=1.0):
    return (rng.standard_normal(shape).astype(f32) * f32(std)).astype(f16)


def main():
    rng = np.random.default_rng(20240607)
    v = {}

    x, w = nf16(rng, (2, 16)), rng.uniform(0.5, 1.5, 16).astype(f32).astype(f16)
    v["rms_norm"] = {"shape": [2, 16], "epsilon": 1e-5, "x": hx(x), "w": hx(w),
                     "y": hx(oracle.rms_norm(np.empty_like(x), x, w, 1e-5))}

    t, pos = nf16(rng, (3, 2, 8)), np.array([0, 5, 1000], np.uint32)
    v["rope"] = {"shape": [3, 2, 8], "theta": 1e4, "t": hx(t), "pos": hx(pos), "out": hx(oracle.rope(t.copy(), pos, 1e4))}

    att = nf16(rng, (2, 3, 8), 2.0)
    v["fused_softmax"] = {"shape": [2, 3, 8], "att": hx(att), "causal": hx(oracle.fused_softmax(att.copy(), True)),
                          "none": hx(oracle.fused_softmax(att.copy(), False))}

    gate, up = nf16(rng, (2, 8), 2.0), nf16(rng, (2, 8))
    v["swiglu"] = {"shape": [2, 8], "gate": hx(gate), "up": hx(up), "out": hx(oracle.swiglu(gate.copy(), up))}

    src = rng.integers(0, 65536, (2, 3, 4)).astype(np.uint16)
    dst = np.zeros((3, 2, 4), np.uint16)
    oracle.rearrange(dst.transpose(1, 0, 2), src)
    v["rearrange"] = {"shape": [2, 3, 4], "src": hx(src), "dst_as_3_2_4": hx(dst)}

    cases = []
    nan = float("nan")
    for name, vals in (("ties keep the last maximum", [1, 5, 2, 5, 3, 5, 0]),
                       ("all equal", [2, 2, 2, 2]),
                       ("negative zero after zero", [0.0, -0.0, -1.0]),
                       ("NaN restarts the scan", [9, nan, 1, 3, 2]),
                       ("trailing NaN wins", [1, 2, nan])):
        lg = np.array(vals, f32).astype(f16)
        idx, val = oracle.argmax(lg)
        cases.append({"name": name, "logits": hx(lg), "n": len(vals), "idx": int(idx), "val_bits": int(val)})
    v["argmax"] = cases

    cases = []
    for n, temp, top_p, top_k, seed in ((40, 0.8, 0.9, 5, 0.37), (40, 1.0, 1.0, 40, 0.99), (33, 0.5, 0.3, 10, 0.0),
                                        (64, 2.0, 0.75, 64, 0.5)):
        lg = nf16(rng, (n,), np.sqrt(3.0))
        lg[3] = lg[17]  # a tie inside the vector
        idx, val = oracle.random_sample(lg, temp, top_p, top_k, seed)
        cases.append({"n": n, "temperature": temp, "top_p": top_p, "top_k": top_k, "seed": seed, "logits": hx(lg),
                      "idx": int(idx), "val_bits": int(val)})
    v["random_sample"] = cases

    a, b, c = nf16(rng, (4, 8)), nf16(rng, (8, 5)), nf16(rng, (4, 5))
    v["mat_mul"] = {"m": 4, "k": 8, "n": 5, "alpha": 0.5, "beta": 1.0, "a": hx(a), "b": hx(b), "c": hx(c),
                    "out": hx(oracle.mat_mul(c.copy(), 1.0, a, b, 0.5))}

    x = nf16(rng, (2, 16), 1.5)
    s, bi = rng.uniform(0.5, 1.5, 16).astype(f32), rng.uniform(-1, 1, 16).astype(f32)
    v["layer_norm"] = {"shape": [2, 16], "epsilon": 1e-5, "x": hx(x), "scale_f32": hx(s), "bias_f32": hx(bi),
                       "y": hx(oracle.layer_norm(np.empty_like(x), x, s, bi, 1e-5))}

    x = nf16(rng, (2, 8), 2.5)
    v["gelu"] = {"shape": [2, 8], "x": hx(x), "out": hx(oracle.gelu(x.copy()))}

    a, b = nf16(rng, (3, 8)), nf16(rng, (3, 8))
    v["add"] = {"shape": [3, 8], "a": hx(a), "b": hx(b), "c": hx(oracle.add(np.zeros_like(a), a, b))}

    dst, srcr, idx = nf16(rng, (2, 2, 8)), nf16(rng, (5, 8)), np.array([[4, 0], [2, 4]], np.uint32)
    v["add_rows"] = {"dst_shape": [2, 2, 8], "src_shape": [5, 8], "dst": hx(dst), "src": hx(srcr), "idx": hx(idx),
                     "out": hx(oracle.add_rows(dst.copy(), srcr, idx))}

    q, k, vv = nf16(rng, (4, 2, 8)), nf16(rng, (2, 5, 8)), nf16(rng, (2, 5, 8))
    v["attention"] = {"nh": 4, "nkvh": 2, "seq": 2, "att": 5, "dh": 8, "q": hx(q), "k": hx(k), "v": hx(vv),
                      "o": hx(oracle.attention(q.copy(), k, vv, np.zeros_like(q), causal=True))}

    with open(os.path.join(HERE, "vectors.json"), "w") as f:
        json.dump(v, f, indent=1)
    print("wrote", os.path.join(HERE, "vectors.json"))


if __name__ == "__main__":
    main()
