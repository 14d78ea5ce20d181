#!/usr/bin/env python3
"""Benchmark of the MI355X backend on the operators-rs hot path.

One "step" is one pass of the Llama-7B-shape decode layer (16 tokens, d = 4096,
32 heads x 128, KV length 2048, FFN 11008) through the operator API: rms_norm,
QKV mat_mul, rope (q and k in one launch: they are adjacent heads of the qkv rows),
QK^T mat_mul, causal softmax, PV mat_mul, O-proj mat_mul, rms_norm, gate/up mat_mul,
swiglu, down mat_mul - eleven launches on one stream, inputs resident in HBM, synthetic data.  `value` is the layer's
algorithmic bytes divided by the measured time per step.

Beside it the script reports, in the same JSON line:
  per_op       every operator at its benchmark shape (and a scaled shape large
               enough to leave the 256 MiB Infinity Cache): us/op, GB/s or
               TFLOP/s, fraction of the roofline; at the benchmark shapes of the single
               operators also `cpu_us`, the CPU oracle's time on the same shape;
  roofline     the dominant kernel of the step (the gate/up weight-streaming
               mat_mul), timed with HIP events inside the timed region;
  cpu_baseline the CPU oracle (a port of the crate's CPU backend) timed on the
               same layer on the host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "operators-rs_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12        # B/s, MI355X HBM3E
MFMA_F16_PEAK = 2.5e15   # flop/s, MI355X dense f16 MFMA

NT, D, NH, DH, KV, DI = 16, 4096, 32, 128, 2048, 11008
f16 = np.float16


def log(*a):
    print(*a, file=sys.stderr, flush=True)


_PROBE_LIB = None


def bench_probe(kind, dst, src, nbytes, iters, seed, blocks, stream):
    """One launch of a measurement probe (bench_probes/probe.hip, a library of its own beside the operator library)."""
    global _PROBE_LIB
    if _PROBE_LIB is None:
        path = os.path.join(ROOT, "bench_probes", "libbenchprobe.so")
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: make -C bench_probes" % path)
        _PROBE_LIB = ctypes.CDLL(path)
        _PROBE_LIB.bench_probe.argtypes = [ctypes.c_char_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint,
                                           ctypes.c_uint, ctypes.c_uint, ctypes.c_void_p]
        _PROBE_LIB.bench_probe_error.restype = ctypes.c_char_p
    ptr = lambda m: None if m is None else (m.ptr if hasattr(m, "ptr") else int(m))
    if _PROBE_LIB.bench_probe(kind.encode(), ptr(dst), ptr(src), nbytes, iters, seed, blocks, stream.handle):
        raise RuntimeError("bench_probe(%s): %s" % (kind, _PROBE_LIB.bench_probe_error().decode()))


def normal_f16(rng, shape, std):
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(f16)


class Layer:
    """Device buffers, Args and operators of one decode layer."""

    def __init__(self, ophip, gpu, rng, host=False):
        L, F16 = ophip.TensorLayout, ophip.dt.F16
        self.ophip, self.gpu = ophip, gpu
        h = self.h = {}
        h["x"] = normal_f16(rng, (NT, D), 1.0)
        h["w_norm1"] = rng.uniform(0.5, 1.5, D).astype(np.float32).astype(f16)
        h["w_norm2"] = rng.uniform(0.5, 1.5, D).astype(np.float32).astype(f16)
        h["w_qkv"] = normal_f16(rng, (D, 3 * D), 0.02)
        h["w_o"] = normal_f16(rng, (D, D), 0.02)
        h["w_gu"] = normal_f16(rng, (D, 2 * DI), 0.02)
        h["w_d"] = normal_f16(rng, (DI, D), 0.02)
        h["k_cache"] = normal_f16(rng, (NH, KV, DH), 1.0)
        h["v_cache"] = normal_f16(rng, (NH, KV, DH), 1.0)
        h["pos"] = (np.arange(NT) + KV - NT).astype(np.uint32)
        d = self.d = {k: gpu.from_host(v) for k, v in h.items()}
        for name, nbytes in [("xn", NT * D * 2), ("qkv", NT * 3 * D * 2), ("att", NH * NT * KV * 2),
                             ("o", NT * D * 2), ("y", NT * D * 2), ("yn", NT * D * 2), ("gu", NT * 2 * DI * 2),
                             ("out", NT * D * 2), ("ws", 64 << 20)]:
            d[name] = gpu.malloc(nbytes)
        if not host:
            self.h = {k: v for k, v in h.items() if k in ("x",)}  # drop host weights

        c = lambda *s: L.new_contiguous(F16, list(s))
        qb_lay = L(F16, [NH, NT, DH], [DH * 2, 3 * D * 2, 2])         # q as [head, token, dh]
        kt_lay = L(F16, [NH, DH, KV], [KV * DH * 2, 2, DH * 2])       # K-cache as K^T
        ob_lay = L(F16, [NH, NT, DH], [DH * 2, D * 2, 2])             # attention output as [token, head*dh]
        half = L(F16, [NT, DI], [2 * DI * 2, 2])                      # gate / up halves of gu
        empty = L(F16, [0, DH], [2 * DH, 2])
        o = ophip
        self.ops = dict(rms=o.RmsNorm(gpu), mm=o.MatMul(gpu), rope=o.Rope(gpu), sm=o.FusedSoftmax(gpu),
                        sw=o.Swiglu(gpu))
        A = self.args = {}
        A["rms_norm_1"] = ("rms", o.RmsNormArgs(c(NT, D), d["xn"], c(NT, D), d["x"], c(D), d["w_norm1"], 1e-5))
        A["qkv"] = ("mm", o.MatMulArgs(c(NT, 3 * D), d["qkv"], 0.0, c(NT, D), d["xn"], c(D, 3 * D), d["w_qkv"], 1.0))
        # q and k sit side by side in every token's qkv row: one rope launch over both, as 2 * NH heads
        qk_lay = L(F16, [NT, 2 * NH, DH], [3 * D * 2, DH * 2, 2])
        A["rope"] = ("rope", o.RopeArgs(qk_lay, d["qkv"].ptr, c(NT), d["pos"], empty, None, empty, None, 1e4))
        A["rope"][1].p_layout = L(o.dt.U32, [NT], [4])
        A["qk_t"] = ("mm", o.MatMulArgs(c(NH, NT, KV), d["att"], 0.0, qb_lay, d["qkv"].ptr, kt_lay, d["k_cache"],
                                        float(1.0 / np.sqrt(DH))))
        A["softmax"] = ("sm", o.FusedSoftmaxArgs(o.AttnMask.CAUSAL, c(NH, NT, KV), d["att"]))
        A["pv"] = ("mm", o.MatMulArgs(ob_lay, d["o"], 0.0, c(NH, NT, KV), d["att"], c(NH, KV, DH), d["v_cache"], 1.0))
        A["o_proj"] = ("mm", o.MatMulArgs(c(NT, D), d["y"], 0.0, c(NT, D), d["o"], c(D, D), d["w_o"], 1.0))
        A["rms_norm_2"] = ("rms", o.RmsNormArgs(c(NT, D), d["yn"], c(NT, D), d["y"], c(D), d["w_norm2"], 1e-5))
        A["gate_up"] = ("mm", o.MatMulArgs(c(NT, 2 * DI), d["gu"], 0.0, c(NT, D), d["yn"], c(D, 2 * DI), d["w_gu"], 1.0))
        A["swiglu"] = ("sw", o.SwigluArgs(half, d["gu"].ptr, half, d["gu"].ptr + DI * 2))
        A["down"] = ("mm", o.MatMulArgs(c(NT, D), d["out"], 0.0, half, d["gu"].ptr, c(DI, D), d["w_d"], 1.0))
        self.order = ["rms_norm_1", "qkv", "rope", "qk_t", "softmax", "pv", "o_proj", "rms_norm_2",
                      "gate_up", "swiglu", "down"]
        # The same layer as a runtime built on the crate would run it: the three attention launches replaced by the
        # crate's own composite attention_kv_cached (which also appends the 16 new k / v rows to the caches at
        # positions KV - NT .. KV, what the scripted chain leaves out).  q, k and v are views of the qkv rows.
        self.ops["akv"] = o.AttnKVCached(gpu)
        kv_new = lambda off: d["qkv"].ptr + off * 2
        A["attention_kv_cached"] = ("akv", o.AttnKVCachedArgs(
            qb_lay, kv_new(0), qb_lay, kv_new(D), qb_lay, kv_new(2 * D), ob_lay, d["o"],
            c(NH, KV, DH), d["k_cache"], c(NH, KV, DH), d["v_cache"], o.AttnMask.CAUSAL, KV - NT))
        self.order_attention_op = ["rms_norm_1", "qkv", "rope", "attention_kv_cached", "o_proj", "rms_norm_2",
                                   "gate_up", "swiglu", "down"]
        for name in self.order + ["attention_kv_cached"]:
            kind, a = A[name]
            self.ops[kind].scheme(a, 64 << 20)

    def launch(self, name, stream):
        kind, a = self.args[name]
        self.ops[kind].launch(a, self.d["ws"], stream)

    def step(self, stream, around=None, own=None, order=None):
        """around: {op: (e0, e1)} records the two events before and after the op's launch; own: {op: (e0, e1)} has
        the op's kernel record its own begin and end into them (ophip_time_next_launch); order: another sequence of
        launches than the benchmark's eleven (order_attention_op)."""
        for name in order or self.order:
            if around and name in around:
                around[name][0].record(stream)
                self.launch(name, stream)
                around[name][1].record(stream)
            elif own and name in own:
                self.gpu.time_next_launch(stream, own[name][0], own[name][1])
                self.launch(name, stream)
            else:
                self.launch(name, stream)


# algorithmic bytes (f16 operands read once, outputs written once) and flops per op of the layer
def layer_work():
    gemm = lambda m, n, k, b=1: (2 * b * (m * k + k * n + m * n), 2 * b * m * n * k)
    w = {
        "rms_norm_1": (2 * NT * D * 2 + D * 2, 0),
        "qkv": gemm(NT, 3 * D, D),
        "rope": (2 * (2 * NT * NH * DH * 2 + NT * 4), 0),  # q and k, the position vector counted for each
        "qk_t": gemm(NT, KV, DH, NH),
        "softmax": (2 * NH * NT * KV * 2, 0),
        "pv": gemm(NT, DH, KV, NH),
        "o_proj": gemm(NT, D, D),
        "rms_norm_2": (2 * NT * D * 2 + D * 2, 0),
        "gate_up": gemm(NT, 2 * DI, D),
        "swiglu": (3 * NT * DI * 2, 0),
        "down": gemm(NT, D, DI),
        # q, o, the new k / v rows read and appended, both caches read once
        "attention_kv_cached": (2 * NT * NH * DH * 2 + 4 * NT * NH * DH * 2 + 2 * NH * KV * DH * 2, 4 * NH * NT * KV * DH),
    }
    return w


def time_launches(gpu, stream, fn, reps, warm=5):
    for _ in range(warm):
        fn()
    e0, e1 = gpu.event(), gpu.event()
    stream.synchronize()
    e0.record(stream)
    for _ in range(reps):
        fn()
    e1.record(stream)
    e1.synchronize()
    return e0.elapsed_ms(e1) * 1e3 / reps  # us per launch


def time_sustained(gpu, stream, fn, seconds=0.3):
    """Per-launch time of a compute-bound kernel in steady state: the core clock takes a few hundred
    milliseconds of load to settle, so warm up for `seconds` and then time about as long."""
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn()
        stream.synchronize()
        n += 8
    return time_launches(gpu, stream, fn, max(n, 8), warm=0)


def profiled_traffic():
    """HBM bytes per launch of the dominant kernel, measured with FETCH_SIZE / WRITE_SIZE in separate
    counter runs and kept as text under profiles/ (a counter run cannot share a process with the timing)."""
    path = os.path.join(ROOT, "profiles", "gemm_stream_gate_up_pmc.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes"):
                return int(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def copy_ceiling(ophip, gpu, stream):
    """What a plain device-to-device copy of 1 GiB reaches (read + write counted): the practical
    ceiling for streaming kernels on this machine, and the known-size kernel that calibrates
    the FETCH_SIZE / WRITE_SIZE counters."""
    a_, b_ = gpu.malloc(1 << 30), gpu.malloc(1 << 30)
    gpu.memset(a_, 0x3C)
    us = time_launches(gpu, stream, lambda: ophip._check(ophip.lib().ophip_memcpy_d2d(
        gpu.handle, ctypes.c_void_p(b_.ptr), ctypes.c_void_p(a_.ptr), ctypes.c_size_t(1 << 30), stream.handle)), 10, warm=2)
    a_.free(); b_.free()
    log("  copy 1 GiB d2d (hipMemcpyAsync): %.1f us, %.1f GB/s read+write" % (us, (2 << 30) / us / 1e3))
    return {"bytes": 2 << 30, "us": round(us, 2), "GBps": round((2 << 30) / us / 1e3, 1),
            "hbm_frac": round((2 << 30) / (us * 1e-6) / HBM_PEAK, 4)}


def read_power():
    """Board power in watts from the amdgpu hwmon files, or None when they cannot be read."""
    import glob
    for pat in ("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average", "/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"):
        for f in sorted(glob.glob(pat)):
            try:
                return int(open(f).read().strip()) / 1e6
            except (OSError, ValueError):
                pass
    return None


def ceilings(ophip, gpu, stream):
    """What this machine gives a plain stream of 1 GiB (hipMemcpyAsync, and the library's probe kernels: read,
    read with non-temporal loads, write, copy; best grid of a few) and a bare MFMA loop (random-looking and all-zero
    operands, from idle clocks and in steady state, with the board power where the driver shows it)."""
    out = {"copy_hipMemcpyAsync": copy_ceiling(ophip, gpu, stream)}
    nbytes = 1 << 30
    a_, b_ = gpu.malloc(nbytes), gpu.malloc(nbytes)
    gpu.memset(a_, 0x3C)
    gpu.memset(b_, 0)
    probe = lambda kind, blocks, iters=0, seed=1, dst=None: bench_probe(kind, dst or b_, a_, nbytes, iters, seed, blocks, stream)
    for kind, moved in (("read", nbytes), ("read_nt", nbytes), ("write", nbytes), ("copy", 2 * nbytes)):
        best = None
        for blocks in (1024, 2048, 4096, 8192, 16384, 65536):
            us = time_launches(gpu, stream, lambda: probe(kind, blocks), 10, warm=2)
            if best is None or us < best[0]:
                best = (us, blocks)
        us, blocks = best
        out[kind] = {"bytes": moved, "us": round(us, 2), "GBps": round(moved / us / 1e3, 1), "blocks": blocks,
                     "hbm_frac": round(moved / (us * 1e-6) / HBM_PEAK, 4)}
        log("  probe %-8s 1 GiB: %8.1f us, %7.1f GB/s (%.1f%% of 8 TB/s), %d workgroups" % (
            kind, us, moved / us / 1e3, 100 * moved / (us * 1e-6) / HBM_PEAK, blocks))
    # bare MFMA loop: 2048 workgroups of 4 waves, 512 trips of 128 MFMA 32x32x16 each
    blocks, iters = 2048, 512
    flop = blocks * 4 * iters * 128 * 32768
    scratch = gpu.malloc(blocks * 1024)
    for name, seed in (("mfma_random", 12345), ("mfma_zero", 0)):
        run = lambda: probe("mfma", blocks, iters, seed, dst=scratch)
        time.sleep(0.5)
        idle_us = time_launches(gpu, stream, run, 5, warm=0)
        n, t0, watts = 0, time.perf_counter(), []
        while time.perf_counter() - t0 < 2.0:   # two seconds of load: clocks and power settle
            for _ in range(4):
                run()
            stream.synchronize()
            n += 4
            w = read_power()
            if w:
                watts.append(w)
        us = time_launches(gpu, stream, run, 20, warm=0)
        out[name] = {"flop": flop, "us_from_idle": round(idle_us, 1), "TFLOPs_from_idle": round(flop / idle_us / 1e6, 1),
                     "us_steady": round(us, 1), "TFLOPs_steady": round(flop / us / 1e6, 1),
                     "mfma_frac_steady": round(flop / (us * 1e-6) / MFMA_F16_PEAK, 4),
                     "watts": round(sum(watts[len(watts) // 2:]) / max(1, len(watts[len(watts) // 2:])), 0) if watts else None}
        log("  probe %-12s %7.1f TFLOP/s from idle clocks, %7.1f TFLOP/s steady (%.1f%% of 2.5 PFLOP/s)%s" % (
            name, flop / idle_us / 1e6, flop / us / 1e6, 100 * flop / (us * 1e-6) / MFMA_F16_PEAK,
            ", %.0f W" % out[name]["watts"] if out[name]["watts"] else ""))
    a_.free(); b_.free(); scratch.free()
    return out


def granule_classes(ophip, gpu, stream):
    """A walk down one 128-column strip of an N-contiguous f16 weight reads one 256-byte granule per row.  Probe
    "granules": one workgroup per strip, each noting its own time, on the decode layer's weight shapes and on row lengths
    of other residues: per class of a strip's first granule (address bits 8..10 of its first byte), the mean time of the
    strips of that class.  The classes that come out slower are the ones mat_mul's planner cuts into more K ranges."""
    out = []
    # (name, rows K, columns N): rows of 172 / 96 / 32 granules (residues 4, 0, 0 modulo 8), then 174 (residue 6), 173 (odd)
    shapes = [("gate_up", 4096, 22016), ("qkv", 4096, 12288), ("o_proj", 4096, 4096), ("rows of 174 granules", 4096, 22272),
              ("rows of 173 granules", 4096, 22144)]
    for name, k, n in shapes:
        nbytes = k * n * 2
        ncopy = max(2, (600 << 20) // nbytes + 1)
        copies = [gpu.malloc(nbytes) for _ in range(ncopy)]
        for c in copies:
            gpu.memset(c, 0x3C)
        strips = (n + 127) // 128
        ticks = gpu.malloc(4 * (strips + 1))
        per_class = np.zeros(8)
        count = np.zeros(8)
        total = []
        reps = 20
        for it in range(reps + 2):
            w = copies[it % ncopy]
            bench_probe("granules", ticks, w, nbytes, n, k, 1, stream)
            t = gpu.to_host(ticks, np.uint32, strips, stream=stream).astype(np.float64) / 100.0  # 100 MHz ticks -> us
            if it < 2:
                continue
            cls = ((w.ptr >> 8) + np.arange(strips)) & 7
            for c in range(8):
                per_class[c] += t[cls == c].sum()
                count[c] += (cls == c).sum()
            total.append(t.max())
        row = {"shape": name, "k": k, "n": n, "strips": strips, "granules_per_row": n * 2 // 256,
               "us_by_class_of_first_granule": [round(float(per_class[c] / max(count[c], 1)), 2) for c in range(8)],
               "slowest_strip_us": round(float(np.mean(total)), 2)}
        out.append(row)
        log("  granules %-22s %d strips, rows of %d granules: us by class %s, slowest strip %.2f" % (
            name, strips, row["granules_per_row"], " ".join("%d:%.1f" % (c, v) for c, v in enumerate(row["us_by_class_of_first_granule"])),
            row["slowest_strip_us"]))
        for c in copies:
            c.free()
        ticks.free()
    return out


def gemm_floors(ophip, gpu, stream, rng, reps):
    """The six GEMMs of the decode layer on cold operands (copies of the weight or cache operand rotate through more than
    600 MB), each beside what a bare read of the same bytes takes: the library's read probe (non-temporal loads) over
    the same cold copies, with as many workgroups as the GEMM launches and with the best of a few grids, and beside an
    empty launch.  What separates a GEMM from its bare read is MFMA work, the activation loads and, with split K, the
    exchange of partial sums."""
    import copy
    layer = Layer(ophip, gpu, rng)
    mm = layer.ops["mm"]
    out = []
    one = gpu.malloc(4096)
    probe = lambda kind, dst, src, nbytes, blocks: bench_probe(kind, dst, src if src else dst, nbytes, 0, 1, blocks, stream)
    empty_us = time_launches(gpu, stream, lambda: probe("write", one, None, 16, 1), 200, warm=10)
    log("  empty launch (16 bytes written by one workgroup), back to back: %.2f us" % empty_us)
    work = layer_work()
    operand = {"qkv": ("w_qkv", D * 3 * D * 2), "qk_t": ("k_cache", NH * KV * DH * 2), "pv": ("v_cache", NH * KV * DH * 2),
               "o_proj": ("w_o", D * D * 2), "gate_up": ("w_gu", D * 2 * DI * 2), "down": ("w_d", DI * D * 2)}
    for name in ("qkv", "qk_t", "pv", "o_proj", "gate_up", "down"):
        buf_name, nbytes = operand[name]
        ncopy = max(2, (600 << 20) // nbytes + 1)
        copies = [gpu.malloc(nbytes) for _ in range(ncopy)]
        for cbuf in copies:
            ophip._check(ophip.lib().ophip_memcpy_d2d(gpu.handle, ctypes.c_void_p(cbuf.ptr), ctypes.c_void_p(layer.d[buf_name].ptr),
                                                      ctypes.c_size_t(nbytes), stream.handle))
        stream.synchronize()
        kind, base = layer.args[name]
        variants = []
        for cbuf in copies:
            a = copy.copy(base)
            a.b_base = cbuf
            variants.append(a)
        what = mm.describe(base)
        split = int(what.split("split_k=")[1]) if "split_k=" in what else 1
        m, n = (NT, {"qkv": 3 * D, "o_proj": D, "gate_up": 2 * DI, "down": D}.get(name, KV if name == "qk_t" else DH))
        batch = NH if name in ("qk_t", "pv") else 1
        wgs = (n + 127) // 128 * split * batch
        it = [0]

        def run_gemm():
            mm.launch(variants[it[0] % ncopy], layer.d["ws"], stream)
            it[0] += 1

        def run_probe(blocks):
            def f():
                probe("read_nt", one, copies[it[0] % ncopy], nbytes, blocks)
                it[0] += 1
            return f
        gemm_us = time_launches(gpu, stream, run_gemm, reps, warm=ncopy)
        same_us = time_launches(gpu, stream, run_probe(wgs), reps, warm=ncopy)
        best = min((time_launches(gpu, stream, run_probe(b), reps, warm=4), b) for b in (256, 512, 1024, 2048))
        rec = {"op": name, "kernel": what, "workgroups": wgs, "operand_bytes": nbytes, "algorithmic_bytes": work[name][0],
               "gemm_us": round(gemm_us, 2), "bare_read_same_grid_us": round(same_us, 2),
               "bare_read_best_us": round(best[0], 2), "bare_read_best_workgroups": best[1], "copies": ncopy}
        out.append(rec)
        log("  %-8s %-34s %4d workgroups: %6.2f us | bare read of the operand (%5.1f MB), same grid %6.2f us, best %6.2f us (%d workgroups)" % (
            name, what, wgs, gemm_us, nbytes / 1e6, same_us, best[0], best[1]))
        for cbuf in copies:
            cbuf.free()
    # The weight-streaming kernel without a K split, one workgroup per 128-column strip, on 64 .. 288 strips (cold
    # weights): what one CU pulls, and how the launch's rate follows the number of CUs that hold a workgroup.
    L, F16 = ophip.TensorLayout, ophip.dt.F16
    prev = os.environ.get("OPHIP_GEMM_SPLITK")
    os.environ["OPHIP_GEMM_SPLITK"] = "1"
    unsplit = ophip.MatMul(gpu)
    if prev is None:
        del os.environ["OPHIP_GEMM_SPLITK"]
    else:
        os.environ["OPHIP_GEMM_SPLITK"] = prev
    strips_out = []
    x = layer.d["xn"]
    for strips in (64, 128, 172, 192, 224, 250, 256, 288):
        n = 128 * strips
        nbytes = D * n * 2
        ncopy = max(2, (600 << 20) // nbytes + 1)
        copies = [gpu.malloc(nbytes) for _ in range(ncopy)]
        src_bytes = D * 2 * DI * 2
        for cbuf in copies:  # any finite f16 will do: the layer's gate/up weight, again and again
            for off in range(0, nbytes, src_bytes):
                ophip._check(ophip.lib().ophip_memcpy_d2d(gpu.handle, ctypes.c_void_p(cbuf.ptr + off), ctypes.c_void_p(layer.d["w_gu"].ptr),
                                                          ctypes.c_size_t(min(nbytes - off, src_bytes)), stream.handle))
        dst = gpu.malloc(NT * n * 2)
        variants = [ophip.MatMulArgs(L.new_contiguous(F16, [NT, n]), dst, 0.0, L.new_contiguous(F16, [NT, D]), x,
                                     L.new_contiguous(F16, [D, n]), cbuf, 1.0) for cbuf in copies]
        what = unsplit.describe(variants[0])
        it = [0]

        def run_strips():
            unsplit.launch(variants[it[0] % ncopy], layer.d["ws"], stream)
            it[0] += 1
        us = time_launches(gpu, stream, run_strips, reps, warm=ncopy)
        busy = min(strips, 256)
        rec = {"strips": strips, "kernel": what, "weight_bytes": nbytes, "us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
               "GBps_per_busy_cu": round(nbytes / us / 1e3 / busy, 2)}
        strips_out.append(rec)
        log("  %3d strips (%s): %6.2f us, %6.1f GB/s, %5.2f GB/s per CU that holds a workgroup" % (
            strips, what, us, rec["GBps"], rec["GBps_per_busy_cu"]))
        for cbuf in copies:
            cbuf.free()
        dst.free()
    # The streaming kernel's access pattern and nothing else (probe "strips": 128-column strips x equal K ranges, four waves
    # per workgroup on every fourth group of 32 rows, three groups in flight per wave; no MFMA, no activations, no
    # epilogue, no exchange of partial sums) on the four weight shapes, at 1 .. 16 K ranges.
    pattern = []
    for name, n, k in (("qkv", 3 * D, D), ("o_proj", D, D), ("gate_up", 2 * DI, D), ("down", D, DI)):
        nbytes = n * k * 2
        ncopy = max(2, (700 << 20) // nbytes + 1)
        copies = [gpu.malloc(nbytes) for _ in range(ncopy)]
        for cbuf in copies:
            gpu.memset(cbuf, 0x3C)
        row = {"op": name, "bytes": nbytes, "us_by_k_ranges": {}}
        for ranges in (1, 2, 4, 8, 16):
            if k % (32 * ranges):
                continue
            it = [0]

            def run_pattern():
                bench_probe("strips", one, copies[it[0] % ncopy], nbytes, n, k, ranges, stream)
                it[0] += 1
            row["us_by_k_ranges"][ranges] = round(time_launches(gpu, stream, run_pattern, reps, warm=ncopy), 2)
        pattern.append(row)
        log("  pattern %-8s %6.1f MB: %s" % (name, nbytes / 1e6, "  ".join("%d ranges (%d workgroups) %6.2f us" % (
            r, (n + 127) // 128 * r, us) for r, us in row["us_by_k_ranges"].items())))
        for cbuf in copies:
            cbuf.free()
    # What one CU pulls with nothing but loads: the read probes on 1 MB per workgroup (as a strip above), 64 / 128 / 256
    # workgroups, 4 or 16 vectors in flight per thread, plain or non-temporal loads.
    per_cu = []
    for blocks in (64, 128, 256):
        nbytes = blocks << 20
        npool = (768 << 20) // nbytes + 1  # more than three times the 256 MiB cache in rotation
        pool = [gpu.malloc(nbytes) for _ in range(npool)]
        for pbuf in pool:
            gpu.memset(pbuf, 0x3C)
        for kind in ("read", "read_nt", "read16", "read_nt16"):
            it = [0]

            def run_probe_kind():
                probe(kind, one, pool[it[0] % npool], nbytes, blocks)
                it[0] += 1
            us = time_launches(gpu, stream, run_probe_kind, reps, warm=npool)
            per_cu.append({"kind": kind, "workgroups": blocks, "bytes": nbytes, "us": round(us, 2),
                           "GBps_per_workgroup": round(nbytes / us / 1e3 / blocks, 2)})
            log("  probe %-9s %3d workgroups x 1 MB: %6.2f us, %5.2f GB/s per workgroup" % (kind, blocks, us, nbytes / us / 1e3 / blocks))
        for pbuf in pool:
            pbuf.free()
    return {"empty_launch_us": round(empty_us, 2), "gemms": out, "unsplit_strips": strips_out, "access_pattern": pattern,
            "probe_per_workgroup": per_cu}


def adder(out, ceiling=None):
    """Returns add(name, shape, bytes, us, flops, note): appends one per-operator record to `out` and logs it.
    `ceiling`: the copy_ceiling record; with it every record carries `ceiling_frac`, its rate against what a plain
    copy reaches on this machine (the practical ceiling of a stream), beside `hbm_frac` (against the 8 TB/s nameplate)."""
    def add(name, shape, nbytes, us, flops=0, note=None):
        rec = {"op": name, "shape": shape, "us": round(us, 3), "bytes": nbytes,
               "GBps": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / (us * 1e-6) / HBM_PEAK, 4)}
        if ceiling:
            rec["ceiling_frac"] = round(nbytes / us / 1e3 / ceiling["GBps"], 4)
        if flops:
            rec["TFLOPs"] = round(flops / us / 1e6, 2)
            rec["mfma_frac"] = round(flops / (us * 1e-6) / MFMA_F16_PEAK, 4)
        if nbytes < (256 << 20):
            rec["cache_resident"] = True
        if note:
            rec["note"] = note
        out.append(rec)
        log("  %-28s %-22s %10.2f us %9.1f GB/s  %5.1f%% HBM%s" % (
            name, shape, us, rec["GBps"], 100 * rec["hbm_frac"],
            ("  %.1f TFLOP/s %.1f%% MFMA" % (rec["TFLOPs"], 100 * rec["mfma_frac"])) if flops else ""))

    return add


def mat_mul_lines(o, gpu, stream, rng, add, launches=0):
    """Compute-bound mat_mul: square shapes in both layouts of B, the prefill GEMMs of a Llama-7B layer
    at 512 tokens, and two shapes that are no multiples of the tile (509 tokens; 4000 x 4000).
    `launches` > 0: that many plain launches per shape and nothing else (counter runs)."""
    from ophip import TensorLayout as L, dt
    c = lambda *s: L.new_contiguous(dt.F16, list(s))
    mm = o.MatMul(gpu)
    shapes = [(4096, 4096, 4096, False), (4096, 4096, 4096, True), (8192, 8192, 8192, False), (8192, 8192, 8192, True),
              (512, 12288, 4096, False), (512, 22016, 4096, False), (512, 4096, 11008, False),
              (509, 12288, 4096, False), (4000, 4000, 4096, False), (8192, 8192, 8192, True, dt.BF16)]
    for m, n, k, b_nk, *et in shapes:
        et = et[0] if et else dt.F16
        # (bf16: the top halves of f32 normals, which are bf16 normals of the same spread)
        mk = normal_f16 if et == dt.F16 else lambda r, sh, std: np.ascontiguousarray(
            (r.standard_normal(sh, dtype=np.float32) * np.float32(std)).view(np.uint32) >> 16).astype(np.uint16)
        c = lambda *s, et=et: L.new_contiguous(et, list(s))
        A_, B_, C_ = gpu.from_host(mk(rng, (m, k), 1.0)), gpu.from_host(mk(rng, (k, n), 0.02)), \
            gpu.malloc(m * n * 2)
        bl = L(et, [k, n], [2, k * 2]) if b_nk else c(k, n)  # the same bytes read as B[N, K] transposed
        a = o.MatMulArgs(c(m, n), C_, 0.0, c(m, k), A_, bl, B_, 1.0)
        ws = gpu.malloc(max(mm.scheme(a, 1 << 32), 1))
        shape = "%dx%dx%d%s%s" % (m, n, k, ", B stored [N,K]" if b_nk else "", ", bf16" if et != dt.F16 else "")
        nbytes, flops = 2 * (m * k + k * n + m * n), 2 * m * n * k
        if launches:
            us = time_launches(gpu, stream, lambda: mm.launch(a, ws, stream), launches, warm=1)
            add("mat_mul", shape, nbytes, us, flops=flops, note="%d launches, %s" % (launches, mm.describe(a)))
        else:
            if m == n == k:
                us = time_launches(gpu, stream, lambda: mm.launch(a, ws, stream), 10, warm=2)
                add("mat_mul", shape, nbytes, us, flops=flops, note="10 launches from idle clocks")
            us = time_sustained(gpu, stream, lambda: mm.launch(a, ws, stream))
            add("mat_mul", shape, nbytes, us, flops=flops, note="steady state (0.3 s warm-up), " + mm.describe(a))
        A_.free(); B_.free(); C_.free(); ws.free()


def attention_lines(o, gpu, stream, rng, add, reps, full=False):
    """attention at prefill shapes (32 heads, dh 128): one pass with the scores kept on the chip where the crate's
    composite writes and reads the [nh, seq, att] score matrix four times.  flops = 4 nh seq att dh, half of it under a
    causal mask (the part of the score matrix the mask keeps); bytes = q, k, v, o once.  `full`: the unmasked shapes too."""
    L = o.TensorLayout
    at = o.Attention(gpu)
    cases = [(512, True, False), (2048, True, False), (2048, True, True), (4096, True, False)]
    for seq, causal, bf in cases + ([(2048, False, False), (4096, False, False)] if full else []):
        c = lambda *s: L.new_contiguous(o.dt.BF16 if bf else o.dt.F16, list(s))
        # (bf16: the top halves of f32 normals, which are bf16 normals of the same spread)
        mk = (lambda: (rng.standard_normal((NH, seq, DH), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)) if bf else \
            (lambda: normal_f16(rng, (NH, seq, DH), 1.0))
        q, k, v = (gpu.from_host(mk()) for _ in range(3))
        od = gpu.malloc(NH * seq * DH * 2)
        a = o.AttentionArgs(c(NH, seq, DH), q, c(NH, seq, DH), k, c(NH, seq, DH), v, c(NH, seq, DH), od,
                            o.AttnMask.CAUSAL if causal else o.AttnMask.NONE)
        us = time_launches(gpu, stream, lambda: at.launch(a, None, stream), reps)
        add("attention", "nh32 seq%d att%d dh128 %s%s" % (seq, seq, "causal" if causal else "no mask", " bf16" if bf else ""),
            4 * NH * seq * DH * 2, us, flops=(2 if causal else 4) * NH * seq * seq * DH,
            note="one pass (attention_prefill.hip)" + ("; flops count the unmasked half of the scores" if causal else ""))
        for m_ in (q, k, v, od):
            m_.free()


def standalone_ops(ophip, gpu, stream, rng, reps, ceiling=None):
    """Every operator at its benchmark shape plus a scaled shape that does not fit the Infinity Cache."""
    o, L, F16 = ophip, ophip.TensorLayout, ophip.dt.F16
    c = lambda *s: L.new_contiguous(F16, list(s))
    out = []

    add = adder(out, ceiling)

    # rms_norm: [64, 4096] and [65536, 4096]
    rms = o.RmsNorm(gpu)
    for n in (64, 65536):
        x = gpu.malloc(n * D * 2)
        y = gpu.malloc(n * D * 2)
        gpu.memset(x, 0x3C)
        w = gpu.from_host(np.ones(D, f16))
        a = o.RmsNormArgs(c(n, D), y, c(n, D), x, c(D), w, 1e-5)
        rms.scheme(a, 0)
        us = time_launches(gpu, stream, lambda: rms.launch(a, None, stream), reps)
        add("rms_norm", "[%d,%d]" % (n, D), 2 * n * D * 2 + D * 2, us)
        x.free(); y.free()
    # rope: [512, 32, 128] and [32768, 32, 128]
    rope = o.Rope(gpu)
    empty = L(F16, [0, DH], [2 * DH, 2])
    for nt in (512, 65536):
        t = gpu.malloc(nt * NH * DH * 2)
        gpu.memset(t, 0x3C)
        pos = gpu.from_host((np.arange(nt) % 4096).astype(np.uint32))
        a = o.RopeArgs(c(nt, NH, DH), t, L(o.dt.U32, [nt], [4]), pos, empty, None, empty, None, 1e4)
        us = time_launches(gpu, stream, lambda: rope.launch(a, None, stream), reps)
        add("rope", "[%d,%d,%d]" % (nt, NH, DH), 2 * nt * NH * DH * 2 + nt * 4, us)
        t.free()
    # rearrange: [32, 512, 128] -> [512, 32, 128] and a 64x larger one
    rea = o.Rearrange(gpu)
    for s0, s1 in ((32, 512), (32, 65536)):
        src = gpu.malloc(s0 * s1 * DH * 2)
        dst = gpu.malloc(s0 * s1 * DH * 2)
        gpu.memset(src, 0x3C)
        a = o.RearrangeArgs(L(F16, [s0, s1, DH], [DH * 2, s0 * DH * 2, 2]), dst, c(s0, s1, DH), src)
        us = time_launches(gpu, stream, lambda: rea.launch(a, None, stream), reps)
        add("rearrange", "[%d,%d,%d]->T" % (s0, s1, DH), 2 * s0 * s1 * DH * 2, us)
        src.free(); dst.free()
    # fused softmax: prefill [32, 512, 512], decode [32, 1, 2048], scaled [32, 8192, 2048] (no mask to keep all columns)
    sm = o.FusedSoftmax(gpu)
    for nh, seq, al, mask in ((32, 512, 512, 1), (32, 1, 2048, 1), (32, 8192, 2048, 0)):
        att_host = None
        att = gpu.malloc(nh * seq * al * 2)
        gpu.memset(att, 0x3C)
        a = o.FusedSoftmaxArgs(mask, c(nh, seq, al), att)
        us = time_launches(gpu, stream, lambda: sm.launch(a, None, stream), reps)
        add("fused_softmax", "[%d,%d,%d]%s" % (nh, seq, al, "" if mask else " nomask"), 2 * nh * seq * al * 2, us)
        att.free()
    # swiglu: [16, 11008] halves and [8192, 11008]
    sw = o.Swiglu(gpu)
    for n in (16, 16384):
        gu = gpu.malloc(n * 2 * DI * 2)
        gpu.memset(gu, 0x3C)
        half = L(F16, [n, DI], [2 * DI * 2, 2])
        a = o.SwigluArgs(half, gu.ptr, half, gu.ptr + DI * 2)
        us = time_launches(gpu, stream, lambda: sw.launch(a, None, stream), reps)
        add("swiglu", "[%d,%d]" % (n, DI), 3 * n * DI * 2, us)
        gu.free()
    # random_sample: 16 rows x [32000], one launch per row as the API prescribes; then a vocabulary of today's
    # models, which a workgroup cannot keep in its registers
    rs = o.RandomSample(gpu)
    for vocab in (32000, 128256):
        logits = gpu.from_host(normal_f16(rng, (16, vocab), np.sqrt(3.0)))
        kv = gpu.malloc(16 * 8)
        shape = "16 x [%d]" % vocab
        for mode, cfg, seed in (("argmax", o.SampleArgs.argmax(), 0.0), ("top-k 50 / top-p 0.9", o.SampleArgs(0.8, 0.9, 50), 0.37)):
            arg_rows = []
            for r in range(16):
                a = o.RandomSampleArgs.layout(F16, vocab)
                a.kv_pair_base, a.logits_base, a.config, a.seed = kv.ptr + 8 * r, logits.ptr + r * vocab * 2, cfg, seed
                arg_rows.append(a)

            def run16():
                for a in arg_rows:
                    rs.launch(a, None, stream)
            us = time_launches(gpu, stream, run16, max(reps // 4, 5))
            add("random_sample " + mode, shape, 16 * (vocab * 2 + 8), us, note="16 launches")
            b = arg_rows[0]
            us = time_launches(gpu, stream, lambda: rs.launch_batch(b, 16, vocab * 2, None, None, stream), reps)
            add("random_sample " + mode, shape, 16 * (vocab * 2 + 8), us, note="1 batched launch (extension)")
        logits.free(); kv.free()
    # the remaining single-device operators, small and out-of-cache
    ln = o.LayerNorm(gpu)
    for n in (64, 65536):
        x, y = gpu.malloc(n * D * 2), gpu.malloc(n * D * 2)
        gpu.memset(x, 0x3C)
        sc, bi = gpu.from_host(np.ones(D, np.float32)), gpu.from_host(np.zeros(D, np.float32))
        a = o.LayerNormArgs(c(n, D), y, c(n, D), x, L.new_contiguous(o.dt.F32, [D]), sc,
                            L.new_contiguous(o.dt.F32, [D]), bi, 1e-5)
        us = time_launches(gpu, stream, lambda: ln.launch(a, None, stream), reps)
        add("layer_norm", "[%d,%d]" % (n, D), 2 * n * D * 2 + 2 * D * 4, us)
        x.free(); y.free()
    ge = o.Gelu(gpu)
    for n in (16, 16384):
        t = gpu.malloc(n * DI * 2)
        gpu.memset(t, 0x3C)
        a = o.GeluArgs(c(n, DI), t)
        us = time_launches(gpu, stream, lambda: ge.launch(a, None, stream), reps)
        add("gelu", "[%d,%d]" % (n, DI), 2 * n * DI * 2, us)
        t.free()
    ad = o.Add(gpu)
    for n in (16, 65536):
        x, y, z = gpu.malloc(n * D * 2), gpu.malloc(n * D * 2), gpu.malloc(n * D * 2)
        gpu.memset(x, 0x3C); gpu.memset(y, 0x3C)
        a = o.AddArgs(c(n, D), z, c(n, D), x, c(n, D), y)
        us = time_launches(gpu, stream, lambda: ad.launch(a, None, stream), reps)
        add("add", "[%d,%d]" % (n, D), 3 * n * D * 2, us)
        x.free(); y.free(); z.free()
    ar = o.AddRows(gpu)
    for m in (16, 32768):   # position-embedding style: dst[1, m, 4096] += table[idx[m], :], table 32000 rows
        dst, table = gpu.malloc(m * D * 2), gpu.malloc(32000 * D * 2)
        gpu.memset(dst, 0x3C); gpu.memset(table, 0x3C)
        idx = gpu.from_host(rng.integers(0, 32000, (1, m)).astype(np.uint32))
        a = o.AddRowsArgs(c(1, m, D), dst, c(32000, D), table, L.new_contiguous(o.dt.U32, [1, m]), idx)
        us = time_launches(gpu, stream, lambda: ar.launch(a, None, stream), reps)
        add("add_rows", "[1,%d,%d] from 32000 rows" % (m, D), 3 * m * D * 2 + m * 4, us)
        dst.free(); table.free()
    # attention_kv_cached, the crate's composite, at the decode-layer shape: two cache appends, a staging copy
    # of the strided q, QK^T, causal softmax, PV and the copy into o - seven launches
    nt, pos = NT, KV - NT
    qkv = gpu.from_host(normal_f16(rng, (nt, 3 * D), 1.0))
    kc, vc = gpu.from_host(normal_f16(rng, (NH, KV, DH), 1.0)), gpu.from_host(normal_f16(rng, (NH, KV, DH), 1.0))
    obuf = gpu.malloc(nt * D * 2)
    head_major = lambda row_bytes: L(F16, [NH, nt, DH], [DH * 2, row_bytes, 2])
    akv = o.AttnKVCached(gpu)
    a = o.AttnKVCachedArgs(head_major(3 * D * 2), qkv.ptr, head_major(3 * D * 2), qkv.ptr + D * 2,
                           head_major(3 * D * 2), qkv.ptr + 2 * D * 2, head_major(D * 2), obuf,
                           c(NH, KV, DH), kc, c(NH, KV, DH), vc, o.AttnMask.CAUSAL, pos)
    ws = gpu.malloc(max(akv.scheme(a, 1 << 30), 1))
    us = time_launches(gpu, stream, lambda: akv.launch(a, ws, stream), reps)
    add("attention_kv_cached", "nh32 seq16 pos2032 dh128", 2 * NH * KV * DH * 2 + 8 * nt * D * 2, us,
        note="one pass over the caches + the merge of its chunks (the crate's composite: 7 launches); bytes = both caches "
             "read once + q, k, v, o and the appended rows; the same two caches every launch (34.6 MB: they stay in the 256 MiB cache)")
    # the same with ten sets of caches in rotation (346 MB), as the layers of a model present them: every launch reads HBM
    sets = [(kc, vc)] + [(gpu.malloc(NH * KV * DH * 2), gpu.malloc(NH * KV * DH * 2)) for _ in range(9)]
    for kb_, vb_ in sets[1:]:
        for dst_, src_ in ((kb_, kc), (vb_, vc)):
            ophip._check(ophip.lib().ophip_memcpy_d2d(gpu.handle, ctypes.c_void_p(dst_.ptr), ctypes.c_void_p(src_.ptr),
                                                      ctypes.c_size_t(NH * KV * DH * 2), stream.handle))
    stream.synchronize()
    rot = [o.AttnKVCachedArgs(head_major(3 * D * 2), qkv.ptr, head_major(3 * D * 2), qkv.ptr + D * 2,
                              head_major(3 * D * 2), qkv.ptr + 2 * D * 2, head_major(D * 2), obuf,
                              c(NH, KV, DH), kb_, c(NH, KV, DH), vb_, o.AttnMask.CAUSAL, pos) for kb_, vb_ in sets]
    turn = [0]

    def launch_rotating():
        akv.launch(rot[turn[0] % len(rot)], ws, stream)
        turn[0] += 1
    us = time_launches(gpu, stream, launch_rotating, max(reps, 2 * len(rot)), warm=len(rot))
    add("attention_kv_cached", "nh32 seq16 pos2032 dh128, ten cache sets in rotation", 2 * NH * KV * DH * 2 + 8 * nt * D * 2, us,
        note="as above on caches that come from HBM")
    # attention itself at the same shape (a caller that keeps its own cache): q from the QKV rows against the full caches
    att_op = o.Attention(gpu)
    rot_at = [o.AttentionArgs(head_major(3 * D * 2), qkv.ptr, c(NH, KV, DH), kb_, c(NH, KV, DH), vb_, head_major(D * 2), obuf,
                              o.AttnMask.CAUSAL) for kb_, vb_ in sets]
    ws_at = gpu.malloc(max(att_op.scheme(rot_at[0], 1 << 30), 1))

    def launch_rotating_attention():
        att_op.launch(rot_at[turn[0] % len(rot_at)], ws_at, stream)
        turn[0] += 1
    us = time_launches(gpu, stream, launch_rotating_attention, max(reps, 2 * len(rot_at)), warm=len(rot_at))
    add("attention", "nh32 seq16 att2048 dh128 causal (decode shape), ten cache sets in rotation", 2 * NH * KV * DH * 2 + 2 * nt * D * 2, us,
        flops=4 * NH * nt * KV * DH, note="the decode kernel of attention_kv_cached with nothing to append (the crate's composite: 5 launches)")
    for kb_, vb_ in sets[1:]:
        kb_.free(); vb_.free()
    attention_lines(o, gpu, stream, rng, add, max(5, reps // 2))
    # the dominant decode GEMM (gate/up) on its own, weights stored [K, N] and [N, K]: two copies of the
    # weights alternate so that no launch finds them in the Infinity Cache
    mm = o.MatMul(gpu)
    xa = gpu.from_host(normal_f16(rng, (nt, D), 1.0))
    ya = gpu.malloc(nt * 2 * DI * 2)
    w2 = [gpu.from_host(normal_f16(rng, (D, 2 * DI), 0.02)) for _ in range(2)]
    wsb = gpu.malloc(64 << 20)
    # (the third line: the same buffers read as bf16 numbers -- every f16 pattern here is a finite bf16 -- by the bf16
    # build of the same kernel)
    for b_nk, et in ((False, F16), (True, F16), (False, o.dt.BF16)):
        ce = lambda *s_: L.new_contiguous(et, list(s_))
        bl = L(et, [D, 2 * DI], [2, D * 2]) if b_nk else ce(D, 2 * DI)
        pair = [o.MatMulArgs(ce(nt, 2 * DI), ya, 0.0, ce(nt, D), xa, bl, w, 1.0) for w in w2]
        flip = [0]

        def run():
            flip[0] ^= 1
            mm.launch(pair[flip[0]], wsb, stream)
        us = time_launches(gpu, stream, run, reps)
        add("mat_mul", "%dx%dx%d%s%s" % (nt, 2 * DI, D, ", B stored [N,K]" if b_nk else "", ", bf16" if et != F16 else ""),
            2 * (nt * D + D * 2 * DI + nt * 2 * DI), us, flops=2 * nt * D * 2 * DI, note="cold weights, " + mm.describe(pair[0]))
    for w in w2:
        w.free()
    wsb.free(); xa.free(); ya.free()
    mat_mul_lines(o, gpu, stream, rng, add)
    return out


def cpu_per_op(oracle, threads):
    """The CPU oracle on the benchmark configurations of the single operators (rms_norm, rope and rearrange,
    causal softmax, random_sample), best of three runs each; keys are (operator, shape) as in `per_op`."""
    rng = np.random.default_rng(0)
    oracle.set_threads(threads)
    out = {}

    def best(fn):
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return min(ts) * 1e6

    try:
        x, w = normal_f16(rng, (64, D), 1.0), (rng.random(D, dtype=np.float32) + 0.5).astype(f16)
        y = np.zeros_like(x)
        out[("rms_norm", "[64,%d]" % D)] = best(lambda: oracle.rms_norm(y, x, w, 1e-5))
        t, pos = normal_f16(rng, (512, NH, DH), 1.0), np.arange(512, dtype=np.uint32)
        out[("rope", "[512,%d,%d]" % (NH, DH))] = best(lambda: oracle.rope(t, pos, 1e4))
        src = normal_f16(rng, (32, 512, DH), 1.0)
        dst = np.zeros((512, 32, DH), f16)
        out[("rearrange", "[32,512,%d]->T" % DH)] = best(lambda: oracle.rearrange(dst.transpose(1, 0, 2), src))
        for seq, al in ((512, 512), (1, 2048)):
            att = normal_f16(rng, (32, seq, al), 2.0)
            out[("fused_softmax", "[32,%d,%d]" % (seq, al))] = best(lambda: oracle.fused_softmax(att, True))
        gu = normal_f16(rng, (16, 2 * DI), 1.0)
        out[("swiglu", "[16,%d]" % DI)] = best(lambda: oracle.swiglu(gu[:, :DI], gu[:, DI:]))
        logits = normal_f16(rng, (16, 32000), np.sqrt(3.0))
        out[("random_sample argmax", "16 x [32000]")] = best(lambda: [oracle.argmax(r) for r in logits])
        out[("random_sample top-k 50 / top-p 0.9", "16 x [32000]")] = best(
            lambda: [oracle.random_sample(r, 0.8, 0.9, 50, 0.37) for r in logits])
    finally:
        oracle.set_threads(1)
    return out


def cpu_layer_step(oracle, h, threads, attention_op=False):
    """The same operations through the CPU oracle (threads on the axes the reference hands to rayon).  attention_op:
    the crate's attention_kv_cached composite (on copies of the caches) instead of the three scripted launches."""
    oracle.set_threads(threads)
    xn = oracle.rms_norm(np.empty_like(h["x"]), h["x"], h["w_norm1"], 1e-5)
    qkv = oracle.mat_mul(np.zeros((NT, 3 * D), f16), 0.0, xn, h["w_qkv"], 1.0)
    oracle.set_threads(1)  # rope is single-threaded in the reference
    oracle.rope(qkv[:, :D].reshape(NT, NH, DH), h["pos"], 1e4)
    oracle.rope(qkv[:, D:2 * D].reshape(NT, NH, DH), h["pos"], 1e4)
    oracle.set_threads(threads)
    q = qkv[:, :D].reshape(NT, NH, DH).transpose(1, 0, 2)
    o = np.zeros((NT, D), f16)
    if attention_op:
        k_new = qkv[:, D:2 * D].reshape(NT, NH, DH).transpose(1, 0, 2)
        v_new = qkv[:, 2 * D:].reshape(NT, NH, DH).transpose(1, 0, 2)
        oracle.attention_kv_cached(q, k_new, v_new, o.reshape(NT, NH, DH).transpose(1, 0, 2), h["k_cache"].copy(),
                                   h["v_cache"].copy(), KV - NT, causal=True)
    else:
        att = oracle.mat_mul(np.zeros((NH, NT, KV), f16), 0.0, q, h["k_cache"].transpose(0, 2, 1), float(1 / np.sqrt(DH)))
        oracle.fused_softmax(att, causal=True)
        oracle.mat_mul(o.reshape(NT, NH, DH).transpose(1, 0, 2), 0.0, att, h["v_cache"], 1.0)
    y = oracle.mat_mul(np.zeros((NT, D), f16), 0.0, o, h["w_o"], 1.0)
    yn = oracle.rms_norm(np.empty_like(y), y, h["w_norm2"], 1e-5)
    gu = oracle.mat_mul(np.zeros((NT, 2 * DI), f16), 0.0, yn, h["w_gu"], 1.0)
    oracle.set_threads(1)  # swiglu is single-threaded in the reference
    oracle.swiglu(gu[:, :DI], gu[:, DI:])
    oracle.set_threads(threads)
    out = oracle.mat_mul(np.zeros((NT, D), f16), 0.0, gu[:, :DI], h["w_d"], 1.0)
    oracle.set_threads(1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--reps", type=int, default=100, help="launches per standalone-operator timing")
    ap.add_argument("--no-per-op", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--mat-mul-only", type=int, nargs="?", const=0, default=None, metavar="LAUNCHES",
                    help="only the compute-bound mat_mul shapes (not the benchmark line); with a number, that many "
                         "plain launches per shape, for hardware-counter runs")
    ap.add_argument("--attention-only", type=int, nargs="?", const=0, default=None, metavar="LAUNCHES",
                    help="only attention at prefill shapes, causal and unmasked; with a number, that many launches per "
                         "shape (hardware-counter runs)")
    ap.add_argument("--floors", action="store_true",
                    help="only the decode layer's GEMMs on cold operands, each beside a bare read of the same bytes")
    ap.add_argument("--granules", action="store_true",
                    help="only the granule-class probe: how long a walk down each 128-column strip of a weight takes")
    ap.add_argument("--ceilings", action="store_true",
                    help="only the machine's ceilings: stream probes (read, write, copy) and the bare MFMA loop")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import ophip
    if not os.path.exists(ophip.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    gpu = ophip.Gpu(0)
    info = gpu.info()
    log("device: %s (%s), %d CUs" % (info.name.decode(), info.arch.decode(), info.compute_units))
    stream = gpu.stream()
    rng = np.random.default_rng(0)
    if args.floors:
        print(json.dumps({"floors": gemm_floors(ophip, gpu, stream, rng, args.reps)}))
        return
    if args.ceilings:
        print(json.dumps({"ceilings": ceilings(ophip, gpu, stream)}))
        return
    if args.granules:
        print(json.dumps({"granules": granule_classes(ophip, gpu, stream)}))
        return
    if args.attention_only is not None:
        lines = []
        attention_lines(ophip, gpu, stream, rng, adder(lines), args.attention_only or 20, full=True)
        print(json.dumps({"attention": lines}))
        return
    if args.mat_mul_only is not None:
        lines = []
        mat_mul_lines(ophip, gpu, stream, rng, adder(lines), launches=args.mat_mul_only)
        print(json.dumps({"mat_mul": lines}))
        return

    # two layers' worth of distinct weights (2 x 404 MB), alternated per step, so no
    # step finds its weights in the 256 MiB Infinity Cache
    layers = [Layer(ophip, gpu, rng, host=(i == 0)) for i in range(2)]
    work = layer_work()
    layer_bytes = sum(work[n][0] for n in layers[0].order)
    layer_flops = sum(work[n][1] for n in layers[0].order)

    for i in range(args.warmup):
        layers[i % 2].step(stream)
    stream.synchronize()

    # The dominant kernel is timed on every EVERY-th step only (an odd stride, so both weight sets are sampled;
    # `roofline.samples` says how many launches that was):
    # its launch carries two events that the kernel itself records at its begin and its end (the figure the
    # rocprofv3 trace must agree with).
    DOM = "gate_up"  # (a launch that carries events costs the step about 4 us: at most a quarter of the steps carry them)
    EVERY = max(1, min(25, args.steps // 4)) | 1
    own = [(gpu.event(), gpu.event()) for _ in range(0, args.steps, EVERY)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        layers[i % 2].step(stream, own={DOM: own[i // EVERY]} if i % EVERY == 0 else None)
    stream.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    dom_us = float(np.mean([a.elapsed_ms(b) for a, b in own])) * 1e3
    # The same steps replayed from a recorded launch graph (two steps, one per weight set, per replay): what the
    # host's launch calls cost the step, if anything.  Reported beside `ms_per_step`, which stays the eager figure.
    stream.begin_capture()
    for lay in layers:
        lay.step(stream)
    graph = stream.end_capture()
    for _ in range(max(1, args.warmup // 2)):
        graph.launch(stream)
    stream.synchronize()
    t0g = time.perf_counter()
    for _ in range(args.steps // 2):
        graph.launch(stream)
    stream.synchronize()
    graph_ms_per_step = (time.perf_counter() - t0g) * 1e3 / (2 * (args.steps // 2)) if args.steps >= 2 else None
    graph.destroy()
    # The layer with the crate's composite attention_kv_cached in place of QK^T / softmax / PV (nine launches of the
    # operator API, ten kernels): what a runtime that calls the crate's attention operator sees.  Reported beside the
    # headline, which stays BASELINE's eleven-launch chain.
    for i in range(max(2, args.warmup // 2)):
        layers[i % 2].step(stream, order=layers[i % 2].order_attention_op)
    stream.synchronize()
    t0a = time.perf_counter()
    for i in range(args.steps):
        layers[i % 2].step(stream, order=layers[i % 2].order_attention_op)
    stream.synchronize()
    attn_ms_per_step = (time.perf_counter() - t0a) * 1e3 / args.steps
    attn_bytes = sum(work[n][0] for n in layers[0].order_attention_op)
    # For comparison, outside the timed region: two separate event records around the same launch, which read
    # longer by most of what an empty pair of records reads.
    pairs = [(gpu.event(), gpu.event()) for _ in range(20)]
    for i, pr in enumerate(pairs):
        layers[i % 2].step(stream, around={DOM: pr})
    stream.synchronize()
    bracketed_us = float(np.mean([a.elapsed_ms(b) for a, b in pairs])) * 1e3
    # What a pair of event records reads with nothing between them, in the same position of the layer
    # (after rms_norm_2): the part of the bracketed time that is not the kernel.
    empties = [(gpu.event(), gpu.event()) for _ in range(40)]
    for e0, e1 in empties:
        layers[0].launch("rms_norm_2", stream)
        e0.record(stream)
        e1.record(stream)
        layers[0].launch("swiglu", stream)
    stream.synchronize()
    event_pair_us = float(np.mean([a.elapsed_ms(b) for a, b in empties])) * 1e3
    dom_bytes = work[DOM][0]

    ceiling = copy_ceiling(ophip, gpu, stream)
    # per-op times inside the layer (back-to-back launches of one op; small ops are cache-resident)
    per_layer = []
    log("decode layer, per op:")
    for name in layers[0].order + ["attention_kv_cached"]:
        us = time_launches(gpu, stream, lambda: layers[0].launch(name, stream), args.reps)
        b, f = work[name]
        rec = {"op": name, "us": round(us, 3), "bytes": b, "GBps": round(b / us / 1e3, 1),
               "hbm_frac": round(b / (us * 1e-6) / HBM_PEAK, 4),
               "ceiling_frac": round(b / us / 1e3 / ceiling["GBps"], 4)}
        if f:
            rec["TFLOPs"] = round(f / us / 1e6, 2)
        if b < (256 << 20):
            rec["cache_resident"] = True
        kind, a = layers[0].args[name]
        if kind == "mm":
            rec["kernel"] = layers[0].ops["mm"].describe(a)  # which kernel family and K cut the planner chose
        per_layer.append(rec)
        log("  %-12s %9.2f us %9.1f GB/s %5.1f%% HBM" % (name, us, rec["GBps"], 100 * rec["hbm_frac"]))

    per_op = []
    if not args.no_per_op:
        log("standalone operators:")
        per_op = standalone_ops(ophip, gpu, stream, rng, args.reps, ceiling)

    cpu = None
    if not args.no_cpu:
        import oracle
        threads = min(oracle.max_threads(), 16)
        h = layers[0].h
        t_cpu, n_cpu = 0.0, 0
        while n_cpu < 2 or (t_cpu < 10.0 and n_cpu < 20):
            c0 = time.perf_counter()
            cpu_layer_step(oracle, h, threads)
            t_cpu += time.perf_counter() - c0
            n_cpu += 1
        # the same oracle on the single-operator configurations, beside their GPU lines
        for (op_name, shape), us in cpu_per_op(oracle, threads).items():
            for rec in per_op:
                if rec["op"] == op_name and rec["shape"] == shape:
                    rec["cpu_us"], rec["cpu_threads"] = round(us, 1), threads
        cpu = {"value": round(layer_bytes / (t_cpu / n_cpu) / 1e9, 3), "unit": "GB/s", "cores": threads,
               "kind": "port", "ms_per_step": round(t_cpu / n_cpu * 1e3, 2),
               "sample": "%d full decode-layer steps of the same workload through the CPU oracle" % n_cpu}

    result = {
        "metric": "per-op HBM GB/s (% of 8 TB/s) + us/op at Llama-7B shapes; mat_mul MFMA %",
        "value": round(layer_bytes / (ms_per_step * 1e-3) / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "graph_replay_ms_per_step": round(graph_ms_per_step, 5) if graph_ms_per_step else None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama7b_decode_layer_16tok_kv2048 (BASELINE.json configs[4])",
                   "launches_per_step": len(layers[0].order), "algorithmic_bytes_per_step": layer_bytes,
                   "flops_per_step": layer_flops, "hbm_frac_of_step": round(layer_bytes / (ms_per_step * 1e-3) / HBM_PEAK, 4),
                   # the same layer through the crate's own attention_kv_cached operator instead of the three scripted
                   # attention launches (not the headline: BASELINE.json's chain is the eleven launches above)
                   "ms_per_step_with_attention_op": round(attn_ms_per_step, 5),
                   "launches_per_step_with_attention_op": len(layers[0].order_attention_op),
                   "algorithmic_bytes_per_step_with_attention_op": attn_bytes},
        "roofline": {"bound": "hbm", "kernel": "gemm_stream_m1 (gate/up mat_mul 16x4096 . 4096x22016)",
                     "achieved": round(dom_bytes / (dom_us * 1e-6) / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(dom_bytes / (dom_us * 1e-6) / HBM_PEAK, 4), "traffic": profiled_traffic(),
                     "us": round(dom_us, 3), "samples": len(own), "algorithmic_bytes": dom_bytes,
                     "bracketed_us": round(bracketed_us, 3) if bracketed_us is not None else None,
                     "event_pair_us": round(event_pair_us, 3),
                     "note": "us is between two events the kernel's own launch records at its begin and end, inside the "
                             "timed steps; bracketed_us is between two separate event records around the launch (20 "
                             "more steps after the timed ones), event_pair_us what such a pair reads with no kernel "
                             "between them"},
        "cpu_baseline": cpu,
        "copy_ceiling": ceiling,
        "per_op_layer": per_layer,
        "per_op": per_op,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
