"""CPU-only checks of the C ABI: the library loads, exports every declared symbol,
and its host-side logic (layout normalisers, validators, allocator bookkeeping)
agrees with the reference's known answers and with the oracle.  No compute call
is made here, so no GPU is needed."""
import os
import re

import numpy as np
import pytest

import ophip
import oracle
from ophip import TensorLayout, dt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F16 = dt.F16


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "ophip.h")).read()
    declared = set(re.findall(r"OPHIP_API[^;(]*?\b(ophip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 60
    L = ophip.lib()
    missing = sorted(s for s in declared if not hasattr(L, s))
    assert not missing, missing
    assert declared == set(ophip.EXPORTS)


def test_status_names_and_dtype_sizes():
    L = ophip.lib()
    names = ["Ok", "TypeNotSupport", "TypeMismatch", "RankNotSupport", "RankMismatch", "ShapeNotSupport",
             "ShapeMismatch", "StridesNotSupport", "ArgsNotSupport", "DynamicNotSupport"]
    assert [L.ophip_status_name(i).decode() for i in range(10)] == names
    assert L.ophip_status_name(100).decode() == "ExecutionFailed"
    for d in range(1, 15):
        assert L.ophip_dtype_nbytes(d) == ophip.dtype_nbytes(d)
    assert L.ophip_dtype_nbytes(99) == 0


def test_no_device_means_no_backend():
    if ophip.device_count() > 0:
        pytest.skip("a GPU is present")
    assert ophip.Gpu.init() is None
    with pytest.raises(ophip.SchemeError) as e:
        ophip.Gpu(0)
    assert e.value.kind == "ExecutionFailed"


def rearr_args(shape, dst_strides, src_strides, dtype=F16, src_shape=None):
    return ophip.RearrangeArgs(TensorLayout(dtype, shape, dst_strides), None,
                               TensorLayout(dtype, src_shape or shape, src_strides), None)


def test_rearrange_plan_reference_known_answers():
    """rearrange/args.rs:242-304"""
    s = ophip.Rearrange.plan(rearr_args([4, 3, 2, 1, 2, 3, 4], [288, 96, 48, 48, 24, 8, 2],
                                        [576, 192, 96, 48, 8, 16, 2]))
    assert s == [8, 144, 6, 3, 1, 48, 24, 8, 96, 8, 16]
    st = [33554432 * 2, 16777216 * 2, 524288 * 2, 128 * 2, 2]
    assert ophip.Rearrange.plan(rearr_args([32, 2, 32, 456, 128], st, st)) == [116736, 2048, 1, 1048576, 1048576]
    assert ophip.Rearrange.plan(rearr_args([32, 512, 128], [256, 8192, 2], [131072, 256, 2])) == \
        [256, 16384, 32, 1, 8192, 256, 256, 131072]


def test_rearrange_plan_matches_oracle_on_random_layouts():
    rng = np.random.default_rng(0)
    for _ in range(300):
        nd = int(rng.integers(0, 6))
        shape = [int(rng.integers(1, 6)) for _ in range(nd)]
        es = int(rng.choice([1, 2, 4, 8]))
        dtype = {1: dt.U8, 2: dt.F16, 4: dt.F32, 8: dt.F64}[es]

        def strides():
            perm = rng.permutation(nd)
            st, mul = [0] * nd, es
            for ax in perm:
                st[ax] = mul * int(rng.choice([1, 1, 1, 2])) * int(rng.choice([1, 1, -1]))
                mul = abs(st[ax]) * shape[ax]
            return st

        ds, ss = strides(), strides()
        want = oracle.rearrange_scheme(shape, ds, ss, es)
        got = ophip.Rearrange.plan(rearr_args(shape, ds, ss, dtype))
        nd_o = (len(want) - 2) // 3
        assert got[: 2 + nd_o] == want[: 2 + nd_o]
        # dims equal under the sort key may come out in either order; the strides are the same multiset
        assert sorted(zip(got[2 + nd_o: 2 + 2 * nd_o], got[2 + 2 * nd_o:])) == \
            sorted(zip(want[2 + nd_o: 2 + 2 * nd_o], want[2 + 2 * nd_o:]))


def test_rearrange_plan_errors():
    cases = [
        (rearr_args([2, 3], [0, 4], [12, 4], dt.F32), "ShapeNotSupport"),
        (rearr_args([2, 3], [12, 4], [12, 4], dt.F32, src_shape=[2, 4]), "ShapeMismatch"),
        (rearr_args([None, 3], [12, 4], [12, 4], dt.F32, src_shape=[None, 3]), "DynamicNotSupport"),
        (ophip.RearrangeArgs(TensorLayout(dt.F32, [2, 3], [12, 4]), None, TensorLayout(dt.F32, [6], [4]), None),
         "RankMismatch"),
        (ophip.RearrangeArgs(TensorLayout(dt.F32, [6], [4]), None, TensorLayout(dt.U32, [6], [4]), None),
         "TypeMismatch"),
    ]
    for args, kind in cases:
        with pytest.raises(ophip.SchemeError) as e:
            ophip.Rearrange.plan(args)
        assert e.value.kind == kind


def mm_args(c, a, b, dtype=F16):
    mk = lambda arr: TensorLayout(dtype, arr.shape, arr.strides)
    return ophip.MatMulArgs(mk(c), None, 1.0, mk(a), None, mk(b), None, 1.0)


def test_mat_mul_plan_matches_oracle_layout():
    f16 = np.float16
    z = lambda *s: np.zeros(s, f16)
    cases = [
        (z(5, 7), z(5, 3), z(3, 7)),
        (z(7, 5).T, z(5, 3), z(3, 7)),
        (z(5, 7), z(3, 5).T, z(7, 3).T),
        (z(7, 5).T, z(3, 5).T, z(3, 7)),
        (z(4, 5, 7), z(4, 5, 3), z(1, 3, 7)),
        (z(4, 5, 7), z(5, 3), z(4, 7, 3).transpose(0, 2, 1)),
        (z(16, 12288), z(16, 4096), z(4096, 12288)),
        (z(32, 16, 2048), z(32, 16, 128), z(32, 2048, 128).transpose(0, 2, 1)),
    ]
    for c, a, b in cases:
        got = mm_args(c, a, b).layout().as_dict()
        want = oracle.mat_mul_layout(2, (c.shape, c.strides), (a.shape, a.strides), (b.shape, b.strides)).as_dict()
        assert got == want, (got, want)
    assert mm_args(*cases[0]).layout().as_dict() == dict(
        ab_swap=1, a_trans=0, b_trans=0, batch=1, m=7, n=5, k=3, c_stride=0, c_ld=7, a_stride=0, a_ld=7,
        b_stride=0, b_ld=3)


def test_mat_mul_plan_errors():
    f16 = np.float16
    z = lambda *s: np.zeros(s, f16)
    cases = [
        ((z(5, 7), z(5, 4), z(3, 7)), "ShapeMismatch"),
        ((z(10, 14)[::2, ::2], z(5, 3), z(3, 7)), "StridesNotSupport"),
        ((z(5, 7), z(10, 6)[::2, ::2], z(3, 7)), "StridesNotSupport"),
        ((z(7), z(5, 3), z(3, 7)), "RankNotSupport"),
        ((z(1, 1, 5, 7), z(5, 3), z(3, 7)), "ShapeNotSupport"),
        ((z(2, 5, 7), z(3, 5, 3), z(3, 7)), "ShapeMismatch"),
    ]
    for (c, a, b), kind in cases:
        with pytest.raises(ophip.SchemeError) as e:
            mm_args(c, a, b).layout()
        assert e.value.kind == kind, kind
    args = mm_args(z(5, 7), z(5, 3), z(3, 7))
    args.a_layout = TensorLayout(F16, [5, None], [6, 2])
    with pytest.raises(ophip.SchemeError) as e:
        args.layout()
    assert e.value.kind == "DynamicNotSupport"
    args = mm_args(z(5, 7), z(5, 3), z(3, 7))
    args.b_layout = TensorLayout(dt.F32, [3, 7], [28, 4])
    with pytest.raises(ophip.SchemeError) as e:
        args.layout()
    assert e.value.kind == "TypeMismatch"


def test_sample_args_constructor_rules():
    """random_sample/args.rs:66-84"""
    with pytest.raises(ophip.SampleArgsError, match="NegativeTemperature"):
        ophip.SampleArgs(-0.1, 0.9, 50)
    with pytest.raises(ophip.SampleArgsError, match="NonPositiveTop"):
        ophip.SampleArgs(0.8, 0.9, 0)
    with pytest.raises(ophip.SampleArgsError, match="NonPositiveTop"):
        ophip.SampleArgs(0.8, 0.0, 50)
    s = ophip.SampleArgs(0.8, 1.7, 50)
    assert s.struct.top_p == 1.0 and not s.is_argmax()
    assert ophip.SampleArgs(0.0, 0.9, 50).is_argmax() and ophip.SampleArgs(0.8, 0.9, 1).is_argmax()
    am = ophip.SampleArgs.argmax()
    assert (am.struct.temperature, am.struct.top_p, am.struct.top_k) == (0.0, 1.0, ophip.DYN_USIZE)


def test_offset_calculator_best_fit_and_coalescing():
    """common/calculator.rs:25-79"""
    c = ophip.OffsetCalculator(256)
    assert c.take(0) == (ophip.DYN_USIZE, ophip.DYN_USIZE)  # zero size: sentinel
    assert c.take(1) is None
    c.put(0x10000, 0x10000 + 4096)
    c.put(0x40000, 0x40000 + 1024)
    a = c.take(1000)  # best fit: the 1 KiB area, not the 4 KiB one
    assert a == (0x40000, 0x40000 + 1000)
    b = c.take(300)  # rounded to 512, carved from the 4 KiB area
    assert b == (0x10000, 0x10000 + 300)
    d = c.take(3584)
    assert d == (0x10000 + 512, 0x10000 + 512 + 3584)
    assert c.take(1) is None
    c.put(*b)
    c.put(*d)  # coalesces with the neighbour to its left
    assert c.take(4096) == (0x10000, 0x10000 + 4096)
    c.put(*a)
    assert c.take(1024) == (0x40000, 0x40000 + 1024)


def test_tile_gemm_code_objects_keep_accumulators_in_registers():
    """A tile-GEMM loop that fails to unroll puts its 256 accumulators into scratch memory and the kernel
    runs an order of magnitude slower without any error: check the private segment size in the built code
    object's metadata.  Skipped where the build directory or the ROCm binutils are absent."""
    import shutil
    import subprocess
    hsaco = os.path.join(os.path.dirname(ophip.__file__), "..", "csrc", "build", "gemm_tile.hsaco")
    readelf = shutil.which("llvm-readelf") or "/opt/rocm/llvm/bin/llvm-readelf"
    if not os.path.exists(hsaco) or not os.path.exists(readelf):
        pytest.skip("no built code object or no llvm-readelf here")
    notes = subprocess.run([readelf, "--notes", hsaco], capture_output=True, text=True, check=True).stdout
    names = re.findall(r"\.name:\s+(\S+)", notes)
    scratch = [int(v) for v in re.findall(r"\.private_segment_fixed_size:\s+(\d+)", notes)]
    assert len(names) == len(scratch) == 24, (names, scratch)  # 3 tiles x 4 operand layouts, whole-tile and ragged builds
    for name, size in zip(names, scratch):
        assert size <= 512, "%s uses %d bytes of scratch per lane" % (name, size)


# ---- the Rust side's declarations against the header, as text (no rustc, no C compiler needed) ----------------

SHIM = os.path.join(ROOT, "operators-rs_amd", "rust_shim", "operators", "src")


def _both_sides():
    import abi_text

    hs, hf, he, ho = abi_text.parse_header(open(os.path.join(ROOT, "include", "ophip.h")).read())
    rs, rf, ro = abi_text.parse_rust_ffi(open(os.path.join(SHIM, "handle", "hip", "ffi.rs")).read())
    return hs, hf, he, ho, rs, rf, ro


def test_rust_ffi_structs_mirror_the_header():
    """Every struct of include/ophip.h exists in ffi.rs with the same fields, in the same order, of the same types
    (C spelling mapped to Rust: size_t = usize, ptrdiff_t = isize, const T * = *const T ...), and ffi.rs has none
    the header lacks."""
    hs, _, _, ho, rs, _, ro = _both_sides()
    assert len(hs) >= 20 and set(hs) == set(rs), (sorted(set(hs) - set(rs)), sorted(set(rs) - set(hs)))
    for name, fields in hs.items():
        assert rs[name] == fields, "%s:\n  header %s\n  ffi.rs %s" % (name, fields, rs[name])
    assert set(ho) == set(ro) - {"ophip_device"} | ({"ophip_device"} & set(ho)), (sorted(set(ho) ^ set(ro)))


def test_rust_ffi_functions_mirror_the_header():
    """Every OPHIP_API function is declared in ffi.rs (the four verbs of an operator through the `verbs!` macro, which
    the reader expands) with the same argument count, order and types and the same return type."""
    _, hf, _, _, _, rf, _ = _both_sides()
    assert len(hf) >= 100 and set(hf) == set(rf), (sorted(set(hf) - set(rf)), sorted(set(rf) - set(hf)))
    for name, sig in hf.items():
        assert rf[name] == sig, "%s:\n  header %s\n  ffi.rs %s" % (name, sig, rf[name])
    assert set(hf) == set(ophip.EXPORTS)


def test_rust_side_uses_the_headers_codes():
    """The status codes the Rust side turns into SchemeErrorKind and the dtype codes it sends are the header's."""
    _, _, he, _, _, _, _ = _both_sides()
    mod = open(os.path.join(SHIM, "handle", "hip", "mod.rs")).read()
    # fn scheme_kind: `1 => TypeNotSupport,` ...
    body = mod[mod.index("fn scheme_kind"):]
    body = body[:body.index("\n}\n")]
    rust_status = {name: int(code) for code, name in re.findall(r"(\d+)\s*=>\s*(\w+)\s*,", body)}
    camel = lambda c: "".join(w.capitalize() for w in c[len("OPHIP_"):].lower().split("_"))
    header_status = {camel(k): v for k, v in he["ophip_status"].items() if 1 <= v <= 9}
    assert rust_status == header_status and len(rust_status) == 9
    L = ophip.lib()
    for name, code in rust_status.items():
        assert L.ophip_status_name(code).decode() == name  # and the library names them the same way
    # fn dt_code: `(ty::F16, 1),` ... and the KVPair code
    body = mod[mod.index("fn dt_code"):]
    body = body[:body.index("\n}\n")]
    rust_dt = {name.upper(): int(code) for name, code in re.findall(r"\(ty::(\w+),\s*(\d+)\)", body)}
    rust_dt["KVPAIR"] = int(re.search(r"KVPair[^\n]*\{\s*return\s+(\d+);", body, flags=re.S).group(1))
    header_dt = {k[len("OPHIP_DT_"):]: v for k, v in he["ophip_dtype"].items()}
    assert rust_dt == header_dt, (rust_dt, header_dt)
    assert he["ophip_attn_mask"] == {"OPHIP_MASK_NONE": 0, "OPHIP_MASK_CAUSAL": 1}


def test_every_operator_of_the_rust_side_names_what_the_header_has():
    """The per-operator modules hand `ophip_*` names to the `hip_operator!` macro and build the argument structs
    field by field: every name is a function, struct or opaque type of the header, and every struct literal sets
    exactly the header's fields."""
    hs, hf, _, ho, _, _, _ = _both_sides()
    known = set(hf) | set(hs) | set(ho) | {"ophip_stream", "ophip_event", "ophip_graph"}  # (the three pointer typedefs)
    used, literals = set(), 0
    for d, _, files in os.walk(SHIM):
        for f in files:
            if not f.endswith(".rs") or f == "ffi.rs":
                continue
            text = re.sub(r"//[^\n]*", " ", open(os.path.join(d, f)).read())
            used |= set(re.findall(r"\b(ophip_[a-z0-9_]+)\b", text))
            for m in re.finditer(r"ffi::(ophip_\w+)\s*\{", text):
                name, depth, top, i = m.group(1), 1, "", m.end()
                if name not in hs:  # `-> *mut ffi::ophip_device {`: a function body, not a literal
                    continue
                while depth:  # the literal's own level, nested literals left out
                    ch = text[i]
                    depth += (ch == "{") - (ch == "}")
                    if depth == 1 and ch not in "{}":
                        top += ch
                    i += 1
                if ".." in top:  # `{ .. }` in a doc example
                    continue
                fields = re.findall(r"(?:^|,)\s*(\w+)\s*:(?!:)", top)
                if not fields:  # `-> ffi::ophip_device_info {`: a function body again
                    continue
                assert fields == [n for n, _ in hs[name]], (f, name, fields)
                literals += 1
    assert len(used) >= 60 and literals >= 11
    assert used <= known, sorted(used - known)


# ---- the kernels' workgroup size against the host's launches, as text ---------------------------------------------

def test_kernels_that_stride_by_their_workgroup_size_are_launched_with_it():
    """The streaming kernels advance by the constant WG_THREADS (device_util.h) instead of blockDim.x (which, read
    inside a __device__ function, costs a vector load and a wait at the head of every workgroup): no kernel source may
    read blockDim inside such a function, and the host must launch every kernel of those files with exactly that many
    threads, or with a size the kernel takes as a template argument."""
    csrc = os.path.join(ROOT, "operators-rs_amd", "csrc")
    util = open(os.path.join(csrc, "kernels", "device_util.h")).read()
    wg = int(re.search(r"constexpr uint32_t WG_THREADS = (\d+);", util).group(1))
    assert wg == 256
    users = []
    for f in sorted(os.listdir(os.path.join(csrc, "kernels"))):
        if not f.endswith(".hip"):
            continue
        text = re.sub(r"//[^\n]*", " ", open(os.path.join(csrc, "kernels", f)).read())
        if "WG_THREADS" in text:
            users.append(f[:-4])
        for m in re.finditer(r"blockDim", text):
            # allowed only directly in a __global__ function: the nearest function head above it is one
            head = text.rfind("__global__", 0, m.start()), text.rfind("__device__", 0, m.start())
            assert head[0] > head[1], (f, text[m.start() - 60:m.start() + 20])
    assert {"add", "add_rows", "gelu", "swiglu", "rearrange", "rope", "rms_norm", "layer_norm"} <= set(users)
    # the host's launches of those modules: Dim3{256}, Dim3{block} (a templated group size) or the 1024-thread stream kernels
    host = "".join(open(os.path.join(csrc, "host", f)).read() for f in ("ops.cpp", "ops_more.cpp", "handle.cpp"))
    sizes = set(re.findall(r"launch\([^;]*?Dim3\{[^;]*?\},\s*Dim3\{([^}]*)\}", host, re.S))
    assert sizes <= {"256", "block", "1024", "256u", "1"}, sizes


def test_null_operators_and_arguments_come_back_as_status_codes():
    """A binding that passes a null operator, null arguments or no queue allocator gets ArgsNotSupport from every
    launch (and a status code, not a crash, from every scheme and create): no device is needed to be refused."""
    import ctypes

    L = ophip.lib()
    names = ["rms_norm", "rope", "fused_softmax", "rearrange", "swiglu", "random_sample", "mat_mul", "attention",
             "attention_kv_cached", "layer_norm", "gelu", "add", "add_rows", "conv"]
    ws = ctypes.c_size_t(0)
    for n in names:
        assert getattr(L, "ophip_%s_create" % n)(None, None) == 8, n
        assert getattr(L, "ophip_%s_launch" % n)(None, None, None, ctypes.c_size_t(0), None) == 8, n
        assert getattr(L, "ophip_%s_scheme" % n)(None, None, ctypes.c_size_t(0), ctypes.byref(ws)) in (0, 8), n
        getattr(L, "ophip_%s_destroy" % n)(None)
    assert L.ophip_random_sample_launch_batch(None, None, ctypes.c_size_t(1), ctypes.c_ssize_t(0), None, None, ctypes.c_size_t(0), None) == 8
    assert L.ophip_mat_mul_launch_static(None, None, None) == 8
    assert L.ophip_sample_args_new(ctypes.c_float(1.0), ctypes.c_float(1.0), ctypes.c_size_t(1), None) == 8
    # layouts of non-zero rank that bring no shape or strides
    empty = ophip._Layout(ctypes.c_uint64(int(dt.F16)), ctypes.c_uint64(3), None, None)

    class NoArrays:
        def c(self):
            return empty

    b = NoArrays()
    makers = {"rms_norm": lambda: ophip.RmsNormArgs(b, None, b, None, b, None, 1e-5), "rope": lambda: ophip.RopeArgs(b, None, b, None, b, None, b, None, 1e4),
              "fused_softmax": lambda: ophip.FusedSoftmaxArgs(1, b, None), "swiglu": lambda: ophip.SwigluArgs(b, None, b, None),
              "attention": lambda: ophip.AttentionArgs(b, None, b, None, b, None, b, None, 1),
              "attention_kv_cached": lambda: ophip.AttnKVCachedArgs(b, None, b, None, b, None, b, None, b, None, b, None, 1, 0),
              "layer_norm": lambda: ophip.LayerNormArgs(b, None, b, None, b, None, b, None, 1e-5), "gelu": lambda: ophip.GeluArgs(b, None),
              "add_rows": lambda: ophip.AddRowsArgs(b, None, b, None, b, None)}
    for rank in (1, 2, 3):
        empty.ndim = rank
        for n, make in makers.items():
            args = make().c()
            assert getattr(L, "ophip_%s_scheme" % n)(None, ctypes.byref(args), ctypes.c_size_t(0), ctypes.byref(ws)) != 0, (n, rank)
        for plan, make in (("ophip_mat_mul_plan", lambda: ophip.MatMulArgs(b, None, 0.0, b, None, b, None, 1.0)),):
            out = ophip.MatMulLayout()
            assert getattr(L, plan)(ctypes.byref(make().c()), ctypes.byref(out)) != 0, rank
    # the handle: a null device, or nowhere to put the result
    Z = ctypes.c_size_t(0)
    handle_calls = {
        "device_get_info": lambda: L.ophip_device_get_info(None, None), "malloc": lambda: L.ophip_malloc(None, Z, None),
        "free": lambda: L.ophip_free(None, None), "memcpy_h2d": lambda: L.ophip_memcpy_h2d(None, None, None, Z, None),
        "memcpy_d2h": lambda: L.ophip_memcpy_d2h(None, None, None, Z, None), "memcpy_d2d": lambda: L.ophip_memcpy_d2d(None, None, None, Z, None),
        "memset": lambda: L.ophip_memset(None, None, 0, Z, None), "stream_create": lambda: L.ophip_stream_create(None, None),
        "stream_destroy": lambda: L.ophip_stream_destroy(None, None), "stream_synchronize": lambda: L.ophip_stream_synchronize(None, None),
        "event_create": lambda: L.ophip_event_create(None, None), "event_record": lambda: L.ophip_event_record(None, None, None),
        "event_synchronize": lambda: L.ophip_event_synchronize(None, None), "event_elapsed_ms": lambda: L.ophip_event_elapsed_ms(None, None, None, None),
        "event_destroy": lambda: L.ophip_event_destroy(None, None), "time_next_launch": lambda: L.ophip_time_next_launch(None, None, None, None),
        "stream_begin_capture": lambda: L.ophip_stream_begin_capture(None, None), "stream_end_capture": lambda: L.ophip_stream_end_capture(None, None, None),
        "graph_launch": lambda: L.ophip_graph_launch(None, None, None), "graph_destroy": lambda: L.ophip_graph_destroy(None, None),
        "queue_alloc_from_stream": lambda: L.ophip_queue_alloc_from_stream(None, None, None), "mem_pool_create": lambda: L.ophip_mem_pool_create(None, None, None),
        "mem_pool_put": lambda: L.ophip_mem_pool_put(None, Z), "mem_pool_queue_alloc": lambda: L.ophip_mem_pool_queue_alloc(None, None),
        "rope_build_pos": lambda: L.ophip_rope_build_pos(ctypes.c_uint64(0), Z, None, Z, None, None), "rearrange_plan": lambda: L.ophip_rearrange_plan(None, None, None),
        "random_sample_build_indices": lambda: L.ophip_random_sample_build_indices(Z, None, None), "mat_mul_plan": lambda: L.ophip_mat_mul_plan(None, None),
        "mat_mul_describe": lambda: L.ophip_mat_mul_describe(None, None, None, Z), "add_plan": lambda: L.ophip_add_plan(None, None, None),
        "device_create": lambda: L.ophip_device_create(0, None, None),
    }
    for name, call in handle_calls.items():
        assert call() == 8, name
    L.ophip_mem_pool_destroy(None), L.ophip_device_release(None), L.ophip_device_retain(None)
    L.ophip_offset_calculator_put(None, Z, Z)
    assert L.ophip_offset_calculator_take(None, Z, None, None) == 0
