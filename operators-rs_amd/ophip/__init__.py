"""ctypes binding of ``libophip.so`` — the MI355X backend behind the operators-rs API.

The names follow the reference crate: ``Gpu`` is the hardware handle, every
operator has ``scheme(args, max_workspace_size)`` and
``launch(args, workspace, queue_alloc)``, arguments are ``*Args`` structs made of
``TensorLayout`` + raw device base pointers + scalars, errors are
``SchemeError`` / ``LaunchError`` values carrying the reference's error kinds.

This module is a thin layer over the C ABI declared in ``include/ophip.h``; it
contains no arithmetic and has no CPU fallback: if the shared library or a GPU
is missing, calls raise.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libophip.so")

DYN_USIZE = 2 ** 64 - 1
DYN_ISIZE = 2 ** 63 - 1


class dt:
    F16, BF16, F32, F64, U8, U16, U32, U64, I8, I16, I32, I64, BOOL, KVPAIR = range(1, 15)


NP_DT = {np.dtype(np.float16): dt.F16, np.dtype(np.float32): dt.F32, np.dtype(np.float64): dt.F64,
         np.dtype(np.uint8): dt.U8, np.dtype(np.uint16): dt.U16, np.dtype(np.uint32): dt.U32,
         np.dtype(np.uint64): dt.U64, np.dtype(np.int8): dt.I8, np.dtype(np.int16): dt.I16,
         np.dtype(np.int32): dt.I32, np.dtype(np.int64): dt.I64}

STATUS = {0: "Ok", 1: "TypeNotSupport", 2: "TypeMismatch", 3: "RankNotSupport", 4: "RankMismatch",
          5: "ShapeNotSupport", 6: "ShapeMismatch", 7: "StridesNotSupport", 8: "ArgsNotSupport",
          9: "DynamicNotSupport", 100: "ExecutionFailed"}


class SchemeError(Exception):
    def __init__(self, code, info=""):
        super().__init__("%s %s" % (STATUS.get(code, code), info))
        self.code = code
        self.kind = STATUS.get(code, str(code))
        self.info = info


class LaunchError(SchemeError):
    pass


class _Layout(ctypes.Structure):
    _fields_ = [("dt", ctypes.c_uint64), ("ndim", ctypes.c_uint64),
                ("shape", ctypes.POINTER(ctypes.c_size_t)), ("strides", ctypes.POINTER(ctypes.c_ssize_t))]


class TensorLayout:
    """common/tensor.rs: dtype + shape + byte strides; ``None`` marks a dynamic value."""

    def __init__(self, dtype, shape, strides):
        assert len(shape) == len(strides)
        self.dt = int(dtype)
        self.shape = [DYN_USIZE if s is None else int(s) for s in shape]
        self.strides = [DYN_ISIZE if s is None else int(s) for s in strides]
        n = max(len(shape), 1)
        self._shape = (ctypes.c_size_t * n)(*self.shape)
        self._strides = (ctypes.c_ssize_t * n)(*self.strides)

    @classmethod
    def new_contiguous(cls, dtype, shape):
        unit = dtype_nbytes(dtype)
        strides, mul = [], unit
        for d in reversed(shape):
            strides.append(mul)
            mul *= d
        return cls(dtype, shape, strides[::-1])

    @classmethod
    def of(cls, array):
        """Layout of a numpy array or view (shape + byte strides)."""
        return cls(NP_DT[array.dtype], array.shape, array.strides)

    def c(self):
        return _Layout(self.dt, len(self.shape), self._shape, self._strides)


class _QueueAlloc(ctypes.Structure):
    _fields_ = [("ctx", ctypes.c_void_p), ("stream", ctypes.c_void_p),
                ("alloc", ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t)),
                ("free", ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p))]


class _RmsNormArgs(ctypes.Structure):
    _fields_ = [("y_layout", _Layout), ("y_base", ctypes.c_void_p), ("x_layout", _Layout),
                ("x_base", ctypes.c_void_p), ("w_layout", _Layout), ("w_base", ctypes.c_void_p),
                ("epsilon", ctypes.c_float)]


class _RopeArgs(ctypes.Structure):
    _fields_ = [("t_layout", _Layout), ("t_base", ctypes.c_void_p), ("p_layout", _Layout),
                ("p_base", ctypes.c_void_p), ("sin_layout", _Layout), ("sin_base", ctypes.c_void_p),
                ("cos_layout", _Layout), ("cos_base", ctypes.c_void_p), ("theta", ctypes.c_float)]


class _RopeSeq(ctypes.Structure):
    _fields_ = [("pos", ctypes.c_size_t), ("len", ctypes.c_size_t)]


class _SoftmaxArgs(ctypes.Structure):
    _fields_ = [("att_mask", ctypes.c_uint8), ("att_layout", _Layout), ("att_base", ctypes.c_void_p)]


class _RearrangeArgs(ctypes.Structure):
    _fields_ = [("dst_layout", _Layout), ("dst_base", ctypes.c_void_p), ("src_layout", _Layout),
                ("src_base", ctypes.c_void_p)]


class _SwigluArgs(ctypes.Structure):
    _fields_ = [("gate_layout", _Layout), ("gate_base", ctypes.c_void_p), ("up_layout", _Layout),
                ("up_base", ctypes.c_void_p)]


class SampleArgsStruct(ctypes.Structure):
    _fields_ = [("temperature", ctypes.c_float), ("top_p", ctypes.c_float), ("top_k", ctypes.c_size_t)]


class _RandomSampleArgs(ctypes.Structure):
    _fields_ = [("kv_pair", _Layout), ("kv_pair_base", ctypes.c_void_p), ("logits", _Layout),
                ("logits_base", ctypes.c_void_p), ("indices", _Layout), ("indices_base", ctypes.c_void_p),
                ("config", SampleArgsStruct), ("seed", ctypes.c_float)]


class _MatMulArgs(ctypes.Structure):
    _fields_ = [("c_layout", _Layout), ("c_base", ctypes.c_void_p), ("beta", ctypes.c_float),
                ("a_layout", _Layout), ("a_base", ctypes.c_void_p), ("b_layout", _Layout),
                ("b_base", ctypes.c_void_p), ("alpha", ctypes.c_float)]


class MatMulLayout(ctypes.Structure):
    _fields_ = [("dt", ctypes.c_uint64), ("ab_swap", ctypes.c_int32), ("a_trans", ctypes.c_int32),
                ("b_trans", ctypes.c_int32), ("_pad", ctypes.c_int32),
                ("batch", ctypes.c_size_t), ("m", ctypes.c_size_t), ("n", ctypes.c_size_t), ("k", ctypes.c_size_t),
                ("c_stride", ctypes.c_ssize_t), ("c_ld", ctypes.c_ssize_t), ("a_stride", ctypes.c_ssize_t),
                ("a_ld", ctypes.c_ssize_t), ("b_stride", ctypes.c_ssize_t), ("b_ld", ctypes.c_ssize_t)]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_ if k not in ("_pad", "dt")}


class DeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("arch", ctypes.c_char * 32), ("compute_units", ctypes.c_int),
                ("wavefront_size", ctypes.c_int), ("max_threads_per_block", ctypes.c_int),
                ("lds_per_block", ctypes.c_size_t), ("total_memory", ctypes.c_size_t), ("clock_khz", ctypes.c_int)]


class KVPair(ctypes.Structure):
    _fields_ = [("idx", ctypes.c_uint32), ("val", ctypes.c_uint32)]
class _AttentionArgs(ctypes.Structure):
    _fields_ = [("q_layout", _Layout), ("q_base", ctypes.c_void_p), ("k_layout", _Layout),
                ("k_base", ctypes.c_void_p), ("v_layout", _Layout), ("v_base", ctypes.c_void_p),
                ("o_layout", _Layout), ("o_base", ctypes.c_void_p), ("mask", ctypes.c_uint8)]


class _AttnKVCachedArgs(ctypes.Structure):
    _fields_ = [("q_layout", _Layout), ("q_base", ctypes.c_void_p), ("k_layout", _Layout),
                ("k_base", ctypes.c_void_p), ("v_layout", _Layout), ("v_base", ctypes.c_void_p),
                ("o_layout", _Layout), ("o_base", ctypes.c_void_p),
                ("k_cache_layout", _Layout), ("k_cache_base", ctypes.c_void_p),
                ("v_cache_layout", _Layout), ("v_cache_base", ctypes.c_void_p),
                ("mask", ctypes.c_uint8), ("pos", ctypes.c_size_t)]


class _LayerNormArgs(ctypes.Structure):
    _fields_ = [("y_layout", _Layout), ("y_base", ctypes.c_void_p), ("x_layout", _Layout),
                ("x_base", ctypes.c_void_p), ("scale_layout", _Layout), ("scale_base", ctypes.c_void_p),
                ("bias_layout", _Layout), ("bias_base", ctypes.c_void_p), ("epsilon", ctypes.c_float)]


class _GeluArgs(ctypes.Structure):
    _fields_ = [("layout", _Layout), ("base", ctypes.c_void_p)]


class _AddArgs(ctypes.Structure):
    _fields_ = [("c_layout", _Layout), ("c_base", ctypes.c_void_p), ("a_layout", _Layout),
                ("a_base", ctypes.c_void_p), ("b_layout", _Layout), ("b_base", ctypes.c_void_p)]


class _AddRowsArgs(ctypes.Structure):
    _fields_ = [("dst_layout", _Layout), ("dst_base", ctypes.c_void_p), ("src_layout", _Layout),
                ("src_base", ctypes.c_void_p), ("idx_layout", _Layout), ("idx_base", ctypes.c_void_p)]


class _ConvArgs(ctypes.Structure):
    _fields_ = [("y_layout", _Layout), ("y_base", ctypes.c_void_p), ("x_layout", _Layout),
                ("x_base", ctypes.c_void_p), ("w_layout", _Layout), ("w_base", ctypes.c_void_p),
                ("b_layout", _Layout), ("b_base", ctypes.c_void_p), ("strides", ctypes.c_size_t * 2),
                ("dilations", ctypes.c_size_t * 2), ("pads", ctypes.c_size_t * 4)]


# every symbol include/ophip.h declares
EXPORTS = [
    "ophip_last_error", "ophip_status_name", "ophip_dtype_nbytes",
    "ophip_device_create", "ophip_device_retain", "ophip_device_release", "ophip_device_count",
    "ophip_device_get_info",
    "ophip_malloc", "ophip_free", "ophip_memcpy_h2d", "ophip_memcpy_d2h", "ophip_memcpy_d2d", "ophip_memset",
    "ophip_stream_create", "ophip_stream_destroy", "ophip_stream_synchronize",
    "ophip_event_create", "ophip_event_destroy", "ophip_event_record", "ophip_event_synchronize",
    "ophip_event_elapsed_ms", "ophip_time_next_launch",
    "ophip_stream_begin_capture", "ophip_stream_end_capture", "ophip_graph_launch", "ophip_graph_destroy",
    "ophip_queue_alloc_from_stream", "ophip_mem_pool_create", "ophip_mem_pool_put",
    "ophip_mem_pool_queue_alloc", "ophip_mem_pool_destroy",
    "ophip_offset_calculator_create", "ophip_offset_calculator_destroy", "ophip_offset_calculator_put",
    "ophip_offset_calculator_take",
    "ophip_rms_norm_create", "ophip_rms_norm_scheme", "ophip_rms_norm_launch", "ophip_rms_norm_destroy",
    "ophip_rope_create", "ophip_rope_scheme", "ophip_rope_launch", "ophip_rope_destroy",
    "ophip_rope_build_pos", "ophip_rope_build_sincos",
    "ophip_fused_softmax_create", "ophip_fused_softmax_scheme", "ophip_fused_softmax_launch",
    "ophip_fused_softmax_destroy",
    "ophip_rearrange_create", "ophip_rearrange_scheme", "ophip_rearrange_launch", "ophip_rearrange_destroy",
    "ophip_rearrange_plan",
    "ophip_swiglu_create", "ophip_swiglu_scheme", "ophip_swiglu_launch", "ophip_swiglu_destroy",
    "ophip_sample_args_new", "ophip_sample_args_argmax",
    "ophip_random_sample_create", "ophip_random_sample_scheme", "ophip_random_sample_launch",
    "ophip_random_sample_destroy", "ophip_random_sample_build_indices", "ophip_random_sample_launch_batch",
    "ophip_mat_mul_plan", "ophip_mat_mul_create", "ophip_mat_mul_scheme", "ophip_mat_mul_launch",
    "ophip_mat_mul_destroy", "ophip_mat_mul_describe", "ophip_mat_mul_launch_static",
    "ophip_attention_create", "ophip_attention_scheme", "ophip_attention_launch", "ophip_attention_destroy",
    "ophip_attention_kv_cached_create", "ophip_attention_kv_cached_scheme", "ophip_attention_kv_cached_launch",
    "ophip_attention_kv_cached_destroy",
    "ophip_layer_norm_create", "ophip_layer_norm_scheme", "ophip_layer_norm_launch", "ophip_layer_norm_destroy",
    "ophip_gelu_create", "ophip_gelu_scheme", "ophip_gelu_launch", "ophip_gelu_destroy",
    "ophip_add_create", "ophip_add_scheme", "ophip_add_launch", "ophip_add_destroy", "ophip_add_plan",
    "ophip_add_rows_create", "ophip_add_rows_scheme", "ophip_add_rows_launch", "ophip_add_rows_destroy",
    "ophip_conv_create", "ophip_conv_scheme", "ophip_conv_launch", "ophip_conv_destroy",
]

_lib = None


def lib():
    """The loaded shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libophip.so is not built: run __graft_entry__.build() or make -C operators-rs_amd/csrc")
        L = ctypes.CDLL(LIB_PATH)
        L.ophip_last_error.restype = ctypes.c_char_p
        L.ophip_status_name.restype = ctypes.c_char_p
        L.ophip_dtype_nbytes.restype = ctypes.c_size_t
        L.ophip_dtype_nbytes.argtypes = [ctypes.c_uint64]
        L.ophip_sample_args_argmax.restype = SampleArgsStruct
        L.ophip_offset_calculator_create.restype = ctypes.c_void_p
        L.ophip_offset_calculator_create.argtypes = [ctypes.c_size_t]
        L.ophip_offset_calculator_destroy.argtypes = [ctypes.c_void_p]
        L.ophip_offset_calculator_put.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t]
        L.ophip_offset_calculator_take.argtypes = [ctypes.c_void_p, ctypes.c_size_t,
                                                   ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
        L.ophip_device_release.argtypes = [ctypes.c_void_p]
        L.ophip_device_release.restype = None
        L.ophip_device_retain.argtypes = [ctypes.c_void_p]
        L.ophip_device_retain.restype = None
        L.ophip_mem_pool_destroy.argtypes = [ctypes.c_void_p]
        L.ophip_mem_pool_destroy.restype = None
        for op in ("rms_norm", "rope", "fused_softmax", "rearrange", "swiglu", "random_sample", "mat_mul"):
            getattr(L, "ophip_%s_destroy" % op).argtypes = [ctypes.c_void_p]
            getattr(L, "ophip_%s_destroy" % op).restype = None
        _lib = L
    return _lib


def dtype_nbytes(d):
    return {dt.F16: 2, dt.BF16: 2, dt.F32: 4, dt.F64: 8, dt.U8: 1, dt.U16: 2, dt.U32: 4, dt.U64: 8, dt.I8: 1,
            dt.I16: 2, dt.I32: 4, dt.I64: 8, dt.BOOL: 1, dt.KVPAIR: 8}[int(d)]


def _check(code, launch=False):
    if code != 0:
        info = lib().ophip_last_error().decode()
        raise (LaunchError if launch else SchemeError)(code, info)


def device_count():
    return lib().ophip_device_count()


class DevMem:
    """A device allocation owned by python (``cuda::DevMem`` in the reference's tests)."""

    def __init__(self, gpu, size):
        self.gpu = gpu
        self.size = int(size)
        p = ctypes.c_void_p()
        _check(lib().ophip_malloc(gpu.handle, ctypes.c_size_t(self.size), ctypes.byref(p)))
        self.ptr = p.value or 0

    def free(self):
        if self.ptr:
            lib().ophip_free(self.gpu.handle, ctypes.c_void_p(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self, gpu):
        self.gpu = gpu
        s = ctypes.c_void_p()
        _check(lib().ophip_stream_create(gpu.handle, ctypes.byref(s)))
        self.handle = s
        qa = _QueueAlloc()
        _check(lib().ophip_queue_alloc_from_stream(gpu.handle, s, ctypes.byref(qa)))
        self.queue_alloc = qa  # `impl QueueAlloc for Stream`

    def synchronize(self):
        _check(lib().ophip_stream_synchronize(self.gpu.handle, self.handle))

    def begin_capture(self):
        """Record the launches that follow on this stream instead of running them."""
        _check(lib().ophip_stream_begin_capture(self.gpu.handle, self.handle))

    def end_capture(self):
        g = ctypes.c_void_p()
        _check(lib().ophip_stream_end_capture(self.gpu.handle, self.handle, ctypes.byref(g)))
        return Graph(self.gpu, g)

    def destroy(self):
        if self.handle is not None:
            lib().ophip_stream_destroy(self.gpu.handle, self.handle)
            self.handle = None


class Graph:
    """A recorded launch sequence (hipGraphExec_t)."""

    def __init__(self, gpu, handle):
        self.gpu, self.handle = gpu, handle

    def launch(self, stream):
        _check(lib().ophip_graph_launch(self.gpu.handle, self.handle, stream.handle), launch=True)

    def destroy(self):
        if self.handle is not None:
            lib().ophip_graph_destroy(self.gpu.handle, self.handle)
            self.handle = None


class Event:
    def __init__(self, gpu):
        self.gpu = gpu
        e = ctypes.c_void_p()
        _check(lib().ophip_event_create(gpu.handle, ctypes.byref(e)))
        self.handle = e

    def record(self, stream):
        _check(lib().ophip_event_record(self.gpu.handle, self.handle, stream.handle))

    def synchronize(self):
        _check(lib().ophip_event_synchronize(self.gpu.handle, self.handle))

    def elapsed_ms(self, later):
        ms = ctypes.c_float()
        _check(lib().ophip_event_elapsed_ms(self.gpu.handle, self.handle, later.handle, ctypes.byref(ms)))
        return ms.value


class StreamMemPool:
    """handle/cuda/alloc.rs StreamMemPool: put() slabs, then use as a QueueAlloc."""

    def __init__(self, gpu, stream):
        self.gpu = gpu
        self.stream = stream
        p = ctypes.c_void_p()
        _check(lib().ophip_mem_pool_create(gpu.handle, stream.handle, ctypes.byref(p)))
        self.handle = p
        qa = _QueueAlloc()
        _check(lib().ophip_mem_pool_queue_alloc(p, ctypes.byref(qa)))
        self.queue_alloc = qa

    def put(self, size):
        _check(lib().ophip_mem_pool_put(self.handle, ctypes.c_size_t(size)))

    def destroy(self):
        if self.handle is not None:
            lib().ophip_mem_pool_destroy(self.handle)
            self.handle = None


class OffsetCalculator:
    """common/calculator.rs OffsetCalculator (host only)."""

    def __init__(self, alignment):
        self.handle = ctypes.c_void_p(lib().ophip_offset_calculator_create(alignment))

    def put(self, start, end):
        lib().ophip_offset_calculator_put(self.handle, start, end)

    def take(self, size):
        s, e = ctypes.c_size_t(), ctypes.c_size_t()
        ok = lib().ophip_offset_calculator_take(self.handle, size, ctypes.byref(s), ctypes.byref(e))
        return (s.value, e.value) if ok else None

    def __del__(self):
        try:
            lib().ophip_offset_calculator_destroy(self.handle)
        except Exception:
            pass


class Gpu:
    """The hardware handle (``Gpu`` of handle/cuda/mod.rs)."""

    def __init__(self, ordinal=0, config=None):
        h = ctypes.c_void_p()
        cfg = None
        if config is not None:
            cfg = (ctypes.c_size_t * 3)(*config)
        _check(lib().ophip_device_create(int(ordinal), cfg, ctypes.byref(h)))
        self.handle = h

    @classmethod
    def init(cls):
        """``Gpu::init()``: None when no device is present."""
        if device_count() == 0:
            return None
        return cls(0)

    def info(self):
        i = DeviceInfo()
        _check(lib().ophip_device_get_info(self.handle, ctypes.byref(i)))
        return i

    def stream(self):
        return Stream(self)

    def event(self):
        return Event(self)

    def time_next_launch(self, stream, start, stop):
        """The next kernel launched on `stream` by this thread records its own begin / end into the two events."""
        _check(lib().ophip_time_next_launch(self.handle, stream.handle, start.handle, stop.handle))

    def malloc(self, size):
        return DevMem(self, size)

    def from_host(self, array, stream=None):
        """Upload a numpy array's bytes (contiguous copy of its buffer)."""
        a = np.ascontiguousarray(array)
        mem = DevMem(self, max(a.nbytes, 1))
        if a.nbytes:
            _check(lib().ophip_memcpy_h2d(self.handle, ctypes.c_void_p(mem.ptr), a.ctypes.data_as(ctypes.c_void_p),
                                          ctypes.c_size_t(a.nbytes), stream.handle if stream else None))
        return mem

    def upload(self, mem, array, offset=0, stream=None):
        a = np.ascontiguousarray(array)
        if a.nbytes:
            _check(lib().ophip_memcpy_h2d(self.handle, ctypes.c_void_p(mem.ptr + offset),
                                          a.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(a.nbytes),
                                          stream.handle if stream else None))

    def to_host(self, mem_or_ptr, dtype, count, offset=0, stream=None):
        out = np.empty(count, dtype=dtype)
        ptr = mem_or_ptr.ptr if isinstance(mem_or_ptr, DevMem) else int(mem_or_ptr)
        if out.nbytes:
            _check(lib().ophip_memcpy_d2h(self.handle, out.ctypes.data_as(ctypes.c_void_p),
                                          ctypes.c_void_p(ptr + offset), ctypes.c_size_t(out.nbytes),
                                          stream.handle if stream else None))
            if stream is not None:
                stream.synchronize()
        return out

    def memset(self, mem, value, size=None, stream=None, offset=0):
        _check(lib().ophip_memset(self.handle, ctypes.c_void_p(mem.ptr + offset), int(value),
                                  ctypes.c_size_t(mem.size - offset if size is None else size),
                                  stream.handle if stream else None))

    def release(self):
        if self.handle is not None:
            lib().ophip_device_release(self.handle)
            self.handle = None


def _qa(queue_alloc):
    qa = getattr(queue_alloc, "queue_alloc", queue_alloc)
    return ctypes.byref(qa)


class _Operator:
    NAME = None

    def __init__(self, node):
        self.node = node
        h = ctypes.c_void_p()
        _check(getattr(lib(), "ophip_%s_create" % self.NAME)(node.handle, ctypes.byref(h)))
        self.handle = h

    def scheme(self, args, max_workspace_size=0):
        ws = ctypes.c_size_t(0)
        _check(getattr(lib(), "ophip_%s_scheme" % self.NAME)(self.handle, ctypes.byref(args.c()),
                                                             ctypes.c_size_t(max_workspace_size), ctypes.byref(ws)))
        return ws.value

    def launch(self, args, workspace, queue_alloc):
        """workspace: None, a DevMem, or a (ptr, len) pair."""
        if workspace is None:
            wp, wl = None, 0
        elif isinstance(workspace, DevMem):
            wp, wl = ctypes.c_void_p(workspace.ptr), workspace.size
        else:
            wp, wl = ctypes.c_void_p(workspace[0]), workspace[1]
        _check(getattr(lib(), "ophip_%s_launch" % self.NAME)(self.handle, ctypes.byref(args.c()), wp,
                                                             ctypes.c_size_t(wl), _qa(queue_alloc)), launch=True)

    def destroy(self):
        if self.handle is not None:
            getattr(lib(), "ophip_%s_destroy" % self.NAME)(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def _p(ptr):
    if ptr is None:
        return None
    if isinstance(ptr, DevMem):
        return ptr.ptr
    return int(ptr)


class RmsNormArgs:
    """rms_norm/args.rs:7-15"""

    def __init__(self, y_layout, y_base, x_layout, x_base, w_layout, w_base, epsilon):
        self.__dict__.update(locals())

    def c(self):
        return _RmsNormArgs(self.y_layout.c(), _p(self.y_base), self.x_layout.c(), _p(self.x_base),
                            self.w_layout.c(), _p(self.w_base), self.epsilon)


class RopeArgs:
    """rope/args.rs:8-18"""

    def __init__(self, t_layout, t_base, p_layout, p_base, sin_layout, sin_base, cos_layout, cos_base, theta):
        self.__dict__.update(locals())

    def c(self):
        return _RopeArgs(self.t_layout.c(), _p(self.t_base), self.p_layout.c(), _p(self.p_base),
                         self.sin_layout.c(), _p(self.sin_base), self.cos_layout.c(), _p(self.cos_base), self.theta)


class AttnMask:
    NONE, CAUSAL = 0, 1


class FusedSoftmaxArgs:
    """fuesd_softmax/args.rs:5-9"""

    def __init__(self, att_mask, att_layout, att_base):
        self.__dict__.update(locals())

    def c(self):
        return _SoftmaxArgs(self.att_mask, self.att_layout.c(), _p(self.att_base))


class RearrangeArgs:
    """rearrange/args.rs:12-17"""

    def __init__(self, dst_layout, dst_base, src_layout, src_base):
        self.__dict__.update(locals())

    def c(self):
        return _RearrangeArgs(self.dst_layout.c(), _p(self.dst_base), self.src_layout.c(), _p(self.src_base))


class SwigluArgs:
    """swiglu/args.rs:7-12"""

    def __init__(self, gate_layout, gate_base, up_layout, up_base):
        self.__dict__.update(locals())

    def c(self):
        return _SwigluArgs(self.gate_layout.c(), _p(self.gate_base), self.up_layout.c(), _p(self.up_base))


class SampleArgsError(Exception):
    pass


class SampleArgs:
    """random_sample/args.rs:20-84"""

    def __init__(self, temperature, top_p, top_k):
        out = SampleArgsStruct()
        r = lib().ophip_sample_args_new(ctypes.c_float(temperature), ctypes.c_float(top_p),
                                        ctypes.c_size_t(min(int(top_k), DYN_USIZE)), ctypes.byref(out))
        if r == 1:
            raise SampleArgsError("NegativeTemperature")
        if r == 2:
            raise SampleArgsError("NonPositiveTop")
        self.struct = out

    @classmethod
    def argmax(cls):
        self = cls.__new__(cls)
        self.struct = lib().ophip_sample_args_argmax()
        return self

    def is_argmax(self):
        return self.struct.temperature == 0.0 or self.struct.top_k == 1


class RandomSampleArgs:
    """random_sample/args.rs:9-18"""

    def __init__(self, kv_pair, kv_pair_base, logits, logits_base, indices, indices_base, config, seed):
        self.__dict__.update(locals())

    @classmethod
    def layout(cls, dtype, n):
        """Args::layout (random_sample/args.rs:34-49): null bases, argmax config."""
        unit = dtype_nbytes(dtype)
        cfg = SampleArgs.argmax()
        cfg.struct.top_p = 0.0
        return cls(TensorLayout(dt.KVPAIR, [], []), None, TensorLayout(dtype, [n], [unit]), None,
                   TensorLayout(dt.U32, [n], [4]), None, cfg, 0.0)

    def c(self):
        return _RandomSampleArgs(self.kv_pair.c(), _p(self.kv_pair_base), self.logits.c(), _p(self.logits_base),
                                 self.indices.c(), _p(self.indices_base), self.config.struct, self.seed)


class MatMulArgs:
    """mat_mul/args.rs:11-20"""

    def __init__(self, c_layout, c_base, beta, a_layout, a_base, b_layout, b_base, alpha):
        self.__dict__.update(locals())

    def c(self):
        return _MatMulArgs(self.c_layout.c(), _p(self.c_base), self.beta, self.a_layout.c(), _p(self.a_base),
                           self.b_layout.c(), _p(self.b_base), self.alpha)

    def layout(self):
        """Args::layout (mat_mul/args.rs:64-121) evaluated by the library."""
        out = MatMulLayout()
        _check(lib().ophip_mat_mul_plan(ctypes.byref(self.c()), ctypes.byref(out)))
        return out


class AttentionArgs:
    """attention/args.rs:10-24"""

    def __init__(self, q_layout, q_base, k_layout, k_base, v_layout, v_base, o_layout, o_base, mask):
        self.__dict__.update(locals())

    def c(self):
        return _AttentionArgs(self.q_layout.c(), _p(self.q_base), self.k_layout.c(), _p(self.k_base),
                              self.v_layout.c(), _p(self.v_base), self.o_layout.c(), _p(self.o_base), self.mask)

    @classmethod
    def new_null(cls, mask, dtype, nh, nkvh, seq, att, dh):
        """Args::new_null (attention/args.rs:36-58): shapes only, every stride dynamic."""
        qo = TensorLayout(dtype, [nh, seq, dh], [None] * 3)
        kv = TensorLayout(dtype, [nkvh, att, dh], [None] * 3)
        return cls(qo, None, kv, None, kv, None, qo, None, mask)


class AttnKVCachedArgs:
    """attention_kv_cached/args.rs:8-30; pos = None is dynamic."""

    def __init__(self, q_layout, q_base, k_layout, k_base, v_layout, v_base, o_layout, o_base,
                 k_cache_layout, k_cache_base, v_cache_layout, v_cache_base, mask, pos):
        self.__dict__.update(locals())

    def c(self):
        return _AttnKVCachedArgs(self.q_layout.c(), _p(self.q_base), self.k_layout.c(), _p(self.k_base),
                                 self.v_layout.c(), _p(self.v_base), self.o_layout.c(), _p(self.o_base),
                                 self.k_cache_layout.c(), _p(self.k_cache_base),
                                 self.v_cache_layout.c(), _p(self.v_cache_base), self.mask,
                                 DYN_USIZE if self.pos is None else self.pos)


class LayerNormArgs:
    """layer_norm/args.rs:7-17"""

    def __init__(self, y_layout, y_base, x_layout, x_base, scale_layout, scale_base, bias_layout, bias_base, epsilon):
        self.__dict__.update(locals())

    def c(self):
        return _LayerNormArgs(self.y_layout.c(), _p(self.y_base), self.x_layout.c(), _p(self.x_base),
                              self.scale_layout.c(), _p(self.scale_base), self.bias_layout.c(), _p(self.bias_base),
                              self.epsilon)


class GeluArgs:
    """gelu/args.rs:4-7"""

    def __init__(self, layout, base):
        self.__dict__.update(locals())

    def c(self):
        return _GeluArgs(self.layout.c(), _p(self.base))


class AddArgs:
    """add/args.rs:12-19"""

    def __init__(self, c_layout, c_base, a_layout, a_base, b_layout, b_base):
        self.__dict__.update(locals())

    def c(self):
        return _AddArgs(self.c_layout.c(), _p(self.c_base), self.a_layout.c(), _p(self.a_base),
                        self.b_layout.c(), _p(self.b_base))


class AddRowsArgs:
    """add_rows/args.rs:10-17"""

    def __init__(self, dst_layout, dst_base, src_layout, src_base, idx_layout, idx_base):
        self.__dict__.update(locals())

    def c(self):
        return _AddRowsArgs(self.dst_layout.c(), _p(self.dst_base), self.src_layout.c(), _p(self.src_base),
                            self.idx_layout.c(), _p(self.idx_base))


class ConvArgs:
    """conv/args.rs:7-19"""

    def __init__(self, y_layout, y_base, x_layout, x_base, w_layout, w_base, b_layout, b_base,
                 strides=(1, 1), dilations=(1, 1), pads=(0, 0, 0, 0)):
        self.__dict__.update(locals())

    def c(self):
        return _ConvArgs(self.y_layout.c(), _p(self.y_base), self.x_layout.c(), _p(self.x_base),
                         self.w_layout.c(), _p(self.w_base), self.b_layout.c(), _p(self.b_base),
                         (ctypes.c_size_t * 2)(*self.strides), (ctypes.c_size_t * 2)(*self.dilations),
                         (ctypes.c_size_t * 4)(*self.pads))


class Conv(_Operator):
    NAME = "conv"


class RmsNorm(_Operator):
    NAME = "rms_norm"


class LayerNorm(_Operator):
    NAME = "layer_norm"


class Gelu(_Operator):
    NAME = "gelu"


class Add(_Operator):
    NAME = "add"

    @staticmethod
    def plan(args):
        """Scheme::new (add/args.rs:42-167) evaluated by the library: [idx strides..., c, a, b strides]."""
        nd_in = len(args.c_layout.shape)
        out = (ctypes.c_ssize_t * (1 + 4 * max(nd_in, 1)))()
        nd = ctypes.c_size_t()
        _check(lib().ophip_add_plan(ctypes.byref(args.c()), out, ctypes.byref(nd)))
        return list(out[: 1 + 4 * nd.value])


class AddRows(_Operator):
    NAME = "add_rows"


class Rope(_Operator):
    NAME = "rope"

    @staticmethod
    def build_pos(dtype, nt, seqs, queue_alloc):
        """Rope::build_pos: seqs is a list of (pos, len); returns a device pointer."""
        arr = (_RopeSeq * max(len(seqs), 1))(*[_RopeSeq(p, n) for p, n in seqs])
        out = ctypes.c_void_p()
        _check(lib().ophip_rope_build_pos(ctypes.c_uint64(dtype), ctypes.c_size_t(nt), arr,
                                          ctypes.c_size_t(len(seqs)), _qa(queue_alloc), ctypes.byref(out)))
        return out.value or 0

    @staticmethod
    def build_sincos(dtype, nctx, dh, queue_alloc):
        out = ctypes.c_void_p()
        n = ctypes.c_size_t()
        _check(lib().ophip_rope_build_sincos(ctypes.c_uint64(dtype), ctypes.c_size_t(nctx), ctypes.c_size_t(dh),
                                             _qa(queue_alloc), ctypes.byref(n), ctypes.byref(out)))
        return n.value, (out.value or 0)


class FusedSoftmax(_Operator):
    NAME = "fused_softmax"


class Rearrange(_Operator):
    NAME = "rearrange"

    @staticmethod
    def plan(args):
        """Scheme::new (rearrange/args.rs:35-153) evaluated by the library: the Vec<isize>."""
        nd_in = len(args.dst_layout.shape)
        out = (ctypes.c_ssize_t * (2 + 3 * (nd_in + 1)))()
        nd = ctypes.c_size_t()
        _check(lib().ophip_rearrange_plan(ctypes.byref(args.c()), out, ctypes.byref(nd)))
        return list(out[: 2 + 3 * nd.value])


class Swiglu(_Operator):
    NAME = "swiglu"


class Attention(_Operator):
    NAME = "attention"


class AttnKVCached(_Operator):
    NAME = "attention_kv_cached"


class RandomSample(_Operator):
    NAME = "random_sample"

    def launch_batch(self, args, rows, row_stride, seeds, workspace, queue_alloc):
        """Extension: `rows` rows in one launch (seeds: None or a device pointer to `rows` f32 draws)."""
        if workspace is None:
            wp, wl = None, 0
        elif isinstance(workspace, DevMem):
            wp, wl = ctypes.c_void_p(workspace.ptr), workspace.size
        else:
            wp, wl = ctypes.c_void_p(workspace[0]), workspace[1]
        _check(lib().ophip_random_sample_launch_batch(self.handle, ctypes.byref(args.c()), ctypes.c_size_t(rows),
                                                      ctypes.c_ssize_t(row_stride),
                                                      ctypes.c_void_p(_p(seeds)) if seeds is not None else None,
                                                      wp, ctypes.c_size_t(wl), _qa(queue_alloc)), launch=True)

    @staticmethod
    def build_indices(n, queue_alloc):
        out = ctypes.c_void_p()
        _check(lib().ophip_random_sample_build_indices(ctypes.c_size_t(n), _qa(queue_alloc), ctypes.byref(out)))
        return out.value or 0


def mat_mul_describe(args):
    """MatMul.describe without an operator or a device: the kernel choice for a device of 256 compute units."""
    buf = ctypes.create_string_buffer(96)
    _check(lib().ophip_mat_mul_describe(None, ctypes.byref(args.c()), buf, ctypes.c_size_t(96)))
    return buf.value.decode()


class MatMul(_Operator):
    NAME = "mat_mul"

    def describe(self, args):
        """Name of the kernel family launch() would pick for these arguments (diagnostics)."""
        buf = ctypes.create_string_buffer(96)
        _check(lib().ophip_mat_mul_describe(self.handle, ctypes.byref(args.c()), buf, ctypes.c_size_t(96)))
        return buf.value.decode()

    def launch_static(self, args, stream):
        """The same product with the library's own scratch array: no workspace, no allocator, nothing allocated."""
        _check(lib().ophip_mat_mul_launch_static(self.handle, ctypes.byref(args.c()), stream.handle), launch=True)
