"""ctypes loader for the CPU oracle (``oracle.c``).

TEST INFRASTRUCTURE ONLY: the tests, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` use it as the checker.  The HIP backend
never imports this package.

Every wrapper takes numpy arrays (or strided views of them) and passes their
data pointer and byte strides straight to the C function, so non-contiguous
layouts are exercised exactly as the reference's ``Args`` structs describe them.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F16, F32, F64, U32, U64 = 1, 2, 3, 4, 5
_DT = {np.dtype(np.float16): F16, np.dtype(np.float32): F32, np.dtype(np.float64): F64,
       np.dtype(np.uint32): U32, np.dtype(np.uint64): U64}

ERROR_NAMES = {
    0: "Ok", 1: "TypeNotSupport", 2: "TypeMismatch", 3: "RankNotSupport", 4: "RankMismatch",
    5: "ShapeNotSupport", 6: "ShapeMismatch", 7: "StridesNotSupport", 8: "ArgsNotSupport",
    9: "DynamicNotSupport",
}

DYN_USIZE = 2 ** 64 - 1
DYN_ISIZE = 2 ** 63 - 1


class OracleError(Exception):
    def __init__(self, code):
        super().__init__(ERROR_NAMES.get(code, str(code)))
        self.code = code
        self.kind = ERROR_NAMES.get(code, str(code))


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class MMLayout(ctypes.Structure):
    _fields_ = [("ab_swap", ctypes.c_int32), ("a_trans", ctypes.c_int32), ("b_trans", ctypes.c_int32),
                ("_pad", ctypes.c_int32),
                ("batch", ctypes.c_size_t), ("m", ctypes.c_size_t), ("n", ctypes.c_size_t),
                ("k", ctypes.c_size_t),
                ("c_stride", ctypes.c_ssize_t), ("c_ld", ctypes.c_ssize_t),
                ("a_stride", ctypes.c_ssize_t), ("a_ld", ctypes.c_ssize_t),
                ("b_stride", ctypes.c_ssize_t), ("b_ld", ctypes.c_ssize_t)]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_ if k != "_pad"}


class KVPair(ctypes.Structure):
    _fields_ = [("idx", ctypes.c_uint32), ("val", ctypes.c_uint32)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        sz, ss, vp, i, f = ctypes.c_size_t, ctypes.c_ssize_t, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        psz, pss = ctypes.POINTER(sz), ctypes.POINTER(ss)
        L.oracle_set_threads.argtypes = [i]
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = f
        L.oracle_f32_to_f16.argtypes = [f]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_rms_norm.argtypes = [vp, ss, ss, vp, ss, ss, vp, ss, sz, sz, f, i, i]
        L.oracle_rope.argtypes = [vp, ss, ss, ss, vp, ss, sz, sz, sz, f, i, i]
        L.oracle_fused_softmax.argtypes = [vp, ss, ss, ss, sz, sz, sz, i, i]
        L.oracle_rearrange_scheme.argtypes = [sz, psz, psz, pss, pss, sz, pss]
        L.oracle_rearrange_distribute_unit.argtypes = [sz, pss, psz, sz, pss]
        L.oracle_rearrange.argtypes = [vp, vp, sz, psz, pss, pss, sz]
        L.oracle_swiglu.argtypes = [vp, ss, ss, vp, ss, ss, sz, sz, i]
        L.oracle_argmax.argtypes = [ctypes.POINTER(KVPair), vp, sz, i]
        L.oracle_random_sample.argtypes = [ctypes.POINTER(KVPair), vp, sz, i, f, f, sz, f]
        L.oracle_mat_mul_layout.argtypes = [ctypes.POINTER(MMLayout), sz, sz, psz, pss, sz, psz, pss,
                                            sz, psz, pss]
        L.oracle_mat_mul.argtypes = [vp, f, vp, vp, f, ctypes.POINTER(MMLayout), i]
        L.oracle_layer_norm.argtypes = [vp, ss, ss, vp, ss, ss, vp, ss, vp, ss, sz, sz, f, i, i]
        L.oracle_gelu.argtypes = [vp, ss, ss, sz, sz, i]
        L.oracle_add.argtypes = [vp, vp, vp, sz, sz, sz, psz, psz, psz, pss, pss, pss, i, i, i]
        L.oracle_add_rows.argtypes = [vp, ss, ss, ss, vp, ss, ss, vp, ss, ss, sz, sz, sz, sz, i, i]
        _lib = L
    return _lib


def set_threads(n):
    lib().oracle_set_threads(int(n))


def max_threads():
    return lib().oracle_max_threads()


def _check(code):
    if code != 0:
        raise OracleError(code)


def _ptr(a):
    return ctypes.c_void_p(a.__array_interface__["data"][0])


def _usz(vals):
    return (ctypes.c_size_t * max(len(vals), 1))(*[int(v) for v in vals])


def _isz(vals):
    return (ctypes.c_ssize_t * max(len(vals), 1))(*[int(v) for v in vals])


def f32_to_f16_bits(x):
    return lib().oracle_f32_to_f16(float(x))


def f16_bits_to_f32(h):
    return lib().oracle_f16_to_f32(int(h))


def rms_norm(y, x, w, epsilon):
    """y[n,d] <- rms_norm(x[n,d], w[d]); arrays may be strided views."""
    n, d = x.shape
    _check(lib().oracle_rms_norm(_ptr(y), y.strides[0], y.strides[1], _ptr(x), x.strides[0],
                                 x.strides[1], _ptr(w), w.strides[0], n, d, epsilon,
                                 _DT[w.dtype], _DT[x.dtype]))
    return y


def rope(t, pos, theta):
    """In-place rotary embedding on t[nt,nh,dh] with positions pos[nt]."""
    nt, nh, dh = t.shape
    _check(lib().oracle_rope(_ptr(t), t.strides[0], t.strides[1], t.strides[2], _ptr(pos),
                             pos.strides[0], nt, nh, dh, theta, _DT[t.dtype], _DT[pos.dtype]))
    return t


def fused_softmax(att, causal=True):
    """In-place masked softmax on att[nh,seq,att_len]."""
    nh, seq, al = att.shape
    _check(lib().oracle_fused_softmax(_ptr(att), att.strides[0], att.strides[1], att.strides[2],
                                      nh, seq, al, 1 if causal else 0, _DT[att.dtype]))
    return att


def rearrange_scheme(shape, dst_strides, src_strides, elem_size, src_shape=None):
    """The reference's Scheme vector [unit, idx..., dst..., src...] as a python list."""
    nd = len(shape)
    out = (ctypes.c_ssize_t * (2 + 3 * (nd + 1)))()
    r = lib().oracle_rearrange_scheme(nd, _usz(shape), _usz(src_shape if src_shape is not None else shape),
                                      _isz(dst_strides), _isz(src_strides), elem_size, out)
    if r < 0:
        raise OracleError(-r)
    return list(out[: 2 + 3 * r])


def rearrange_distribute_unit(scheme, candidates):
    nd = (len(scheme) - 2) // 3
    out = (ctypes.c_ssize_t * (2 + 3 * (nd + 1)))()
    r = lib().oracle_rearrange_distribute_unit(nd, _isz(scheme), _usz(candidates), len(candidates), out)
    if r < 0:
        raise ValueError("no candidate divides the unit")
    return list(out[: 2 + 3 * r])


def rearrange(dst, src):
    """Strided copy src -> dst (numpy views of equal shape and dtype)."""
    assert dst.shape == src.shape and dst.dtype == src.dtype
    _check(lib().oracle_rearrange(_ptr(dst), _ptr(src), dst.ndim, _usz(dst.shape), _isz(dst.strides),
                                  _isz(src.strides), dst.dtype.itemsize))
    return dst


def rearrange_raw(dst_ptr, src_ptr, shape, dst_strides, src_strides, elem_size):
    _check(lib().oracle_rearrange(ctypes.c_void_p(dst_ptr), ctypes.c_void_p(src_ptr), len(shape),
                                  _usz(shape), _isz(dst_strides), _isz(src_strides), elem_size))


def swiglu(gate, up):
    n, d = gate.shape
    _check(lib().oracle_swiglu(_ptr(gate), gate.strides[0], gate.strides[1], _ptr(up), up.strides[0],
                               up.strides[1], n, d, _DT[gate.dtype]))
    return gate


def argmax(logits):
    """Returns (idx, val_bits) as the reference's KVPair."""
    kv = KVPair()
    assert logits.ndim == 1 and logits.strides[0] == logits.dtype.itemsize
    _check(lib().oracle_argmax(ctypes.byref(kv), _ptr(logits), logits.shape[0], _DT[logits.dtype]))
    return kv.idx, kv.val


def random_sample(logits, temperature, top_p, top_k, seed):
    """Returns (idx, val_bits); argmax when temperature == 0 or top_k == 1."""
    kv = KVPair()
    assert logits.ndim == 1 and logits.strides[0] == logits.dtype.itemsize
    top_k = min(int(top_k), DYN_USIZE)
    _check(lib().oracle_random_sample(ctypes.byref(kv), _ptr(logits), logits.shape[0],
                                      _DT[logits.dtype], temperature, top_p, top_k, seed))
    return kv.idx, kv.val


def mat_mul_layout(elem_size, c, a, b):
    """c, a, b are (shape, byte_strides) pairs; returns MMLayout."""
    out = MMLayout()
    _check(lib().oracle_mat_mul_layout(ctypes.byref(out), elem_size,
                                       len(c[0]), _usz(c[0]), _isz(c[1]),
                                       len(a[0]), _usz(a[0]), _isz(a[1]),
                                       len(b[0]), _usz(b[0]), _isz(b[1])))
    return out


def mat_mul(c, beta, a, b, alpha):
    """c <- alpha * a @ b + beta * c on numpy views (rank 2 or 3, any supported strides)."""
    L = mat_mul_layout(c.dtype.itemsize, (c.shape, c.strides), (a.shape, a.strides), (b.shape, b.strides))
    _check(lib().oracle_mat_mul(_ptr(c), beta, _ptr(a), _ptr(b), alpha, ctypes.byref(L), _DT[c.dtype]))
    return c


def _heads_and_tokens_merge(q):
    """ArrayLayout::merge_be(0, 2) as attention/operator.rs:186 uses it: can q[nh, seq, dh] be
    viewed as [nh * seq, dh]?  (The layout crate, ndarray-layout, is not part of the reference
    tree; a dimension of length 1 is taken to merge with anything.  The choice only decides
    whether q is staged in workspace - the outputs are the same either way.)"""
    nh, seq, _ = q.shape
    return nh == 1 or seq == 1 or q.strides[0] == seq * q.strides[1]


def attention(q, k, v, o, causal=True):
    """The attention composite (attention/operator.rs:143-277) over the CPU restatements:
    q, o [nh, seq, dh]; k, v [nkvh, att, dh] as numpy views.  att = q . k^T / sqrt(dh) per
    kv-head group, masked softmax, q <- att . v, o <- q.  Like the reference, q itself is
    overwritten when its heads and tokens merge into one dimension."""
    nh, seq, dh = q.shape
    nkvh, att, _ = k.shape
    assert nh % nkvh == 0
    group = nh // nkvh
    if _heads_and_tokens_merge(q):
        rows = np.lib.stride_tricks.as_strided(
            q, (nh * seq, dh), (q.strides[0] if seq == 1 else q.strides[1], q.strides[2]))
        qx = np.lib.stride_tricks.as_strided(
            rows, (nkvh, group * seq, dh), (group * seq * rows.strides[0], rows.strides[0], rows.strides[1]))
        q_work = q
    else:
        q_work = np.empty((nh, seq, dh), q.dtype)
        rearrange(q_work, q)
        qx = q_work.reshape(nkvh, group * seq, dh)
    att_buf = np.zeros((nkvh, group * seq, att), q.dtype)
    alpha = float(np.float32(1.0) / np.sqrt(np.float32(dh)))
    mat_mul(att_buf, 0.0, qx, k.transpose(0, 2, 1), alpha)
    fused_softmax(att_buf.reshape(nh, seq, att), causal=causal)
    mat_mul(qx, 0.0, att_buf, v, 1.0)
    if q_work is not o:
        rearrange(o, q_work)
    return o


def attention_kv_cached(q, k, v, o, k_cache, v_cache, pos, causal=True):
    """attention_kv_cached/operator.rs:79-183: k, v [nkvh, seq, dh] are copied into rows
    [pos, pos + seq) of the caches [nkvh, buf, dh], then attention runs over rows
    [0, pos + seq).  Both caches must share one layout (the reference addresses the v-cache
    with the k-cache's strides)."""
    seq = q.shape[1]
    att = pos + seq
    if k_cache.shape[1] < att or v_cache.shape[1] < att:
        raise OracleError(6)  # ShapeMismatch: "Out of cache buffer"
    assert k_cache.strides == v_cache.strides
    rearrange(k_cache[:, pos:att], k)
    rearrange(v_cache[:, pos:att], v)
    return attention(q, k_cache[:, :att], v_cache[:, :att], o, causal=causal)


def layer_norm(y, x, scale, bias, epsilon):
    """y[n,d] <- layer_norm(x[n,d]; scale[d], bias[d]); epsilon is added to the standard deviation."""
    n, d = x.shape
    _check(lib().oracle_layer_norm(_ptr(y), y.strides[0], y.strides[1], _ptr(x), x.strides[0], x.strides[1],
                                   _ptr(scale), scale.strides[0], _ptr(bias), bias.strides[0], n, d,
                                   float(epsilon), _DT[x.dtype], _DT[scale.dtype]))
    return y


def gelu(t):
    """In-place tanh-form gelu on t[n,d]."""
    n, d = t.shape
    _check(lib().oracle_gelu(_ptr(t), t.strides[0], t.strides[1], n, d, _DT[t.dtype]))
    return t


def add(c, a, b):
    """c <- a + b on numpy views of equal shape (any strides; stride 0 in a or b broadcasts)."""
    _check(lib().oracle_add(_ptr(c), _ptr(a), _ptr(b), c.ndim, a.ndim, b.ndim, _usz(c.shape), _usz(a.shape),
                            _usz(b.shape), _isz(c.strides), _isz(a.strides), _isz(b.strides),
                            _DT[c.dtype], _DT[a.dtype], _DT[b.dtype]))
    return c


def add_rows(dst, src, idx):
    """dst[b,m,:] += src[idx[b,m],:]; idx is uint32 or uint64."""
    batch, m, n = dst.shape
    k = src.shape[0]
    _check(lib().oracle_add_rows(_ptr(dst), dst.strides[0], dst.strides[1], dst.strides[2], _ptr(src),
                                 src.strides[0], src.strides[1], _ptr(idx), idx.strides[0], idx.strides[1],
                                 batch, m, n, k, _DT[dst.dtype], _DT[idx.dtype]))
    return dst


def conv(y, x, w, b, strides=(1, 1), dilations=(1, 1), pads=(0, 0, 0, 0)):
    """The conv composite (conv/im2col.rs:85-242) over the CPU restatements: y[n,m,hy,wy] <- bias,
    x unfolded to [n, c*hk*wk, hy*wy] by a strided copy, then y += w . unfolded (mat_mul, beta 1)."""
    if any(pads):
        raise OracleError(8)  # ArgsNotSupport: non-zero padding for im2col is not supported
    n, c, h, wd_ = x.shape
    m, _, hk, wk = w.shape
    _, _, hy, wy = y.shape
    (hs, ws), (hd, wd) = strides, dilations
    hkd, wkd = (hk - 1) * hd + 1, (wk - 1) * wd + 1
    if (h - hkd) % hs or (wd_ - wkd) % ws:
        raise OracleError(7)  # StridesNotSupport: output size not divisible by strides
    as_strided = np.lib.stride_tricks.as_strided
    if not (hy == 1 or wy == 1 or y.strides[2] == wy * y.strides[3]):
        raise OracleError(7)
    c_y = as_strided(y, (n, m, hy * wy), (y.strides[0], y.strides[1], y.strides[2] if wy == 1 else y.strides[3]))
    rearrange(c_y, as_strided(b, (n, m, hy * wy), (0, b.strides[0], 0)))
    unfolded = np.empty((n, c, hk, wk, hy, wy), x.dtype)
    xs = x.strides
    rearrange(unfolded, as_strided(x, unfolded.shape, (xs[0], xs[1], xs[2] * hd, xs[3] * wd, xs[2] * hs, xs[3] * ws)))
    w2 = np.ascontiguousarray(w).reshape(m, c * hk * wk) if not w.flags.c_contiguous else w.reshape(m, c * hk * wk)
    a_w = as_strided(w2, (n, m, c * hk * wk), (0, w2.strides[0], w2.strides[1]))
    mat_mul(c_y, 1.0, a_w, unfolded.reshape(n, c * hk * wk, hy * wy), 1.0)
    return y
