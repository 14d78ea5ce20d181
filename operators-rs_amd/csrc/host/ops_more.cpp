// layer_norm, gelu, add and add_rows on the HIP backend: argument validation as in the
// reference's Args::meta / Scheme::new, kernel selection, asynchronous launch on the
// caller's queue.
#include <algorithm>
#include <string>
#include <vector>

#include "handle.hpp"

using namespace ophip;

namespace {

const char *dt_tag(uint64_t dt) {
    return dt == OPHIP_DT_F16 ? "f16" : dt == OPHIP_DT_BF16 ? "bf16" : dt == OPHIP_DT_F32 ? "f32" : dt == OPHIP_DT_F64 ? "f64" : "?";
}
bool is_float_dt(uint64_t dt) { return dt == OPHIP_DT_F16 || dt == OPHIP_DT_BF16 || dt == OPHIP_DT_F32 || dt == OPHIP_DT_F64; }
// integers by width (signed and unsigned sums are the same bits), bool on its own; null for anything else
const char *int_tag(uint64_t dt) {
    switch (dt) {
        case OPHIP_DT_U8: case OPHIP_DT_I8: return "i8";
        case OPHIP_DT_U16: case OPHIP_DT_I16: return "i16";
        case OPHIP_DT_U32: case OPHIP_DT_I32: return "i32";
        case OPHIP_DT_U64: case OPHIP_DT_I64: return "i64";
        case OPHIP_DT_BOOL: return "bool";
        default: return nullptr;
    }
}

}  // namespace

// ============================================================= layer_norm ===
// Args::meta: layer_norm/args.rs:26-55.  The CUDA backend only takes d that is a multiple of
// the warp size (layer_norm/cuda/mod.rs:186-195); this one takes any d.

struct ophip_layer_norm : OpBase {
    using OpBase::OpBase;
};

namespace {

struct LayerNormMeta {
    uint64_t dt_a, dt_w;
    size_t n, d;
};

LayerNormMeta layer_norm_meta(const ophip_layer_norm_args &a) {
    expect_rank(a.y_layout, "y", 2);
    expect_rank(a.x_layout, "x", 2);
    expect_rank(a.scale_layout, "scale", 1);
    expect_rank(a.bias_layout, "bias", 1);
    LayerNormMeta m;
    m.dt_a = type_distinct({a.y_layout.dt, a.x_layout.dt});
    m.dt_w = type_distinct({a.scale_layout.dt, a.bias_layout.dt});
    m.n = dim_distinct({a.y_layout.shape[0], a.x_layout.shape[0]});
    m.d = dim_distinct({a.y_layout.shape[1], a.x_layout.shape[1], a.scale_layout.shape[0], a.bias_layout.shape[0]});
    return m;
}

}  // namespace

extern "C" int ophip_layer_norm_create(ophip_device *dev, ophip_layer_norm **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_layer_norm(dev);
    });
}
extern "C" void ophip_layer_norm_destroy(ophip_layer_norm *op) { delete op; }

extern "C" int ophip_layer_norm_scheme(ophip_layer_norm *, const ophip_layer_norm_args *args, size_t, size_t *ws) {
    return guard([&] {
        if (!args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        (void)layer_norm_meta(*args);
    });
}

extern "C" int ophip_layer_norm_launch(const ophip_layer_norm *op, const ophip_layer_norm_args *args, void *, size_t,
                                       const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const LayerNormMeta m = layer_norm_meta(*args);
        const size_t n = static_of(m.n), d = static_of(m.d);
        const ptrdiff_t nsy = static_of(args->y_layout.strides[0]), dsy = static_of(args->y_layout.strides[1]);
        const ptrdiff_t nsx = static_of(args->x_layout.strides[0]), dsx = static_of(args->x_layout.strides[1]);
        const ptrdiff_t dss = static_of(args->scale_layout.strides[0]), dsb = static_of(args->bias_layout.strides[0]);
        const bool f64 = m.dt_a == OPHIP_DT_F64 && m.dt_w == OPHIP_DT_F64;
        // The pairs with vector kernels: the CPU backend's (layer_norm/common_cpu/mod.rs:94-97), and bf16 rows with bf16
        // or f32 parameters.  The CUDA backend compiles a kernel for any pair of named types
        // (layer_norm/cuda/mod.rs:158-159): every other pairing of f16 / bf16 / f32 runs on the element-wise kernel;
        // f64 mixed with a narrower type and non-floating types are refused.
        const bool tuned = (m.dt_a == OPHIP_DT_F16 && (m.dt_w == OPHIP_DT_F16 || m.dt_w == OPHIP_DT_F32)) ||
                           (m.dt_a == OPHIP_DT_BF16 && (m.dt_w == OPHIP_DT_BF16 || m.dt_w == OPHIP_DT_F32)) ||
                           (m.dt_a == OPHIP_DT_F32 && m.dt_w == OPHIP_DT_F32);
        auto narrow = [](uint64_t dt) { return dt == OPHIP_DT_F16 || dt == OPHIP_DT_BF16 || dt == OPHIP_DT_F32; };
        if (!((narrow(m.dt_a) && narrow(m.dt_w)) || f64))
            throw type_not_support("layer_norm supports rows and parameters of f16, bf16 or f32 in any pairing, and (f64, f64)");
        const ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(m.dt_a), wunit = (ptrdiff_t)ophip_dtype_nbytes(m.dt_w);
        if (dsy != unit || dsx != unit || dss != wunit || dsb != wunit)
            throw strides_not_support("layer_norm needs contiguous inner dimensions");
        if (nsy % unit != 0 || nsx % unit != 0) throw strides_not_support("misaligned strides");
        if (n == 0 || d == 0) return;
        if (n > 0x7fffffffu || d > 0x7fffffffu) throw shape_not_support("layer_norm dimension too large");

        LayerNormParams p{};
        p.y = args->y_base;
        p.x = args->x_base;
        p.scale = args->scale_base;
        p.bias = args->bias_base;
        p.nsy = nsy;
        p.nsx = nsx;
        p.n = (uint32_t)n;
        p.d = (uint32_t)d;
        p.epsilon = args->epsilon;
        const std::string base = std::string("layer_norm_") + dt_tag(m.dt_a) + "_" + dt_tag(m.dt_w);
        const size_t vec_elems = 16 / (size_t)unit;
        const bool vec = tuned && d % vec_elems == 0 && aligned16(p.y) && aligned16(p.x) && aligned16(p.scale) &&
                         aligned16(p.bias) && mult16(nsy) && mult16(nsx);
        if (!p.y || !p.x || !p.scale || !p.bias) throw args_not_support("null base address");
        op->dev->make_current();
        if (!vec) {
            launch(op->dev->kernel("layer_norm", (base + "_scalar").c_str()), Dim3{(unsigned)n}, Dim3{256}, 0,
                   stream_of(qa), p);
            return;
        }
        // group width: 8 vectors per thread fit in registers; widen the group when there are too
        // few rows to occupy the machine with one wave per row
        const size_t nvec = d / vec_elems;
        unsigned G = nvec <= 64 * 8 ? 64 : nvec <= 256 * 8 ? 256 : 1024;
        while (G < 1024 && n * (G / 64) < 2048 && nvec >= 4 * (size_t)G) G *= 4;
        const unsigned cus = (unsigned)op->dev->props.multiProcessorCount;
        if (G == 64 && unit == 2 && d <= 4096 && n >= (size_t)cus * 64 &&
            n * d * (size_t)unit >= ((size_t)32 << 20)) {
            // many rows and more bytes than the L2s hold: persistent workgroups (four per CU: 32 KiB
            // of LDS each for scale and bias) whose waves stream rows
            // (8 / 4 / 2 rows of up to 512 / 1024 / 2048 elements per wave and trip)
            const char *tail = nvec <= 64 ? "_rows_s1" : nvec <= 128 ? "_rows_s2" : nvec <= 256 ? "_rows_s4" : "_rows";
            launch(op->dev->kernel("layer_norm", (base + tail).c_str()), Dim3{cus * 4}, Dim3{256}, 0, stream_of(qa), p);
            return;
        }
        if (unit == 2 && d > 4096 && d <= 8192 && n >= (size_t)cus * 32 && n * d * (size_t)unit >= ((size_t)32 << 20)) {
            // the same for rows of 4097 .. 8192 elements: 16 vectors per lane, 64 KiB of LDS, two workgroups per CU
            launch(op->dev->kernel("layer_norm", (base + "_rows16").c_str()), Dim3{cus * 2}, Dim3{256}, 0, stream_of(qa), p);
            return;
        }
        const unsigned block = G < 256 ? 256 : G, rpb = block / G;
        const std::string name = base + (G == 64 ? "_g64" : G == 256 ? "_g256" : "_g1024");
        launch(op->dev->kernel("layer_norm", name.c_str()), Dim3{ceil_div(n, rpb)}, Dim3{block}, 0, stream_of(qa), p);
    });
}

// =================================================================== gelu ===
// Args::meta: gelu/args.rs:24-36; launch checks: gelu/cuda/mod.rs:52-95.

struct ophip_gelu : OpBase {
    using OpBase::OpBase;
};

extern "C" int ophip_gelu_create(ophip_device *dev, ophip_gelu **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_gelu(dev);
    });
}
extern "C" void ophip_gelu_destroy(ophip_gelu *op) { delete op; }

extern "C" int ophip_gelu_scheme(ophip_gelu *, const ophip_gelu_args *args, size_t, size_t *ws) {
    return guard([&] {
        if (!args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        expect_rank(args->layout, "layout", 2);
    });
}

extern "C" int ophip_gelu_launch(const ophip_gelu *op, const ophip_gelu_args *args, void *, size_t,
                                 const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        expect_rank(args->layout, "layout", 2);
        const uint64_t dt = args->layout.dt;
        const size_t n = static_of(args->layout.shape[0]), d = static_of(args->layout.shape[1]);
        const ptrdiff_t sn = static_of(args->layout.strides[0]), sd = static_of(args->layout.strides[1]);
        // (bf16: in neither backend of the reference; the f16 kernels on bf16 elements)
        if (!is_float_dt(dt)) throw type_not_support("gelu supports f16, bf16, f32 and f64");
        const ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(dt);
        if (sd != unit) throw strides_not_support("gelu needs a contiguous inner dimension");
        if (sn % unit != 0) throw strides_not_support("misaligned strides");
        if (n == 0 || d == 0) return;
        if (n > 0x7fffffffu || d > 0x7fffffffu) throw shape_not_support("gelu dimension too large");
        GeluParams p{};
        p.base = args->base;
        p.sn = sn;
        p.n = (uint32_t)n;
        p.d = (uint32_t)d;
        // rows that follow each other in memory are one long row: a row's vectors seldom fill whole workgroups
        // (11008 columns are 5.4 of them; [16384, 11008]: 80 -> 88 % of 8 TB/s)
        if (sn == (ptrdiff_t)d * unit && n * d <= 0x7fffffffu) {
            p.d = (uint32_t)(n * d);
            p.n = 1;
        }
        const bool vec = (dt == OPHIP_DT_F16 || dt == OPHIP_DT_BF16) && p.d % 8 == 0 && aligned16(p.base) && mult16(sn);
        const size_t items = vec ? p.d / 8 : p.d;
        const unsigned gx = (unsigned)std::min<size_t>(ceil_div(items, 256), (size_t)1 << 22);
        const unsigned gy = (unsigned)std::min<size_t>(p.n, 65535);
        const std::string name = std::string("gelu_") + dt_tag(dt) + (vec ? "_vec" : "_scalar");
        if (!p.base) throw args_not_support("null base address");
        op->dev->make_current();
        launch(op->dev->kernel("gelu", name.c_str()), Dim3{gx, gy}, Dim3{256}, 0, stream_of(qa), p);
    });
}

// ==================================================================== add ===
// Scheme::new: add/args.rs:42-167.

struct ophip_add : OpBase {
    using OpBase::OpBase;
};

namespace {

struct AddDim {
    size_t d;
    ptrdiff_t c, a, b;
};

struct AddScheme {
    uint64_t dt;
    std::vector<AddDim> dims;  // merged, in visiting order
    size_t count() const {
        size_t n = 1;
        for (const AddDim &x : dims) n *= x.d;
        return n;
    }
};

AddScheme add_scheme(const ophip_add_args &args) {
    const ophip_tensor_layout &c = args.c_layout, &a = args.a_layout, &b = args.b_layout;
    AddScheme s;
    s.dt = type_distinct({c.dt, a.dt, b.dt});
    const size_t ndim = c.ndim;
    expect_arrays(c);
    expect_arrays(a);
    expect_arrays(b);
    if (a.ndim != ndim || b.ndim != ndim)
        throw rank_mismatch("c.ndim = " + std::to_string(c.ndim) + ", a.ndim = " + std::to_string(a.ndim) +
                            ", b.ndim = " + std::to_string(b.ndim));
    for (size_t i = 0; i < ndim; ++i) {
        const size_t d = static_of(c.shape[i]), da = static_of(a.shape[i]), db = static_of(b.shape[i]);
        const ptrdiff_t sc = static_of(c.strides[i]), sa = static_of(a.strides[i]), sb = static_of(b.strides[i]);
        if (da != d || db != d) throw shape_mismatch("c, a and b differ in shape");
        if (d != 1) {  // dimensions of length 1 are dropped
            if (sc == 0) throw shape_not_support("Reducing is not allowed for add");
            s.dims.push_back({d, sc, sa, sb});
        }
    }
    auto mag = [](ptrdiff_t v) { return v < 0 ? -v : v; };
    std::sort(s.dims.begin(), s.dims.end(), [&](const AddDim &x, const AddDim &y) {
        if (mag(x.c) != mag(y.c)) return mag(x.c) > mag(y.c);
        if (mag(x.a) != mag(y.a)) return mag(x.a) > mag(y.a);
        if (mag(x.b) != mag(y.b)) return mag(x.b) > mag(y.b);
        return x.d < y.d;
    });
    // merge neighbours that continue each other in all three tensors
    for (size_t i = s.dims.size(); i-- > 1;) {
        AddDim &f = s.dims[i - 1], &bk = s.dims[i];
        const ptrdiff_t d = (ptrdiff_t)bk.d;
        if (bk.c * d == f.c && bk.a * d == f.a && bk.b * d == f.b) {
            f = AddDim{bk.d * f.d, bk.c, bk.a, bk.b};
            bk = AddDim{1, 0, 0, 0};
        }
    }
    s.dims.erase(std::remove_if(s.dims.begin(), s.dims.end(), [](const AddDim &x) { return x.d == 1; }), s.dims.end());
    return s;
}

}  // namespace

extern "C" int ophip_add_create(ophip_device *dev, ophip_add **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_add(dev);
    });
}
extern "C" void ophip_add_destroy(ophip_add *op) { delete op; }

// add/cuda/mod.rs:36-47: only the data types are looked at
extern "C" int ophip_add_scheme(ophip_add *, const ophip_add_args *args, size_t, size_t *ws) {
    return guard([&] {
        if (!args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        (void)type_distinct({args->c_layout.dt, args->a_layout.dt, args->b_layout.dt});
    });
}

extern "C" int ophip_add_plan(const ophip_add_args *args, ptrdiff_t *out, size_t *ndim_out) {
    return guard([&] {
        if (!args || !out || !ndim_out) throw args_not_support("null argument");
        const AddScheme s = add_scheme(*args);
        const size_t nd = s.dims.size();
        *ndim_out = nd;
        out[nd] = 1;
        for (size_t i = nd; i-- > 0;) out[i] = (ptrdiff_t)s.dims[i].d * out[i + 1];
        for (size_t i = 0; i < nd; ++i) {
            out[1 + nd + i] = s.dims[i].c;
            out[1 + 2 * nd + i] = s.dims[i].a;
            out[1 + 3 * nd + i] = s.dims[i].b;
        }
    });
}

extern "C" int ophip_add_launch(const ophip_add *op, const ophip_add_args *args, void *, size_t,
                                const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        AddScheme s = add_scheme(*args);
        // (bf16, integers, bool: no CPU kernel in the reference, but its CUDA backend adds any named type,
        // add/cuda/mod.rs:105-123)
        if (!is_float_dt(s.dt) && !int_tag(s.dt)) throw type_not_support("add supports the float, integer and bool types");
        if (s.dims.size() > OPHIP_REARRANGE_MAXD)
            throw rank_not_support("add supports at most " + std::to_string(OPHIP_REARRANGE_MAXD) +
                                   " non-mergeable dimensions");
        const size_t unit = ophip_dtype_nbytes(s.dt);
        for (const AddDim &x : s.dims)
            if (x.c % (ptrdiff_t)unit || x.a % (ptrdiff_t)unit || x.b % (ptrdiff_t)unit)
                throw strides_not_support("misaligned strides");
        if (s.count() == 0) return;
        AddParams p{};
        p.c = args->c_base;
        p.a = args->a_base;
        p.b = args->b_base;
        // 16-byte vectors along the innermost dimension when it is contiguous in all three tensors
        bool vec = false;
        const size_t per = 16 / unit;
        if (!s.dims.empty()) {
            AddDim &in = s.dims.back();
            vec = is_float_dt(s.dt) && s.dt != OPHIP_DT_F64 && in.c == (ptrdiff_t)unit && in.a == (ptrdiff_t)unit && in.b == (ptrdiff_t)unit && in.d % per == 0 &&
                  aligned16(p.c) && aligned16(p.a) && aligned16(p.b);
            for (size_t i = 0; vec && i + 1 < s.dims.size(); ++i)
                vec = mult16(s.dims[i].c) && mult16(s.dims[i].a) && mult16(s.dims[i].b);
            if (vec) in = AddDim{in.d / per, 16, 16, 16};
        }
        const size_t total = s.count();
        if (total > 0x7fffffffu) throw shape_not_support("add: too many elements");
        p.total = (uint32_t)total;
        p.ndim = (uint32_t)s.dims.size();

        size_t items = 1;  // items per step of dimension i = product of the dimensions after it
        for (size_t i = s.dims.size(); i-- > 0;) {
            p.idx_div[i] = make_fastdiv((uint32_t)items);
            p.c_s[i] = s.dims[i].c;
            p.a_s[i] = s.dims[i].a;
            p.b_s[i] = s.dims[i].b;
            items *= s.dims[i].d;
        }
        // (more output than the caches hold: the build that stores with the non-temporal hint)
        const bool nt = vec && total * 16 >= ((size_t)64 << 20);
        const std::string name = std::string("add_") + (is_float_dt(s.dt) ? dt_tag(s.dt) : int_tag(s.dt)) + (vec ? (nt ? "_vec_nt" : "_vec") : "_scalar");
        const unsigned blocks = (unsigned)std::min<size_t>(ceil_div(total, 256), 1u << 20);
        if (!p.c || !p.a || !p.b) throw args_not_support("null base address");
        op->dev->make_current();
        launch(op->dev->kernel("add", name.c_str()), Dim3{blocks}, Dim3{256}, 0, stream_of(qa), p);
    });
}

// =============================================================== add_rows ===
// Args::meta: add_rows/args.rs:48-81; launch checks: add_rows/cuda/mod.rs:40-118.

struct ophip_add_rows : OpBase {
    using OpBase::OpBase;
};

namespace {

struct AddRowsMeta {
    uint64_t dt, dt_idx;
    size_t batch, m, n, k;
};

AddRowsMeta add_rows_meta(const ophip_add_rows_args &a) {
    AddRowsMeta r;
    r.dt = type_distinct({a.dst_layout.dt, a.src_layout.dt});
    r.dt_idx = a.idx_layout.dt;
    if (!is_unsigned_dtype(r.dt_idx)) throw type_not_support("idx must be unsigned integers");
    expect_rank(a.dst_layout, "dst", 3);
    expect_rank(a.src_layout, "src", 2);
    expect_rank(a.idx_layout, "idx", 2);
    r.batch = dim_distinct({a.dst_layout.shape[0], a.idx_layout.shape[0]});
    r.m = dim_distinct({a.dst_layout.shape[1], a.idx_layout.shape[1]});
    r.n = dim_distinct({a.dst_layout.shape[2], a.src_layout.shape[1]});
    r.k = a.src_layout.shape[0];
    return r;
}

struct AddRowsScalarParams {  // the element-wise kernels' parameter block
    AddRowsParams p;
    int64_t nsd, nss;
};

}  // namespace

extern "C" int ophip_add_rows_create(ophip_device *dev, ophip_add_rows **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_add_rows(dev);
    });
}
extern "C" void ophip_add_rows_destroy(ophip_add_rows *op) { delete op; }

extern "C" int ophip_add_rows_scheme(ophip_add_rows *, const ophip_add_rows_args *args, size_t, size_t *ws) {
    return guard([&] {
        if (!args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        (void)add_rows_meta(*args);
    });
}

extern "C" int ophip_add_rows_launch(const ophip_add_rows *op, const ophip_add_rows_args *args, void *, size_t,
                                     const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const AddRowsMeta r = add_rows_meta(*args);
        const size_t batch = static_of(r.batch), m = static_of(r.m), n = static_of(r.n), k = static_of(r.k);
        const ptrdiff_t bsd = static_of(args->dst_layout.strides[0]), msd = static_of(args->dst_layout.strides[1]),
                        nsd = static_of(args->dst_layout.strides[2]);
        const ptrdiff_t bsi = static_of(args->idx_layout.strides[0]), msi = static_of(args->idx_layout.strides[1]);
        const ptrdiff_t kss = static_of(args->src_layout.strides[0]), nss = static_of(args->src_layout.strides[1]);
        // (bf16, integers, bool: no CPU kernel in the reference, but its CUDA backend compiles one for any named type,
        // add_rows/cuda/mod.rs:135-163)
        if (!is_float_dt(r.dt) && !int_tag(r.dt)) throw type_not_support("add_rows supports the float, integer and bool types");
        if (r.dt_idx != OPHIP_DT_U32 && r.dt_idx != OPHIP_DT_U64) throw type_not_support("idx must be u32 or u64");
        const ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(r.dt), iunit = (ptrdiff_t)ophip_dtype_nbytes(r.dt_idx);
        for (ptrdiff_t st : {bsd, msd, nsd, kss, nss})
            if (st % unit != 0) throw strides_not_support("misaligned strides");
        if (bsi % iunit != 0 || msi % iunit != 0) throw strides_not_support("misaligned index strides");
        if (batch == 0 || m == 0 || n == 0) return;
        if (batch * m > 0x7fffffffu || n > 0x7fffffffu || k > 0xffffffffu)
            throw shape_not_support("add_rows dimension too large");
        AddRowsScalarParams q{};
        AddRowsParams &p = q.p;
        p.dst = args->dst_base;
        p.src = args->src_base;
        p.idx = args->idx_base;
        p.bsd = bsd;
        p.msd = msd;
        p.kss = kss;
        p.bsi = bsi;
        p.msi = msi;
        p.batch = (uint32_t)batch;
        p.m = (uint32_t)m;
        p.n = (uint32_t)n;
        p.k = (uint32_t)k;
        p.idx_is_u64 = r.dt_idx == OPHIP_DT_U64;
        q.nsd = nsd;
        q.nss = nss;
        const bool vec = (r.dt == OPHIP_DT_F16 || r.dt == OPHIP_DT_BF16) && nsd == unit && nss == unit && n % 8 == 0 && aligned16(p.dst) &&
                         aligned16(p.src) && mult16(bsd) && mult16(msd) && mult16(kss);
        const size_t items = vec ? n / 8 : n;
        const unsigned gx = std::min<unsigned>(ceil_div(items, 256), 65535u);
        const unsigned gy = (unsigned)std::min<size_t>(batch * m, 65535);
        if (!p.dst || !p.src || !p.idx) throw args_not_support("null base address");
        op->dev->make_current();
        if (vec) {
            launch(op->dev->kernel("add_rows", r.dt == OPHIP_DT_F16 ? "add_rows_f16_vec" : "add_rows_bf16_vec"), Dim3{gx, gy}, Dim3{256}, 0,
               stream_of(qa), p);
        } else {
            const std::string name = std::string("add_rows_") + (is_float_dt(r.dt) ? dt_tag(r.dt) : int_tag(r.dt)) + "_scalar";
            launch(op->dev->kernel("add_rows", name.c_str()), Dim3{gx, gy}, Dim3{256}, 0, stream_of(qa), q);
        }
    });
}
