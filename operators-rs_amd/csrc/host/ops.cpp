// rms_norm, rope, fuesd_softmax, rearrange and swiglu on the HIP backend:
// argument validation as in the reference's Args::meta / Scheme::new, kernel
// selection, and asynchronous launch on the caller's queue.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <mutex>

#include "../kernels/params.h"
#include "handle.hpp"

using namespace ophip;

namespace {

const char *dt_tag(uint64_t dt) {
    return dt == OPHIP_DT_F16 ? "f16" : dt == OPHIP_DT_BF16 ? "bf16" : dt == OPHIP_DT_F32 ? "f32" : dt == OPHIP_DT_F64 ? "f64" : "?";
}

}  // namespace

// =============================================================== rms_norm ===
// Args::meta: rms_norm/args.rs:25-49.  Launch-time checks follow
// rms_norm/cuda/mod.rs:49-114 (static shapes, contiguous inner dims).

struct RmsNormMeta {
    uint64_t dt_a, dt_w;
    size_t n, d;
};

static RmsNormMeta rms_norm_meta(const ophip_rms_norm_args &a) {
    expect_rank(a.y_layout, "y", 2);
    expect_rank(a.x_layout, "x", 2);
    expect_rank(a.w_layout, "w", 1);
    RmsNormMeta m;
    m.dt_a = type_distinct({a.y_layout.dt, a.x_layout.dt});
    m.dt_w = a.w_layout.dt;
    m.n = dim_distinct({a.y_layout.shape[0], a.x_layout.shape[0]});
    m.d = dim_distinct({a.y_layout.shape[1], a.x_layout.shape[1], a.w_layout.shape[0]});
    return m;
}

// The pairs with vector kernels: those of the CPU backend (rms_norm/common_cpu/mod.rs:84-90; anything else is `todo!()`
// there) and bf16 activations with bf16 or f32 weights.
static bool rms_norm_tuned_pair(uint64_t dt_a, uint64_t dt_w) {
    return (dt_a == OPHIP_DT_F16 && (dt_w == OPHIP_DT_F16 || dt_w == OPHIP_DT_F32)) ||
           (dt_a == OPHIP_DT_BF16 && (dt_w == OPHIP_DT_BF16 || dt_w == OPHIP_DT_F32)) ||
           (dt_a == OPHIP_DT_F32 && dt_w == OPHIP_DT_F32) || (dt_a == OPHIP_DT_F64 && dt_w == OPHIP_DT_F64);
}
static void rms_norm_check_types(uint64_t dt_a, uint64_t dt_w) {
    // The CUDA backend compiles a kernel for any pair of named types (rms_norm/cuda/mod.rs:117-122): every pair of
    // f16 / bf16 / f32 is taken here (the pairs without a vector kernel on the element-wise one), and (f64, f64); f64
    // mixed with a narrower type, which CUDA would compute in f32, and non-floating types are refused.
    auto narrow = [](uint64_t dt) { return dt == OPHIP_DT_F16 || dt == OPHIP_DT_BF16 || dt == OPHIP_DT_F32; };
    if (!((narrow(dt_a) && narrow(dt_w)) || (dt_a == OPHIP_DT_F64 && dt_w == OPHIP_DT_F64)))
        throw type_not_support("rms_norm supports activations and weights of f16, bf16 or f32 in any pairing, and (f64, f64)");
}

struct RmsKey {
    uint64_t dt_a, dt_w;
    size_t d;
    bool operator==(const RmsKey &o) const { return dt_a == o.dt_a && dt_w == o.dt_w && d == o.d; }
};
struct RmsKeyHash {
    size_t operator()(const RmsKey &k) const { return k.d * 1315423911u ^ (k.dt_a << 8) ^ k.dt_w; }
};
struct RmsScheme {  // kernels for one (dt_a, dt_w, d): a vector variant per group width plus the scalar one
    hipFunction_t g64, g256, g1024, scalar;
    hipFunction_t rows;  // f16 and bf16 activations only: one wave per row over many rows
    hipFunction_t rows_short[3] = {};  // the same, 8 / 4 / 2 rows of up to 512 / 1024 / 2048 elements per wave and trip
    hipFunction_t rows16 = nullptr;  // the same for rows of up to 8192 elements (activations and weights of one two-byte type)
};

struct ophip_rms_norm : OpBase {
    mutable LruCache<RmsKey, RmsScheme, RmsKeyHash> schemes;
    explicit ophip_rms_norm(ophip_device *d) : OpBase(d), schemes(d->config.low_diversity_cache) {}

    RmsScheme scheme_for(const RmsKey &key) const {
        return schemes.get_or_insert(key, [&] {
            const std::string base = std::string("rms_norm_") + dt_tag(key.dt_a) + "_" + dt_tag(key.dt_w);
            RmsScheme s{};
            if (key.dt_a == OPHIP_DT_F64 || !rms_norm_tuned_pair(key.dt_a, key.dt_w)) {  // one kernel only
                s.scalar = dev->kernel("rms_norm", (base + "_scalar").c_str());
                return s;
            }
            s.g64 = dev->kernel("rms_norm", (base + "_g64").c_str());
            s.g256 = dev->kernel("rms_norm", (base + "_g256").c_str());
            s.g1024 = dev->kernel("rms_norm", (base + "_g1024").c_str());
            s.scalar = dev->kernel("rms_norm", (base + "_scalar").c_str());
            s.rows = key.dt_a == OPHIP_DT_F16 || key.dt_a == OPHIP_DT_BF16 ? dev->kernel("rms_norm", (base + "_rows").c_str()) : nullptr;
            if (s.rows && key.dt_w == key.dt_a) s.rows16 = dev->kernel("rms_norm", (base + "_rows16").c_str());
            if (s.rows)
                for (int i = 0; i < 3; ++i) s.rows_short[i] = dev->kernel("rms_norm", (base + "_rows_s" + std::to_string(1 << i)).c_str());
            return s;
        });
    }
};

extern "C" int ophip_rms_norm_create(ophip_device *dev, ophip_rms_norm **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_rms_norm(dev);
    });
}
extern "C" void ophip_rms_norm_destroy(ophip_rms_norm *op) { delete op; }

extern "C" int ophip_rms_norm_scheme(ophip_rms_norm *op, const ophip_rms_norm_args *args, size_t, size_t *ws) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        const RmsNormMeta m = rms_norm_meta(*args);
        const size_t d = static_of(m.d);  // rms_norm/cuda/mod.rs:38-39
        rms_norm_check_types(m.dt_a, m.dt_w);
        op->scheme_for(RmsKey{m.dt_a, m.dt_w, d});
    });
}

extern "C" int ophip_rms_norm_launch(const ophip_rms_norm *op, const ophip_rms_norm_args *args, void *, size_t,
                                     const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const RmsNormMeta m = rms_norm_meta(*args);
        const size_t n = static_of(m.n), d = static_of(m.d);
        const ptrdiff_t nsy = static_of(args->y_layout.strides[0]), dsy = static_of(args->y_layout.strides[1]);
        const ptrdiff_t nsx = static_of(args->x_layout.strides[0]), dsx = static_of(args->x_layout.strides[1]);
        const ptrdiff_t dsw = static_of(args->w_layout.strides[0]);
        rms_norm_check_types(m.dt_a, m.dt_w);
        const ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(m.dt_a);
        if (dsy != unit || dsx != unit || dsw != (ptrdiff_t)ophip_dtype_nbytes(m.dt_w))
            throw strides_not_support("rms_norm needs contiguous inner dimensions");
        if (n == 0 || d == 0) return;
        if (n > 0x7fffffffu || d > 0x7fffffffu) throw shape_not_support("rms_norm dimension too large");
        if (!args->y_base || !args->x_base || !args->w_base) throw args_not_support("rms_norm: null base pointer");

        const RmsScheme s = op->scheme_for(RmsKey{m.dt_a, m.dt_w, d});
        RmsNormParams p{};
        p.y = args->y_base;
        p.x = args->x_base;
        p.w = args->w_base;
        p.nsy = nsy;
        p.nsx = nsx;
        p.n = (uint32_t)n;
        p.d = (uint32_t)d;
        p.epsilon = args->epsilon;

        const size_t vec_elems = 16 / (size_t)unit;
        const bool vec = s.g64 != nullptr && d % vec_elems == 0 && aligned16(p.y) && aligned16(p.x) && aligned16(p.w) && mult16(nsy) &&
                         mult16(nsx);
        op->dev->make_current();
        if (!vec) {
            launch(s.scalar, Dim3{(unsigned)n}, Dim3{256}, 0, stream_of(qa), p);
            return;
        }
        // group width: 8 vectors per thread fit in registers; widen the group when
        // there are too few rows to occupy the machine with one wave per row
        const size_t nvec = d / vec_elems;
        unsigned G = nvec <= 64 * 8 ? 64 : nvec <= 256 * 8 ? 256 : 1024;
        while (G < 1024 && n * (G / 64) < 2048 && nvec >= 4 * (size_t)G) G *= 4;
        const unsigned cus = (unsigned)op->dev->props.multiProcessorCount;
        if (G == 64 && s.rows && n >= (size_t)cus * 64) {
            // enough rows for several per wave: as many waves as stay resident (registers allow
            // 16 per CU with two-byte weights, 12 with f32), each streaming rows with w held in registers
            const unsigned per_cu = m.dt_w == OPHIP_DT_F32 ? 3 : 4;
            hipFunction_t fn = nvec <= 64 ? s.rows_short[0] : nvec <= 128 ? s.rows_short[1] : nvec <= 256 ? s.rows_short[2] : s.rows;
            launch(fn, Dim3{cus * per_cu}, Dim3{256}, 0, stream_of(qa), p);
            return;
        }
        // rows of 4097 .. 8192 two-byte elements, many of them: the same with 16 vectors per lane (a workgroup per row
        // gives [52428, 5120] 62 % of 8 TB/s, this 76 %; [32768, 8192] 69 -> 72 %)
        if (s.rows16 && nvec > 64 * 8 && nvec <= 64 * 16 && n >= (size_t)cus * 32) {
            launch(s.rows16, Dim3{cus * 2}, Dim3{256}, 0, stream_of(qa), p);
            return;
        }
        const unsigned block = G < 256 ? 256 : G, rpb = block / G;
        hipFunction_t fn = G == 64 ? s.g64 : G == 256 ? s.g256 : s.g1024;
        launch(fn, Dim3{ceil_div(n, rpb)}, Dim3{block}, 0, stream_of(qa), p);
    });
}

// =================================================================== rope ===
// Args::meta: rope/args.rs:29-72.  Launch checks: rope/cuda/mod.rs:82-160 and
// rope/common_cpu/mod.rs:98-100.

struct RopeMeta {
    uint64_t dt_t, dt_p;
    size_t nt, dh;
};

static RopeMeta rope_meta(const ophip_rope_args &a) {
    expect_rank(a.t_layout, "t", 3);
    expect_rank(a.p_layout, "p", 1);
    expect_rank(a.sin_layout, "sin", 2);
    expect_rank(a.cos_layout, "cos", 2);
    RopeMeta m;
    m.dt_t = a.t_layout.dt;
    m.dt_p = a.p_layout.dt;
    if (!is_float_dtype(m.dt_t)) throw type_not_support("t must be floating-point numbers");
    if (!is_unsigned_dtype(m.dt_p)) throw type_not_support("p must be unsigned integers");
    m.nt = dim_distinct({a.t_layout.shape[0], a.p_layout.shape[0]});
    m.dh = dim_distinct({a.t_layout.shape[2], a.sin_layout.shape[1], a.cos_layout.shape[1]});
    return m;
}

struct ophip_rope : OpBase {
    hipFunction_t f16_vec, f16_pairs, bf16_vec, bf16_pairs, f32_pairs, f64_pairs, f16_vec_multi, bf16_vec_multi;
    // theta^(k / (dh/2)) of the last (theta, dh) launched: a model has one such pair
    mutable std::mutex den_mu;
    mutable float den_theta = 0.f;
    mutable size_t den_half = 0;
    mutable float den[128];
    void denominators(float theta, size_t half, float *out) const {
        std::lock_guard<std::mutex> lock(den_mu);
        if (den_half != half || den_theta != theta) {
            for (size_t k = 0; k < half; ++k) den[k] = std::pow(theta, (float)k / (float)half);  // powf, as the reference's
            den_theta = theta;
            den_half = half;
        }
        std::memcpy(out, den, half * sizeof(float));
    }
    explicit ophip_rope(ophip_device *d) : OpBase(d) {
        f16_vec = d->kernel("rope", "rope_f16_vec");
        f16_vec_multi = d->kernel("rope", "rope_f16_vec_multi");
        bf16_vec_multi = d->kernel("rope", "rope_bf16_vec_multi");
        f16_pairs = d->kernel("rope", "rope_f16_pairs");
        bf16_vec = d->kernel("rope", "rope_bf16_vec");
        bf16_pairs = d->kernel("rope", "rope_bf16_pairs");
        f32_pairs = d->kernel("rope", "rope_f32_pairs");
        f64_pairs = d->kernel("rope", "rope_f64_pairs");
    }
};

extern "C" int ophip_rope_create(ophip_device *dev, ophip_rope **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_rope(dev);
    });
}
extern "C" void ophip_rope_destroy(ophip_rope *op) { delete op; }

extern "C" int ophip_rope_scheme(ophip_rope *, const ophip_rope_args *args, size_t, size_t *ws) {
    return guard([&] {
        if (!args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        (void)rope_meta(*args);
    });
}

extern "C" int ophip_rope_launch(const ophip_rope *op, const ophip_rope_args *args, void *, size_t,
                                 const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const RopeMeta m = rope_meta(*args);
        // (bf16: in neither backend of the reference; the f16 kernels on bf16 elements)
        if (m.dt_t != OPHIP_DT_F16 && m.dt_t != OPHIP_DT_BF16 && m.dt_t != OPHIP_DT_F32 && m.dt_t != OPHIP_DT_F64)
            throw type_not_support("rope supports f16, bf16, f32 and f64 tokens");
        if (m.dt_p != OPHIP_DT_U32 && m.dt_p != OPHIP_DT_U64) throw type_not_support("rope supports u32 and u64 positions");
        const size_t nt = static_of(m.nt), nh = static_of(args->t_layout.shape[1]), dh = static_of(m.dh);
        const ptrdiff_t st = static_of(args->t_layout.strides[0]), sh = static_of(args->t_layout.strides[1]),
                        sd = static_of(args->t_layout.strides[2]), sp = static_of(args->p_layout.strides[0]);
        const ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(m.dt_t), punit = (ptrdiff_t)ophip_dtype_nbytes(m.dt_p);
        if (sd != unit) throw strides_not_support("rope needs a contiguous head dimension");
        if (sp % punit != 0 || st % unit != 0 || sh % unit != 0) throw strides_not_support("misaligned strides");
        if (nt == 0 || nh == 0 || dh < 2) return;
        if (nt > 0x7fffffffu || nh > 0xffffffu || dh > 0xffffffu) throw shape_not_support("rope dimension too large");
        const size_t smem = (dh / 2) * (m.dt_t == OPHIP_DT_F64 ? 16 : 8);
        if (smem > 64 * 1024) throw shape_not_support("rope head dimension too large");
        if (!args->t_base || !args->p_base) throw args_not_support("null base address");

        RopeParams p{};
        p.t = args->t_base;
        p.pos = args->p_base;
        p.st = st;
        p.sh = sh;
        p.sp = sp;
        p.nt = (uint32_t)nt;
        p.nh = (uint32_t)nh;
        p.dh = (uint32_t)dh;
        p.theta = args->theta;
        p.pos_is_u64 = m.dt_p == OPHIP_DT_U64;
        p.has_den = dh / 2 <= 128;
        if (p.has_den) op->denominators(args->theta, dh / 2, p.den);

        const bool half = m.dt_t == OPHIP_DT_F16 || m.dt_t == OPHIP_DT_BF16;
        const bool vec = half && dh % 8 == 0 && aligned16(p.t) && mult16(st) && mult16(sh);
        // split a token's heads over blockIdx.y when there are few tokens, keeping >= 256 items per block
        const size_t per_head = vec ? dh / 8 : dh / 2;
        size_t max_by = std::max<size_t>(1, nh * per_head / 256);
        size_t want_by = (2048 + nt - 1) / nt;
        size_t by = std::min(std::min(max_by, want_by), nh);
        size_t hpb = (nh + by - 1) / by;
        by = (nh + hpb - 1) / hpb;
        if (by > 65535) throw shape_not_support("too many heads");
        p.heads_per_block = (uint32_t)hpb;
        hipFunction_t fn = m.dt_t == OPHIP_DT_F16    ? (vec ? op->f16_vec : op->f16_pairs)
                           : m.dt_t == OPHIP_DT_BF16 ? (vec ? op->bf16_vec : op->bf16_pairs)
                           : m.dt_t == OPHIP_DT_F32  ? op->f32_pairs
                                                     : op->f64_pairs;
        op->dev->make_current();
        // many tokens of few vectors each (8 heads of 128, 16 of 64: 128 vectors; twice that up to 64 K tokens): several
        // consecutive tokens per workgroup, about 1024 vectors.  [204800, 8, 128] 49 -> 70 % of 8 TB/s, [8192, 16, 128]
        // 71 -> 79 %; tokens of 512 vectors gain nothing, and beyond 64 K tokens those of 256 lose 4 points.
        const size_t per_token = nh * (dh / 8), tpb = per_token ? std::min<size_t>(8, 1024 / std::max<size_t>(per_token, 1)) : 0;
        if (vec && by == 1 && nt >= 4096 && (tpb == 8 || (tpb >= 4 && nt < 65536))) {
            p.tokens_per_block = (uint32_t)tpb;
            launch(m.dt_t == OPHIP_DT_F16 ? op->f16_vec_multi : op->bf16_vec_multi, Dim3{(unsigned)((nt + tpb - 1) / tpb)}, Dim3{256}, smem * tpb,
                   stream_of(qa), p);
            return;
        }
        launch(fn, Dim3{(unsigned)nt, (unsigned)by}, Dim3{256}, smem, stream_of(qa), p);
    });
}

// fill_pos (rope/mod.rs:46-58) + upload (rope/cuda/mod.rs:36-56)
extern "C" int ophip_rope_build_pos(uint64_t dt, size_t nt, const ophip_rope_seq *seqs, size_t nseq,
                                    const ophip_queue_alloc *qa, void **out) {
    return guard([&] {
        if (!qa || !qa->alloc || !out) throw args_not_support("null argument");
        if (dt != OPHIP_DT_U32 && dt != OPHIP_DT_U64) throw type_not_support("positions must be u32 or u64");
        const size_t unit = ophip_dtype_nbytes(dt);
        std::vector<unsigned char> host(unit * nt, 0);
        size_t o = 0;
        for (size_t s = 0; s < nseq && o < nt; ++s)
            for (size_t q = seqs[s].pos; q < seqs[s].pos + seqs[s].len && o < nt; ++q, ++o) {
                if (dt == OPHIP_DT_U32) {
                    const uint32_t v = (uint32_t)q;
                    std::memcpy(&host[o * 4], &v, 4);
                } else {
                    const uint64_t v = (uint64_t)q;
                    std::memcpy(&host[o * 8], &v, 8);
                }
            }
        void *mem = qa->alloc(qa->ctx, host.size());
        if (!mem && !host.empty()) throw execution_failed("queue allocator returned null");
        if (!host.empty()) {
            check_hip(hipMemcpyAsync(mem, host.data(), host.size(), hipMemcpyHostToDevice, stream_of(qa)),
                      "hipMemcpyAsync");
            // the staging buffer dies with this call, so the copy must have left it
            check_hip(hipStreamSynchronize(stream_of(qa)), "hipStreamSynchronize");
        }
        *out = mem;
    });
}

extern "C" int ophip_rope_build_sincos(uint64_t, size_t, size_t, const ophip_queue_alloc *qa, size_t *nctx_out,
                                       void **out) {
    return guard([&] {
        if (!qa || !qa->alloc || !out) throw args_not_support("null argument");
        if (nctx_out) *nctx_out = 0;
        *out = qa->alloc(qa->ctx, 0);
    });
}

// ========================================================== fuesd_softmax ===
// Args::meta: fuesd_softmax/args.rs:31-37; launch checks: fuesd_softmax/cuda/mod.rs:52-119.

struct SoftmaxVariant {
    int vec, pt, g;
    hipFunction_t fn;
};

struct ophip_fused_softmax : OpBase {
    std::vector<SoftmaxVariant> variants[2];  // [f16 / bf16]
    hipFunction_t stream_fn[2], stream_f32, stream_f64, rows4[2];  // rows4 (f16): four rows per wave, 1 or 2 vectors per lane and row
    explicit ophip_fused_softmax(ophip_device *d) : OpBase(d) {
        static const int table[][3] = {{8, 1, 64},  {8, 2, 64},   {8, 4, 64},   {8, 1, 256},  {8, 2, 256},
                                       {8, 4, 256}, {8, 8, 256},  {8, 4, 1024}, {8, 8, 1024}, {1, 8, 64},
                                       {1, 16, 64}, {1, 8, 256},  {1, 16, 256}, {1, 32, 256}, {1, 16, 1024}};
        for (int e = 0; e < 2; ++e) {
            const std::string tag = e ? "bf16" : "f16";
            for (auto &t : table) {
                const std::string name = "softmax_" + tag + "_v" + std::to_string(t[0]) + "_p" + std::to_string(t[1]) + "_g" +
                                         std::to_string(t[2]);
                variants[e].push_back({t[0], t[1], t[2], d->kernel("fused_softmax", name.c_str())});
            }
            stream_fn[e] = d->kernel("fused_softmax", ("softmax_" + tag + "_stream").c_str());
        }
        stream_f32 = d->kernel("fused_softmax", "softmax_f32_stream");
        stream_f64 = d->kernel("fused_softmax", "softmax_f64_stream");
        rows4[0] = d->kernel("fused_softmax", "softmax_f16_rows4_p1");
        rows4[1] = d->kernel("fused_softmax", "softmax_f16_rows4_p2");
    }
};

extern "C" int ophip_fused_softmax_create(ophip_device *dev, ophip_fused_softmax **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_fused_softmax(dev);
    });
}
extern "C" void ophip_fused_softmax_destroy(ophip_fused_softmax *op) { delete op; }

extern "C" int ophip_fused_softmax_scheme(ophip_fused_softmax *, const ophip_fused_softmax_args *args, size_t,
                                          size_t *ws) {
    return guard([&] {
        if (!args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        if (args->att_layout.ndim != 3) throw rank_not_support("");
        expect_arrays(args->att_layout);
        const uint64_t dt = args->att_layout.dt;
        if (dt != OPHIP_DT_F16 && dt != OPHIP_DT_BF16 && dt != OPHIP_DT_F32 && dt != OPHIP_DT_F64)
            throw type_not_support("fused softmax supports f16, bf16, f32 and f64");
    });
}

extern "C" int ophip_fused_softmax_launch(const ophip_fused_softmax *op, const ophip_fused_softmax_args *args, void *,
                                          size_t, const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const ophip_tensor_layout &l = args->att_layout;
        if (l.ndim != 3) throw rank_not_support("");
        expect_arrays(l);
        // (bf16: in neither backend of the reference; the f16 kernels on bf16 elements)
        if (l.dt != OPHIP_DT_F16 && l.dt != OPHIP_DT_BF16 && l.dt != OPHIP_DT_F32 && l.dt != OPHIP_DT_F64)
            throw type_not_support("fused softmax supports f16, bf16, f32 and f64");
        const ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(l.dt);
        if (args->att_mask != OPHIP_MASK_NONE && args->att_mask != OPHIP_MASK_CAUSAL)
            throw args_not_support("unknown attention mask");
        const size_t nh = static_of(l.shape[0]), seq = static_of(l.shape[1]), att = static_of(l.shape[2]);
        const ptrdiff_t sh = static_of(l.strides[0]), ss = static_of(l.strides[1]), sa = static_of(l.strides[2]);
        if (sa != unit) throw strides_not_support("fused softmax needs a contiguous last dimension");
        if (sh % unit != 0 || ss % unit != 0) throw strides_not_support("misaligned strides");
        const size_t rows = nh * seq;
        if (rows == 0) return;
        const bool causal = args->att_mask == OPHIP_MASK_CAUSAL;
        // a row that keeps no column has no maximum: the reference panics there
        if (att == 0 || (causal && att < seq)) throw shape_not_support("a softmax row keeps no column");
        if (rows > 0x7fffffffu || att > 0x7fffffffu) throw shape_not_support("softmax dimension too large");

        SoftmaxParams p{};
        p.att = args->att_base;
        p.sh = sh;
        p.ss = ss;
        p.nh = (uint32_t)nh;
        p.seq = (uint32_t)seq;
        p.att_len = (uint32_t)att;
        p.causal = causal;

        if (!p.att) throw args_not_support("null base address");
        if (l.dt != OPHIP_DT_F16 && l.dt != OPHIP_DT_BF16) {
            op->dev->make_current();
            launch(l.dt == OPHIP_DT_F32 ? op->stream_f32 : op->stream_f64, Dim3{(unsigned)rows}, Dim3{1024}, 0, stream_of(qa), p);
            return;
        }
        const bool vec = aligned16(p.att) && mult16(sh) && mult16(ss);
        const int want_vec = vec ? 8 : 1;
        // narrowest group that holds the row in registers; with few rows prefer a
        // whole workgroup per row so more lanes pull on memory
        const SoftmaxVariant *pick = nullptr;
        const int e = l.dt == OPHIP_DT_BF16 ? 1 : 0;
        for (const auto &v : op->variants[e]) {
            if (v.vec != want_vec) continue;
            if ((size_t)v.vec * v.pt * v.g < att) continue;
            if (rows < 2048 && v.g < 256 && att >= (size_t)256 * v.vec) continue;
            if (!pick || v.g < pick->g || (v.g == pick->g && v.pt < pick->pt)) pick = &v;
        }
        op->dev->make_current();
        if (e == 0 && vec && att % 8 == 0 && att <= 1024 && rows >= 8192) {
            // many short rows: four per wave, their loads in flight together (16384 waves of one 512-column row
            // each cost more in start-up than in traffic: [32, 512, 512] causal 9.6 -> see the kernel's note)
            const size_t waves = nh * ((seq + 3) / 4);
            launch(op->rows4[att <= 512 ? 0 : 1], Dim3{ceil_div(waves, 4)}, Dim3{256}, 0, stream_of(qa), p);
            return;
        }
        if (!pick) {
            launch(op->stream_fn[e], Dim3{(unsigned)rows}, Dim3{1024}, 0, stream_of(qa), p);
            return;
        }
        const unsigned block = pick->g < 256 ? 256 : pick->g, rpb = block / pick->g;
        launch(pick->fn, Dim3{ceil_div(rows, rpb)}, Dim3{block}, 0, stream_of(qa), p);
    });
}

// ============================================================== rearrange ===
// Scheme::new: rearrange/args.rs:35-153.

namespace {
struct RDim {
    size_t len;
    ptrdiff_t dst, src;
};
struct RScheme {
    size_t unit = 0;
    std::vector<size_t> idx;  // ndim + 1 entries: count ... 1
    std::vector<ptrdiff_t> dst, src;
    size_t ndim() const { return dst.size(); }
    size_t count() const { return idx.empty() ? 1 : idx[0]; }
};

ptrdiff_t iabs(ptrdiff_t v) { return v < 0 ? -v : v; }

RScheme rearrange_scheme(const ophip_rearrange_args &a) {
    const ophip_tensor_layout &D = a.dst_layout, &S = a.src_layout;
    (void)type_distinct({D.dt, S.dt});
    expect_arrays(D);
    expect_arrays(S);
    if (D.ndim != S.ndim)
        throw rank_mismatch("dst.ndim = " + std::to_string(D.ndim) + ", src.ndim = " + std::to_string(S.ndim));
    std::vector<RDim> dims;
    for (size_t i = 0; i < D.ndim; ++i) {
        const size_t dd = static_of(D.shape[i]), ds = static_of(S.shape[i]);
        if (dd != ds)
            throw shape_mismatch("dst[" + std::to_string(i) + "] = " + std::to_string(dd) + ", src[" +
                                 std::to_string(i) + "] = " + std::to_string(ds));
        RDim dim{dd, static_of(D.strides[i]), static_of(S.strides[i])};
        if (dim.len != 1) {
            if (dim.dst == 0) throw shape_not_support("Reducing is not allowed for rearrangement.");
            dims.push_back(dim);
        }
    }
    // |dst| descending, |src| descending, len ascending
    std::sort(dims.begin(), dims.end(), [](const RDim &x, const RDim &y) {
        if (iabs(x.dst) != iabs(y.dst)) return iabs(x.dst) > iabs(y.dst);
        if (iabs(x.src) != iabs(y.src)) return iabs(x.src) > iabs(y.src);
        return x.len < y.len;
    });
    ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(D.dt);
    if (unit == 0) throw type_not_support("unknown data type");
    size_t ndim = dims.size();
    for (size_t r = dims.size(); r-- > 0;) {  // trailing contiguous dims fold into the unit
        if (dims[r].dst == unit && dims[r].src == unit) {
            unit *= (ptrdiff_t)dims[r].len;
            --ndim;
        } else {
            break;
        }
    }
    dims.resize(ndim);
    for (size_t i = dims.size(); i-- > 1;) {  // neighbours with proportional strides merge
        RDim &f = dims[i - 1], &b = dims[i];
        const ptrdiff_t len = (ptrdiff_t)b.len;
        if (b.dst * len == f.dst && b.src * len == f.src) {
            f = RDim{b.len * f.len, b.dst, b.src};
            b = RDim{1, 0, 0};
            --ndim;
        }
    }
    RScheme s;
    s.unit = (size_t)unit;
    std::vector<size_t> lens;
    for (const RDim &d : dims)
        if (d.len != 1) {
            lens.push_back(d.len);
            s.dst.push_back(d.dst);
            s.src.push_back(d.src);
        }
    s.idx.assign(ndim + 1, 1);
    for (size_t i = ndim; i-- > 0;) s.idx[i] = lens[i] * s.idx[i + 1];
    return s;
}
}  // namespace

extern "C" int ophip_rearrange_plan(const ophip_rearrange_args *args, ptrdiff_t *out, size_t *ndim_out) {
    return guard([&] {
        if (!args || !out) throw args_not_support("null argument");
        const RScheme s = rearrange_scheme(*args);
        const size_t nd = s.ndim();
        out[0] = (ptrdiff_t)s.unit;
        for (size_t i = 0; i <= nd; ++i) out[1 + i] = (ptrdiff_t)s.idx[i];
        for (size_t i = 0; i < nd; ++i) {
            out[2 + nd + i] = s.dst[i];
            out[2 + 2 * nd + i] = s.src[i];
        }
        if (ndim_out) *ndim_out = nd;
    });
}

struct ophip_rearrange : OpBase {
    hipFunction_t k32[5], k32_nt[5], k32_one[5], k64[5];  // chunk sizes 16, 8, 4, 2, 1; k32_one: one chunk per thread; k32_nt: non-temporal stores
    hipFunction_t transpose[3];  // units of 2, 4, 8 bytes turned in LDS tiles
    explicit ophip_rearrange(ophip_device *d) : OpBase(d) {
        static const int sizes[5] = {16, 8, 4, 2, 1};
        for (int i = 0; i < 5; ++i) {
            k32[i] = d->kernel("rearrange", ("rearrange_b" + std::to_string(sizes[i])).c_str());
            k32_one[i] = d->kernel("rearrange", ("rearrange1_b" + std::to_string(sizes[i])).c_str());
            k32_nt[i] = d->kernel("rearrange", ("rearrange_nt_b" + std::to_string(sizes[i])).c_str());
            k64[i] = d->kernel("rearrange", ("rearrange64_b" + std::to_string(sizes[i])).c_str());
            if (i < 3) transpose[i] = d->kernel("rearrange", ("rearrange_transpose_b" + std::to_string(2 << i)).c_str());
        }
    }
};

extern "C" int ophip_rearrange_create(ophip_device *dev, ophip_rearrange **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_rearrange(dev);
    });
}
extern "C" void ophip_rearrange_destroy(ophip_rearrange *op) { delete op; }

// The reference's scheme() does no work at all (rearrange/cuda/mod.rs:45-52).
extern "C" int ophip_rearrange_scheme(ophip_rearrange *, const ophip_rearrange_args *, size_t, size_t *ws) {
    return guard([&] {
        if (ws) *ws = 0;
    });
}

extern "C" int ophip_rearrange_launch(const ophip_rearrange *op, const ophip_rearrange_args *args, void *, size_t,
                                      const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const RScheme s = rearrange_scheme(*args);
        if (s.unit == 0 || s.count() == 0) return;
        if (!args->dst_base || !args->src_base) throw args_not_support("null base address");
        op->dev->make_current();
        if (s.ndim() == 0) {  // one contiguous run: a device-to-device copy (rearrange/cuda/mod.rs:64-70)
            // beyond the caches, in whole aligned 16-byte chunks: the copy kernel with non-temporal loads and stores
            // (512 MiB: 79 % of 8 TB/s against the runtime's copy at 67 %)
            const size_t chunks = s.unit / 16;
            if (s.unit >= ((size_t)64 << 20) && s.unit % 16 == 0 && chunks <= 0x7fffffffu && aligned16(args->dst_base) &&
                aligned16(args->src_base)) {
                RearrangeParams p{};
                p.dst = args->dst_base;
                p.src = args->src_base;
                p.total = chunks;
                p.ndim = 0;
                p.chunks_per_unit = (uint32_t)chunks;
                p.cpu_div = make_fastdiv((uint32_t)chunks);
                launch(op->k32_nt[0], Dim3{ceil_div(chunks, 256 * 4)}, Dim3{256}, 0, stream_of(qa), p);
                return;
            }
            check_hip(hipMemcpyAsync(args->dst_base, args->src_base, s.unit, hipMemcpyDeviceToDevice, stream_of(qa)),
                      "hipMemcpyAsync");
            return;
        }
        if (s.ndim() > OPHIP_REARRANGE_MAXD)
            throw rank_not_support("rearrange supports at most " + std::to_string(OPHIP_REARRANGE_MAXD) +
                                   " non-mergeable dimensions");
        // A transposition of small units: the destination contiguous along its innermost dimension A, the source along
        // another one, B, both at least 32 long: 64 x 64 tiles through LDS.
        if ((s.unit == 2 || s.unit == 4 || s.unit == 8) && s.ndim() >= 2 && s.dst[s.ndim() - 1] == (ptrdiff_t)s.unit &&
            reinterpret_cast<uintptr_t>(args->dst_base) % s.unit == 0 && reinterpret_cast<uintptr_t>(args->src_base) % s.unit == 0) {
            const size_t A = s.ndim() - 1;
            size_t Bd = A;
            for (size_t i = 0; i < A; ++i)
                if (s.src[i] == (ptrdiff_t)s.unit) Bd = i;
            std::vector<size_t> len(s.ndim());
            for (size_t i = 0; i < s.ndim(); ++i) len[i] = s.idx[i] / s.idx[i + 1];
            bool fits = Bd != A && len[A] >= 32 && len[Bd] >= 32 && len[A] <= 0x7fffffffu && len[Bd] <= 0x7fffffffu;
            for (size_t i = 0; i < s.ndim() && fits; ++i)
                if (s.dst[i] % (ptrdiff_t)s.unit != 0 || s.src[i] % (ptrdiff_t)s.unit != 0) fits = false;
            if (fits) {
                TransposeParams t{};
                t.dst = args->dst_base;
                t.src = args->src_base;
                t.len_a = (uint32_t)len[A];
                t.len_b = (uint32_t)len[Bd];
                t.dst_b = s.dst[Bd];
                t.src_a = s.src[A];
                t.tiles_a = (uint32_t)((len[A] + 63) / 64);
                t.tiles_b = (uint32_t)((len[Bd] + 63) / 64);
                size_t outer = 1;
                std::vector<size_t> od;
                for (size_t i = 0; i < s.ndim(); ++i)
                    if (i != A && i != Bd) od.push_back(i);
                t.nouter = (uint32_t)od.size();
                for (size_t q = od.size(); q-- > 0;) {
                    t.outer_div[q] = make_fastdiv((uint32_t)outer);
                    t.outer_dst[q] = s.dst[od[q]];
                    t.outer_src[q] = s.src[od[q]];
                    outer *= len[od[q]];
                }
                const size_t tiles = (size_t)t.tiles_a * t.tiles_b;
                if (outer <= 0x7fffffffu && tiles <= 0x7fffffffu && outer * tiles <= 0x7fffffffu) {
                    t.tiles_div = make_fastdiv((uint32_t)tiles);
                    t.tb_div = make_fastdiv(t.tiles_b);
                    launch(op->transpose[s.unit == 2 ? 0 : s.unit == 4 ? 1 : 2], Dim3{(unsigned)(outer * tiles)}, Dim3{256}, 0, stream_of(qa), t);
                    return;
                }
            }
        }
        // widest chunk that divides the unit and keeps every access aligned
        uintptr_t bits = (uintptr_t)s.unit | reinterpret_cast<uintptr_t>(args->dst_base) |
                         reinterpret_cast<uintptr_t>(args->src_base);
        for (size_t i = 0; i < s.ndim(); ++i) bits |= (uintptr_t)iabs(s.dst[i]) | (uintptr_t)iabs(s.src[i]);
        int ci = 0;
        size_t B = 16;
        while (bits & (B - 1)) {
            B >>= 1;
            ++ci;
        }
        RearrangeParams p{};
        p.dst = args->dst_base;
        p.src = args->src_base;
        const size_t cpu = s.unit / B;

        // Visiting order of the units.  The scheme's order walks the destination
        // linearly, so the source is gathered in `unit`-byte runs that may sit far
        // apart.  When another dimension is (nearly) contiguous in the source, walk
        // small 2-D tiles instead - A = innermost destination dimension, B = the
        // source-contiguous one - so that a workgroup's 16 KB touches runs of a few KB
        // on both sides.  Any visiting order copies every unit exactly once.
        std::vector<size_t> lens(s.ndim());
        for (size_t i = 0; i < s.ndim(); ++i) lens[i] = s.idx[i] / s.idx[i + 1];
        std::vector<size_t> o_len(lens);
        std::vector<ptrdiff_t> o_dst(s.dst), o_src(s.src);
        if (s.ndim() >= 2 && s.unit <= 2048) {
            const size_t A = s.ndim() - 1;
            size_t Bd = A;
            for (size_t i = 0; i < A; ++i)
                if (iabs(s.src[i]) < iabs(s.src[Bd])) Bd = i;
            if (Bd != A && iabs(s.src[A]) > 4096 && iabs(s.src[Bd]) <= 4096) {
                auto divisor_at_most = [](size_t len, size_t cap) {
                    size_t best = 1;
                    for (size_t t = 1; t <= cap && t <= len; ++t)
                        if (len % t == 0) best = t;
                    return best;
                };
                const size_t per_tile = std::max<size_t>(1, 16384 / s.unit);  // units in one workgroup's share
                const size_t tA = divisor_at_most(lens[A], std::max<size_t>(1, std::min<size_t>(per_tile, 2048 / s.unit)));
                const size_t tB = divisor_at_most(lens[Bd], std::max<size_t>(1, per_tile / tA));
                if (tA * tB > 1) {
                    o_len.clear(); o_dst.clear(); o_src.clear();
                    auto push = [&](size_t len, ptrdiff_t d, ptrdiff_t sr) {
                        if (len == 1) return;
                        o_len.push_back(len); o_dst.push_back(d); o_src.push_back(sr);
                    };
                    for (size_t i = 0; i < s.ndim(); ++i)
                        if (i != A && i != Bd) push(lens[i], s.dst[i], s.src[i]);
                    // B's outer part goes outside A's: consecutive workgroups then finish one
                    // destination region after another instead of revisiting each several times
                    push(lens[Bd] / tB, s.dst[Bd] * (ptrdiff_t)tB, s.src[Bd] * (ptrdiff_t)tB);
                    push(lens[A] / tA, s.dst[A] * (ptrdiff_t)tA, s.src[A] * (ptrdiff_t)tA);
                    push(tB, s.dst[Bd], s.src[Bd]);
                    push(tA, s.dst[A], s.src[A]);
                    if (o_len.size() > OPHIP_REARRANGE_MAXD) {  // keep the plain order
                        o_len = lens; o_dst = s.dst; o_src = s.src;
                    }
                }
            }
        }
        const size_t nd = o_len.size();
        std::vector<size_t> o_idx(nd + 1, 1);
        for (size_t i = nd; i-- > 0;) o_idx[i] = o_len[i] * o_idx[i + 1];

        p.ndim = (uint32_t)nd;
        p.total = (uint64_t)s.count() * cpu;
        bool small = p.total <= 0x7fffffffu && cpu <= 0x7fffffffu;
        for (size_t i = 0; i < nd; ++i) {
            p.idx[i] = o_idx[i + 1];
            p.dst_s[i] = o_dst[i];
            p.src_s[i] = o_src[i];
            if (o_idx[i + 1] > 0x7fffffffu) small = false;
        }
        p.chunks_per_unit = (uint32_t)cpu;
        if (small) {
            p.cpu_div = make_fastdiv((uint32_t)cpu);
            for (size_t i = 0; i < nd; ++i) p.idx_div[i] = make_fastdiv((uint32_t)o_idx[i + 1]);
            // four chunks per thread, unless that leaves fewer than eight workgroups per CU: then one
            const unsigned cus = (unsigned)op->dev->props.multiProcessorCount;
            const bool one = p.total < (uint64_t)cus * 8 * 256 * 4;
            const bool nt = p.total * B >= ((uint64_t)64 << 20);  // more than the caches hold
            launch(one ? op->k32_one[ci] : nt ? op->k32_nt[ci] : op->k32[ci], Dim3{ceil_div(p.total, one ? 256 : 256 * 4)}, Dim3{256}, 0,
                   stream_of(qa), p);
        } else {
            if (cpu > 0xffffffffu) throw shape_not_support("rearrange unit too large");
            const uint64_t blocks = std::min<uint64_t>((p.total + 255) / 256, 1u << 20);
            launch(op->k64[ci], Dim3{(unsigned)blocks}, Dim3{256}, 0, stream_of(qa), p);
        }
    });
}

// ================================================================= swiglu ===
// Args::meta: swiglu/args.rs:31-50; launch checks: swiglu/cuda/mod.rs:53-98.

struct ophip_swiglu : OpBase {
    hipFunction_t f16_vec, f16_vec_nt, f16_scalar, f32_scalar, f64_scalar, bf16_vec, bf16_vec_nt, bf16_scalar;
    explicit ophip_swiglu(ophip_device *d) : OpBase(d) {
        bf16_vec = d->kernel("swiglu", "swiglu_bf16_vec");
        bf16_vec_nt = d->kernel("swiglu", "swiglu_bf16_vec_nt");
        bf16_scalar = d->kernel("swiglu", "swiglu_bf16_scalar");
        f16_vec = d->kernel("swiglu", "swiglu_f16_vec");
        f16_scalar = d->kernel("swiglu", "swiglu_f16_scalar");
        f32_scalar = d->kernel("swiglu", "swiglu_f32_scalar");
        f64_scalar = d->kernel("swiglu", "swiglu_f64_scalar");
        f16_vec_nt = d->kernel("swiglu", "swiglu_f16_vec_nt");
    }
};

struct SwigluMeta {
    uint64_t dt;
    size_t n, d;
};
static SwigluMeta swiglu_meta(const ophip_swiglu_args &a) {
    expect_rank(a.gate_layout, "gate", 2);
    expect_rank(a.up_layout, "up", 2);
    SwigluMeta m;
    m.dt = type_distinct({a.gate_layout.dt, a.up_layout.dt});
    m.n = dim_distinct({a.gate_layout.shape[0], a.up_layout.shape[0]});
    m.d = dim_distinct({a.gate_layout.shape[1], a.up_layout.shape[1]});
    return m;
}

extern "C" int ophip_swiglu_create(ophip_device *dev, ophip_swiglu **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_swiglu(dev);
    });
}
extern "C" void ophip_swiglu_destroy(ophip_swiglu *op) { delete op; }

extern "C" int ophip_swiglu_scheme(ophip_swiglu *, const ophip_swiglu_args *args, size_t, size_t *ws) {
    return guard([&] {
        if (!args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        (void)swiglu_meta(*args);
    });
}

extern "C" int ophip_swiglu_launch(const ophip_swiglu *op, const ophip_swiglu_args *args, void *, size_t,
                                   const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const SwigluMeta m = swiglu_meta(*args);
        // (bf16: in neither backend of the reference; the f16 kernels on bf16 elements)
        if (m.dt != OPHIP_DT_F16 && m.dt != OPHIP_DT_BF16 && m.dt != OPHIP_DT_F32 && m.dt != OPHIP_DT_F64)
            throw type_not_support("swiglu supports f16, bf16, f32 and f64");
        const size_t n = static_of(m.n), d = static_of(m.d);
        const ptrdiff_t sgn = static_of(args->gate_layout.strides[0]), sgd = static_of(args->gate_layout.strides[1]);
        const ptrdiff_t sun = static_of(args->up_layout.strides[0]), sud = static_of(args->up_layout.strides[1]);
        const ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(m.dt);
        if (sgd != unit || sud != unit) throw strides_not_support("swiglu needs contiguous inner dimensions");
        if (sgn % unit != 0 || sun % unit != 0) throw strides_not_support("misaligned strides");
        if (n == 0 || d == 0) return;
        if (n > 0x7fffffffu || d > 0x7fffffffu) throw shape_not_support("swiglu dimension too large");
        SwigluParams p{};
        p.gate = args->gate_base;
        p.up = args->up_base;
        p.sgn = sgn;
        p.sun = sun;
        p.n = (uint32_t)n;
        p.d = (uint32_t)d;
        const bool bf = m.dt == OPHIP_DT_BF16;
        const bool vec = (m.dt == OPHIP_DT_F16 || bf) && d % 8 == 0 && aligned16(p.gate) && aligned16(p.up) && mult16(sgn) &&
                         mult16(sun);
        const size_t items = vec ? d / 8 : d;
        const unsigned gx = std::min<unsigned>(ceil_div(items, 256), 65535u);
        const unsigned gy = (unsigned)std::min<size_t>(n, 65535);
        // more than the caches hold (and few enough vectors to number them with 32 bits, one per thread)
        const bool big = n * d * (size_t)unit >= ((size_t)64 << 20) && vec && n * items < ((size_t)1 << 31);
        if (big) {
            p.total = (uint32_t)(n * items);
            p.per_row = make_fastdiv((uint32_t)items);
        }
        hipFunction_t fn = vec ? (bf ? (big ? op->bf16_vec_nt : op->bf16_vec) : (big ? op->f16_vec_nt : op->f16_vec))
                           : m.dt == OPHIP_DT_F16 ? op->f16_scalar
                           : bf                   ? op->bf16_scalar
                           : m.dt == OPHIP_DT_F32 ? op->f32_scalar
                                                  : op->f64_scalar;
        if (!p.gate || !p.up) throw args_not_support("null base address");
        op->dev->make_current();
        if (big) launch(fn, Dim3{(unsigned)ceil_div(n * items, 256)}, Dim3{256}, 0, stream_of(qa), p);
        else launch(fn, Dim3{gx, gy}, Dim3{256}, 0, stream_of(qa), p);
    });
}
