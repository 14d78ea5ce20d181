/*
 * CPU oracle for the operators-rs transformer hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement, written from
 * the source text, of what the reference crate's CPU backend computes for
 * rms_norm, rope, fuesd_softmax, rearrange, swiglu, random_sample and mat_mul.
 * Only the test-suite, the smoke check and the benchmark's cpu_baseline leg may
 * load it; nothing in the shipped HIP backend links, imports or calls it.
 *
 * Fidelity rules (why this can be bit-faithful to the Rust code):
 *   - Rust never contracts a*b+c and never reassociates: build with
 *     -ffp-contract=off -fno-fast-math (see Makefile); every expression below is
 *     written in the evaluation order of the Rust source.
 *   - f32::exp / powf / sin / cos lower to the platform libm: glibc here too.
 *   - half::f16::from_f32 is round-to-nearest-even incl. subnormals; to_f32 is exact.
 *   - Iterator::sum and every running sum in the reference are sequential in
 *     index order; rayon only ever splits independent rows / elements.
 *
 * Parity status per function is stated in each function's comment.  The one
 * "parity unpinned" item is the summation order inside mat_mul: the reference
 * delegates to the un-vendored crate `gemm` 0.18 (operators/Cargo.toml:29),
 * whose f16 blocking cannot be read from /root/reference.
 *
 * Threads: the `threads` knob mirrors which axes the reference hands to rayon;
 * results do not depend on it.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* dtype codes of the oracle's own C interface */
enum { ORACLE_F16 = 1, ORACLE_F32 = 2, ORACLE_F64 = 3, ORACLE_U32 = 4, ORACLE_U64 = 5 };
/* error codes: the reference's SchemeErrorKind in declaration order
 * (operators/src/common/error.rs:2-12), 1-based; 0 = ok */
enum {
    ORACLE_OK = 0,
    ORACLE_TYPE_NOT_SUPPORT = 1,
    ORACLE_TYPE_MISMATCH = 2,
    ORACLE_RANK_NOT_SUPPORT = 3,
    ORACLE_RANK_MISMATCH = 4,
    ORACLE_SHAPE_NOT_SUPPORT = 5,
    ORACLE_SHAPE_MISMATCH = 6,
    ORACLE_STRIDES_NOT_SUPPORT = 7,
    ORACLE_ARGS_NOT_SUPPORT = 8,
    ORACLE_DYNAMIC_NOT_SUPPORT = 9,
};

static int g_threads = 1;

ORACLE_API void oracle_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
ORACLE_API int oracle_get_threads(void) { return g_threads; }
ORACLE_API int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_num_procs();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ f16 -- */

/* half::f16::to_f32 — exact widening. */
ORACLE_API float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* half::f16::from_f32 — IEEE round-to-nearest-even, subnormals kept, NaN stays NaN. */
ORACLE_API uint16_t oracle_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 0xff) { /* inf / nan */
        if (man == 0) return sign | 0x7c00u;
        return sign | 0x7c00u | 0x0200u | (uint16_t)(man >> 13);
    }
    int e = (int)exp - 127 + 15;
    if (e >= 31) return sign | 0x7c00u; /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return sign; /* underflow to zero (below half of min subnormal) */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return sign | (uint16_t)half_man;
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++; /* may carry into exp: correct */
    return sign | (uint16_t)half;
}

static inline float ld_f16(const void *p) {
    uint16_t h;
    memcpy(&h, p, 2);
    return oracle_f16_to_f32(h);
}
static inline void st_f16(void *p, float v) {
    uint16_t h = oracle_f32_to_f16(v);
    memcpy(p, &h, 2);
}
static inline float ld_f32(const void *p) {
    float v;
    memcpy(&v, p, 4);
    return v;
}
static inline void st_f32(void *p, float v) { memcpy(p, &v, 4); }
static inline double ld_f64(const void *p) {
    double v;
    memcpy(&v, p, 8);
    return v;
}
static inline void st_f64(void *p, double v) { memcpy(p, &v, 8); }

/* ------------------------------------------------------------- rms_norm -- */

/*
 * operators/src/rms_norm/common_cpu/mod.rs:128-137 (k) and :195-208 (calculate).
 * Rows run one after another; inside a row the reference sums x^2 on one thread
 * and then hands the d independent output elements to rayon.
 *   k = 1 / sqrt( sum_j x^2 / d + eps )          (f32 for f16/f32 data, f64 for f64)
 *   y = (k * w) * x                              (left-to-right product, :203)
 * Supported (w, a) pairs are the reference's :84-90.
 * Pinned by: closed forms in tests (constant row, scale covariance, d = 1, f64
 * restatement) — no reference-held vector exists for the CPU backend itself.
 */
ORACLE_API int oracle_rms_norm(void *y, ptrdiff_t nsy, ptrdiff_t dsy, const void *x,
                               ptrdiff_t nsx, ptrdiff_t dsx, const void *w, ptrdiff_t dsw,
                               size_t n, size_t d, float epsilon, int dt_w, int dt_a) {
    const char *xb = (const char *)x, *wb = (const char *)w;
    char *yb = (char *)y;
    int combo;
    if (dt_w == ORACLE_F16 && dt_a == ORACLE_F16) combo = 0;
    else if (dt_w == ORACLE_F32 && dt_a == ORACLE_F16) combo = 1;
    else if (dt_w == ORACLE_F32 && dt_a == ORACLE_F32) combo = 2;
    else if (dt_w == ORACLE_F64 && dt_a == ORACLE_F64) combo = 3;
    else return ORACLE_TYPE_NOT_SUPPORT; /* the reference hits todo!() here */

    for (ptrdiff_t i = 0; i < (ptrdiff_t)n; i++) {
        if (combo == 3) {
            double sum = 0.0;
            for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
                double v = ld_f64(xb + i * nsx + j * dsx);
                sum = sum + v * v;
            }
            double k = 1.0 / sqrt(sum / (double)d + (double)epsilon);
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
            for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
                double wv = ld_f64(wb + j * dsw);
                double xv = ld_f64(xb + i * nsx + j * dsx);
                st_f64(yb + i * nsy + j * dsy, k * wv * xv);
            }
        } else {
            float sum = 0.0f;
            for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
                const char *p = xb + i * nsx + j * dsx;
                float v = combo == 2 ? ld_f32(p) : ld_f16(p);
                sum = sum + v * v;
            }
            float k = 1.0f / sqrtf(sum / (float)d + epsilon);
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
            for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
                const char *pw = wb + j * dsw;
                const char *px = xb + i * nsx + j * dsx;
                float wv = combo == 0 ? ld_f16(pw) : ld_f32(pw);
                float xv = combo == 2 ? ld_f32(px) : ld_f16(px);
                float r = k * wv * xv;
                if (combo == 2) st_f32(yb + i * nsy + j * dsy, r);
                else st_f16(yb + i * nsy + j * dsy, r);
            }
        }
    }
    return ORACLE_OK;
}

/* ----------------------------------------------------------------- rope -- */

/*
 * operators/src/rope/common_cpu/mod.rs:193-202 (freq_sin_cos), :152-191
 * (Activation::calculate), :212-240 (loop).  Entirely single-threaded in the
 * reference.  Adjacent pairs (2k, 2k+1); H = dh/2;
 *   ang = (calc)pos / powf((calc)theta, (calc)k / (calc)H);  (sin, cos) = (sin ang, cos ang)
 *   [a, b] <- [a*cos - b*sin, a*sin + b*cos]
 * calc = f32 for f16/f32 data, f64 for f64 data.  The last-dim stride must be
 * the element size (:98-100).
 * Pinned by: pos = 0 leaves the tensor bit-identical; pair k = 0 rotates by
 * exactly pos radians; pair norms are preserved; f64 closed form with the
 * interleaved pairing and exponent k/(dh/2).
 */
ORACLE_API int oracle_rope(void *t, ptrdiff_t st, ptrdiff_t sh, ptrdiff_t sd, const void *p,
                           ptrdiff_t sp, size_t nt, size_t nh, size_t dh, float theta, int dt_t,
                           int dt_p) {
    size_t esz = dt_t == ORACLE_F16 ? 2 : dt_t == ORACLE_F32 ? 4 : dt_t == ORACLE_F64 ? 8 : 0;
    if (!esz) return ORACLE_TYPE_NOT_SUPPORT;
    if (dt_p != ORACLE_U32 && dt_p != ORACLE_U64) return ORACLE_TYPE_NOT_SUPPORT;
    if (sd != (ptrdiff_t)esz) return ORACLE_STRIDES_NOT_SUPPORT;
    ptrdiff_t H = (ptrdiff_t)dh / 2;
    ptrdiff_t pair = 2 * (ptrdiff_t)esz;
    char *tb = (char *)t;
    const char *pb = (const char *)p;
    for (ptrdiff_t i = 0; i < (ptrdiff_t)nt; i++) {
        uint64_t pos;
        if (dt_p == ORACLE_U32) {
            uint32_t v;
            memcpy(&v, pb + i * sp, 4);
            pos = v;
        } else {
            memcpy(&pos, pb + i * sp, 8);
        }
        for (ptrdiff_t j = 0; j < (ptrdiff_t)nh; j++) {
            for (ptrdiff_t k = 0; k < H; k++) {
                char *q = tb + i * st + j * sh + k * pair;
                if (dt_t == ORACLE_F64) {
                    double ang = (double)pos / pow((double)theta, (double)k / (double)H);
                    double s = sin(ang), c = cos(ang);
                    double a = ld_f64(q), b = ld_f64(q + 8);
                    st_f64(q, a * c - b * s);
                    st_f64(q + 8, a * s + b * c);
                } else {
                    float ang = (float)pos / powf(theta, (float)k / (float)H);
                    float s = sinf(ang), c = cosf(ang);
                    if (dt_t == ORACLE_F16) {
                        float a = ld_f16(q), b = ld_f16(q + 2);
                        st_f16(q, a * c - b * s);
                        st_f16(q + 2, a * s + b * c);
                    } else {
                        float a = ld_f32(q), b = ld_f32(q + 4);
                        st_f32(q, a * c - b * s);
                        st_f32(q + 4, a * s + b * c);
                    }
                }
            }
        }
    }
    return ORACLE_OK;
}

/* -------------------------------------------------------- fuesd_softmax -- */

/* f16::total_cmp key (IEEE totalOrder on the bit pattern) */
static inline int16_t f16_total_key(uint16_t bits) {
    int16_t v = (int16_t)bits;
    v ^= (int16_t)(((uint16_t)(v >> 15)) >> 1);
    return v;
}
static inline int32_t f32_total_key(float f) {
    int32_t v;
    memcpy(&v, &f, 4);
    v ^= (int32_t)(((uint32_t)(v >> 31)) >> 1);
    return v;
}
static inline int64_t f64_total_key(double f) {
    int64_t v;
    memcpy(&v, &f, 8);
    v ^= (int64_t)(((uint64_t)(v >> 63)) >> 1);
    return v;
}

/*
 * operators/src/fuesd_softmax/common_cpu/mod.rs:99-114 (row loop, rayon over
 * nh*seq rows) and :117-145 (f16), :147-169 (f32), :171-193 (f64: the f32 code in f64).
 * Row (h, r) keeps `causal = att_len - seq_len + r + 1` columns (mask 1) or all
 * (mask 0).  f16: max by total order; e = exp(f32(x) - max) is stored as f16
 * while the un-rounded e is summed sequentially; the stored f16 is re-read and
 * scaled by 1/sum; the masked tail becomes +0.
 * A row that keeps no column makes the reference panic (unwrap on an empty
 * max_by): reported here as ORACLE_SHAPE_NOT_SUPPORT.
 * Pinned by: masked tail exactly +0, row sums, seq = 1 keeps everything,
 * single kept column gives exactly 1.0, shift invariance, f64 closed form.
 */
ORACLE_API int oracle_fused_softmax(void *att, ptrdiff_t sh, ptrdiff_t ss, ptrdiff_t sa, size_t nh,
                                    size_t seq_len, size_t att_len, int mask, int dt) {
    if (dt != ORACLE_F16 && dt != ORACLE_F32 && dt != ORACLE_F64) return ORACLE_TYPE_NOT_SUPPORT;
    if (mask == 1 && att_len < seq_len) return ORACLE_SHAPE_NOT_SUPPORT;
    if (att_len == 0 && nh * seq_len != 0) return ORACLE_SHAPE_NOT_SUPPORT;
    char *base = (char *)att;
    ptrdiff_t rows = (ptrdiff_t)(nh * seq_len);
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1) schedule(static)
    for (ptrdiff_t i = 0; i < rows; i++) {
        ptrdiff_t j = i / (ptrdiff_t)seq_len, r = i % (ptrdiff_t)seq_len;
        char *row = base + j * sh + r * ss;
        ptrdiff_t causal =
            mask ? (ptrdiff_t)att_len - (ptrdiff_t)seq_len + r + 1 : (ptrdiff_t)att_len;
        if (dt == ORACLE_F16) {
            uint16_t best;
            memcpy(&best, row, 2);
            for (ptrdiff_t c = 1; c < causal; c++) {
                uint16_t v;
                memcpy(&v, row + c * sa, 2);
                /* max_by keeps the later element unless the earlier is strictly greater */
                if (!(f16_total_key(best) > f16_total_key(v))) best = v;
            }
            float mx = oracle_f16_to_f32(best);
            float sum = 0.0f;
            for (ptrdiff_t c = 0; c < causal; c++) {
                float e = expf(ld_f16(row + c * sa) - mx);
                st_f16(row + c * sa, e);
                sum = sum + e;
            }
            float div = 1.0f / sum;
            for (ptrdiff_t c = 0; c < causal; c++)
                st_f16(row + c * sa, ld_f16(row + c * sa) * div);
            for (ptrdiff_t c = causal; c < (ptrdiff_t)att_len; c++) {
                uint16_t z = 0;
                memcpy(row + c * sa, &z, 2);
            }
        } else if (dt == ORACLE_F64) {
            double best = ld_f64(row);
            for (ptrdiff_t c = 1; c < causal; c++) {
                double v = ld_f64(row + c * sa);
                if (!(f64_total_key(best) > f64_total_key(v))) best = v;
            }
            double sum = 0.0;
            for (ptrdiff_t c = 0; c < causal; c++) {
                double e = exp(ld_f64(row + c * sa) - best);
                st_f64(row + c * sa, e);
                sum = sum + e;
            }
            double div = 1.0 / sum;
            for (ptrdiff_t c = 0; c < causal; c++)
                st_f64(row + c * sa, ld_f64(row + c * sa) * div);
            for (ptrdiff_t c = causal; c < (ptrdiff_t)att_len; c++) st_f64(row + c * sa, 0.0);
        } else {
            float best = ld_f32(row);
            for (ptrdiff_t c = 1; c < causal; c++) {
                float v = ld_f32(row + c * sa);
                if (!(f32_total_key(best) > f32_total_key(v))) best = v;
            }
            float sum = 0.0f;
            for (ptrdiff_t c = 0; c < causal; c++) {
                float e = expf(ld_f32(row + c * sa) - best);
                st_f32(row + c * sa, e);
                sum = sum + e;
            }
            float div = 1.0f / sum;
            for (ptrdiff_t c = 0; c < causal; c++)
                st_f32(row + c * sa, ld_f32(row + c * sa) * div);
            for (ptrdiff_t c = causal; c < (ptrdiff_t)att_len; c++) st_f32(row + c * sa, 0.0f);
        }
    }
    return ORACLE_OK;
}

/* ------------------------------------------------------------ rearrange -- */

typedef struct {
    size_t len;
    ptrdiff_t dst, src;
} rdim_t;

static ptrdiff_t pabs(ptrdiff_t v) { return v < 0 ? -v : v; }

/* Ord for Dim, operators/src/rearrange/args.rs:93-104:
 * |dst| descending, then |src| descending, then len ascending */
static int rdim_cmp(const void *pa, const void *pb) {
    const rdim_t *a = (const rdim_t *)pa, *b = (const rdim_t *)pb;
    ptrdiff_t ad = pabs(a->dst), bd = pabs(b->dst);
    if (ad != bd) return ad > bd ? -1 : 1;
    ptrdiff_t as = pabs(a->src), bs = pabs(b->src);
    if (as != bs) return as > bs ? -1 : 1;
    if (a->len != b->len) return a->len < b->len ? -1 : 1;
    return 0;
}

/*
 * Scheme::new, operators/src/rearrange/args.rs:35-153.
 * out[] receives [unit, idx_strides(ndim+1 entries, the first is `count`, the
 * last is 1), dst_strides(ndim), src_strides(ndim)], i.e. 2 + 3*ndim values,
 * exactly the reference's Vec<isize>.  Returns the merged ndim (>= 0) or
 * -(error code).  `out` must hold 2 + 3*ndim_in entries.
 * Pinned by: the reference's own known-answer test args.rs:242-304 (both layouts).
 */
ORACLE_API int oracle_rearrange_scheme(size_t ndim_in, const size_t *shape_dst,
                                       const size_t *shape_src, const ptrdiff_t *dst_strides,
                                       const ptrdiff_t *src_strides, size_t elem_size,
                                       ptrdiff_t *out) {
    rdim_t *dims = (rdim_t *)malloc(sizeof(rdim_t) * (ndim_in ? ndim_in : 1));
    size_t nd = 0;
    for (size_t i = 0; i < ndim_in; i++) {
        if (shape_dst[i] == SIZE_MAX || shape_src[i] == SIZE_MAX) {
            free(dims);
            return -ORACLE_DYNAMIC_NOT_SUPPORT;
        }
        if (shape_dst[i] != shape_src[i]) {
            free(dims);
            return -ORACLE_SHAPE_MISMATCH;
        }
        if (dst_strides[i] == PTRDIFF_MAX || src_strides[i] == PTRDIFF_MAX) {
            free(dims);
            return -ORACLE_DYNAMIC_NOT_SUPPORT;
        }
        if (shape_dst[i] != 1) {
            if (dst_strides[i] == 0) {
                free(dims);
                return -ORACLE_SHAPE_NOT_SUPPORT;
            }
            dims[nd].len = shape_dst[i];
            dims[nd].dst = dst_strides[i];
            dims[nd].src = src_strides[i];
            nd++;
        }
    }
    qsort(dims, nd, sizeof(rdim_t), rdim_cmp);
    ptrdiff_t unit = (ptrdiff_t)elem_size;
    size_t ndim = nd;
    /* fold trailing contiguous dims into unit (:108-119) */
    for (size_t r = nd; r-- > 0;) {
        if (dims[r].dst == unit && dims[r].src == unit) {
            unit *= (ptrdiff_t)dims[r].len;
            ndim--;
        } else {
            break;
        }
    }
    nd = ndim; /* truncate */
    /* merge neighbours with proportional strides (:121-139) */
    for (size_t i = nd; i-- > 1;) {
        rdim_t *f = &dims[i - 1], *b = &dims[i];
        ptrdiff_t len = (ptrdiff_t)b->len;
        if (b->dst * len == f->dst && b->src * len == f->src) {
            f->len = b->len * f->len;
            f->dst = b->dst;
            f->src = b->src;
            b->len = 1;
            b->dst = 0;
            b->src = 0;
            ndim--;
        }
    }
    /* layout vector (:141-152) */
    for (size_t i = 0; i < 2 + 3 * ndim; i++) out[i] = 0;
    out[0] = unit;
    out[ndim + 1] = 1;
    size_t o = 0;
    for (size_t i = 0; i < nd; i++) {
        if (dims[i].len == 1) continue;
        out[1 + o] = (ptrdiff_t)dims[i].len;
        out[2 + ndim + o] = dims[i].dst;
        out[2 + 2 * ndim + o] = dims[i].src;
        o++;
    }
    for (size_t i = ndim; i >= 1; i--) out[i] *= out[i + 1];
    free(dims);
    return (int)ndim;
}

/*
 * Scheme::distribute_unit, operators/src/rearrange/args.rs:157-195.
 * `in` is a scheme of `ndim` dims (2 + 3*ndim values); `out` receives
 * 2 + 3*(ndim+1) values unless the chosen unit equals the current one, in which
 * case the scheme is copied.  Returns the new ndim, or -1 if no candidate divides.
 * Pinned by: the second half of the reference KAT (args.rs:290-303).
 */
ORACLE_API int oracle_rearrange_distribute_unit(size_t ndim, const ptrdiff_t *in,
                                                const size_t *candidates, size_t ncand,
                                                ptrdiff_t *out) {
    size_t unit_old = (size_t)in[0], unit = 0;
    for (size_t i = 0; i < ncand; i++)
        if (candidates[i] != 0 && unit_old % candidates[i] == 0) {
            unit = candidates[i];
            break;
        }
    if (!unit) return -1;
    if (unit == unit_old) {
        memcpy(out, in, sizeof(ptrdiff_t) * (2 + 3 * ndim));
        return (int)ndim;
    }
    ptrdiff_t extra = (ptrdiff_t)(unit_old / unit);
    out[0] = (ptrdiff_t)unit;
    ptrdiff_t *idx = out + 1;              /* ndim + 2 entries */
    ptrdiff_t *dst = out + 1 + ndim + 2;   /* ndim + 1 entries */
    ptrdiff_t *src = dst + ndim + 1;       /* ndim + 1 entries */
    const ptrdiff_t *idx_ = in + 1;        /* ndim + 1 entries */
    const ptrdiff_t *dst_ = in + 2 + ndim; /* ndim entries */
    const ptrdiff_t *src_ = dst_ + ndim;
    for (size_t i = 0; i < ndim + 1; i++) idx[i] = idx_[i] * extra;
    idx[ndim + 1] = 1;
    for (size_t i = 0; i < ndim; i++) {
        dst[i] = dst_[i];
        src[i] = src_[i];
    }
    dst[ndim] = (ptrdiff_t)unit;
    src[ndim] = (ptrdiff_t)unit;
    return (int)ndim + 1;
}

/*
 * launch, operators/src/rearrange/common_cpu/mod.rs:35-58: one memcpy(unit) when
 * count == 1, else rayon over the flat unit index with a mixed-radix decode.
 * Byte-exact by construction; pinned against numpy strided copies in the tests.
 */
ORACLE_API int oracle_rearrange(void *dst, const void *src, size_t ndim_in, const size_t *shape,
                                const ptrdiff_t *dst_strides, const ptrdiff_t *src_strides,
                                size_t elem_size) {
    ptrdiff_t *sch = (ptrdiff_t *)malloc(sizeof(ptrdiff_t) * (2 + 3 * (ndim_in + 1)));
    int nd = oracle_rearrange_scheme(ndim_in, shape, shape, dst_strides, src_strides, elem_size, sch);
    if (nd < 0) {
        free(sch);
        return -nd;
    }
    size_t unit = (size_t)sch[0];
    ptrdiff_t count = sch[1];
    if (count == 1) {
        memcpy(dst, src, unit);
    } else {
        const ptrdiff_t *idx = sch + 2, *ds = sch + 2 + nd, *ss = sch + 2 + 2 * nd;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1) schedule(static)
        for (ptrdiff_t f = 0; f < count; f++) {
            ptrdiff_t rem = f;
            char *d = (char *)dst;
            const char *s = (const char *)src;
            for (int q = 0; q < nd; q++) {
                ptrdiff_t k = rem / idx[q];
                d += k * ds[q];
                s += k * ss[q];
                rem %= idx[q];
            }
            memcpy(d, s, unit);
        }
    }
    free(sch);
    return ORACLE_OK;
}

/* --------------------------------------------------------------- swiglu -- */

/*
 * operators/src/swiglu/common_cpu/mod.rs:98-137: gate <- (a * sigmoid(a)) * b
 * with sigmoid(x) = 1 / (1 + exp(-x)), f32 arithmetic for f16 data.
 * Single-threaded double loop in the reference.
 * Pinned by: gate = 0 gives zero, up = 1 gives SiLU, saturation, f64 closed form.
 */
ORACLE_API int oracle_swiglu(void *gate, ptrdiff_t sgn, ptrdiff_t sgd, const void *up,
                             ptrdiff_t sun, ptrdiff_t sud, size_t n, size_t d, int dt) {
    if (dt != ORACLE_F16 && dt != ORACLE_F32 && dt != ORACLE_F64) return ORACLE_TYPE_NOT_SUPPORT;
    char *g = (char *)gate;
    const char *u = (const char *)up;
    for (ptrdiff_t i = 0; i < (ptrdiff_t)n; i++)
        for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
            char *pg = g + i * sgn + j * sgd;
            const char *pu = u + i * sun + j * sud;
            if (dt == ORACLE_F16) {
                float a = ld_f16(pg), b = ld_f16(pu);
                st_f16(pg, a * (1.0f / (1.0f + expf(-a))) * b);
            } else if (dt == ORACLE_F32) {
                float a = ld_f32(pg), b = ld_f32(pu);
                st_f32(pg, a * (1.0f / (1.0f + expf(-a))) * b);
            } else {
                double a = ld_f64(pg), b = ld_f64(pu);
                st_f64(pg, a * (1.0 / (1.0 + exp(-a))) * b);
            }
        }
    return ORACLE_OK;
}

/* -------------------------------------------------------- random_sample -- */

typedef struct {
    uint32_t idx;
    uint32_t val; /* value bytes in the low bytes (kv_pair.rs:19-32) */
} oracle_kv_pair;

typedef struct {
    uint32_t idx;
    float val;
} kvf_t;

/* Ord for KVPair<f32>, operators/src/random_sample/kv_pair.rs:73-83:
 * value descending, ties by index ascending, unordered (NaN) counts as equal */
static int kvf_cmp(const void *pa, const void *pb) {
    const kvf_t *a = (const kvf_t *)pa, *b = (const kvf_t *)pb;
    if (a->val == b->val) return a->idx < b->idx ? -1 : a->idx > b->idx ? 1 : 0;
    if (a->val < b->val) return 1;  /* Less reversed -> Greater */
    if (a->val > b->val) return -1; /* Greater reversed -> Less */
    return 0;                       /* None */
}

static float load_logit(const void *base, size_t i, int dt) {
    return dt == ORACLE_F16 ? ld_f16((const char *)base + 2 * i)
                            : ld_f32((const char *)base + 4 * i);
}

/*
 * argmax, operators/src/random_sample/common_cpu/mod.rs:102-109:
 * Iterator::max_by keeps the LATER element unless the earlier one compares
 * strictly Greater; partial_cmp failures (NaN) count as Equal, so a NaN always
 * replaces the running best and is itself replaced by the next element.
 * The pair carries the winning logit's own bits.
 * Pinned by: brute force n-1-argmax(reversed) on NaN-free data, crafted ties.
 */
ORACLE_API int oracle_argmax(oracle_kv_pair *out, const void *logits, size_t n, int dt) {
    if (dt != ORACLE_F16 && dt != ORACLE_F32) return ORACLE_TYPE_NOT_SUPPORT;
    if (n == 0) return ORACLE_SHAPE_NOT_SUPPORT; /* reference: unwrap on None panics */
    size_t best = 0;
    float bv = load_logit(logits, 0, dt);
    for (size_t i = 1; i < n; i++) {
        float v = load_logit(logits, i, dt);
        if (!(bv > v)) {
            best = i;
            bv = v;
        }
    }
    out->idx = (uint32_t)best;
    out->val = 0;
    memcpy(&out->val, (const char *)logits + (dt == ORACLE_F16 ? 2 : 4) * best,
           dt == ORACLE_F16 ? 2 : 4);
    return ORACLE_OK;
}

/*
 * random, operators/src/random_sample/common_cpu/mod.rs:111-144.
 *   pairs (idx, f32 logit) sorted by kvf_cmp; max = first; first.val = 1;
 *   val[i] = val[i-1] + exp((val[i] - max) / t)       sequential f32 running sum
 *   pk = val[min(top_k, n) - 1]; pp = val[n-1] * top_p; plimit = seed * min(pk, pp)
 *   answer = first pair with val >= plimit; its val (the running sum) is cast to T.
 * sort_unstable over a strict total order (indices are unique) has one possible
 * result, so qsort reproduces it; NaN logits make the order unspecified in the
 * reference too.
 * Pinned by: a brute-force restatement on small n (numpy lexsort + cumsum),
 * seed -> 0 gives the smallest index among the maxima, index always inside the
 * top-k set, monotone in seed.
 */
ORACLE_API int oracle_random_sample(oracle_kv_pair *out, const void *logits, size_t n, int dt,
                                    float temperature, float top_p, size_t top_k, float seed) {
    if (dt != ORACLE_F16 && dt != ORACLE_F32) return ORACLE_TYPE_NOT_SUPPORT;
    if (n == 0) return ORACLE_SHAPE_NOT_SUPPORT;
    if (temperature == 0.0f || top_k == 1) return oracle_argmax(out, logits, n, dt);
    kvf_t *v = (kvf_t *)malloc(sizeof(kvf_t) * n);
    for (size_t i = 0; i < n; i++) {
        v[i].idx = (uint32_t)i;
        v[i].val = load_logit(logits, i, dt);
    }
    qsort(v, n, sizeof(kvf_t), kvf_cmp);
    float mx = v[0].val;
    v[0].val = 1.0f;
    for (size_t i = 1; i < n; i++) v[i].val = v[i - 1].val + expf((v[i].val - mx) / temperature);
    size_t kk = top_k < n ? top_k : n;
    float pk = v[kk - 1].val;
    float pp = v[n - 1].val * top_p;
    float plimit = seed * fminf(pk, pp);
    size_t ans = n;
    for (size_t i = 0; i < n; i++)
        if (v[i].val >= plimit) {
            ans = i;
            break;
        }
    if (ans == n) { /* reference: find().unwrap() panics (seed > 1 or NaN) */
        free(v);
        return ORACLE_ARGS_NOT_SUPPORT;
    }
    out->idx = v[ans].idx;
    out->val = 0;
    if (dt == ORACLE_F16) {
        uint16_t h = oracle_f32_to_f16(v[ans].val);
        memcpy(&out->val, &h, 2);
    } else {
        memcpy(&out->val, &v[ans].val, 4);
    }
    free(v);
    return ORACLE_OK;
}

/* -------------------------------------------------------------- mat_mul -- */

/* SchemeLayout, operators/src/mat_mul/args.rs:22-42 (strides / lds in elements) */
typedef struct {
    int32_t ab_swap, a_trans, b_trans;
    int32_t _pad;
    size_t batch, m, n, k;
    ptrdiff_t c_stride, c_ld, a_stride, a_ld, b_stride, b_ld;
} oracle_mm_layout;

typedef struct {
    size_t batch;
    ptrdiff_t stride;
    size_t r, c;
    ptrdiff_t rs, cs;
} mtx_t;

/* Matrix::try_from, args.rs:134-172 */
static int mtx_from(mtx_t *m, size_t ndim, const size_t *shape, const ptrdiff_t *strides,
                    size_t unit) {
    for (size_t i = 0; i < ndim; i++)
        if (shape[i] == SIZE_MAX || strides[i] == PTRDIFF_MAX) return ORACLE_DYNAMIC_NOT_SUPPORT;
    if (ndim < 2) return ORACLE_RANK_NOT_SUPPORT;
    if (ndim > 3) return ORACLE_SHAPE_NOT_SUPPORT;
    if (ndim == 2 || shape[0] == 1) {
        m->batch = 1;
        m->stride = 0;
    } else {
        m->batch = shape[0];
        m->stride = strides[0] / (ptrdiff_t)unit;
    }
    m->r = shape[ndim - 2];
    m->c = shape[ndim - 1];
    m->rs = strides[ndim - 2] / (ptrdiff_t)unit;
    m->cs = strides[ndim - 1] / (ptrdiff_t)unit;
    return ORACLE_OK;
}
static void mtx_transpose(mtx_t *m) {
    size_t t = m->r;
    m->r = m->c;
    m->c = t;
    ptrdiff_t s = m->rs;
    m->rs = m->cs;
    m->cs = s;
}
static int mtx_ld_trans(const mtx_t *m, ptrdiff_t *ld, int32_t *trans) {
    if (m->rs == 1) {
        *ld = m->cs;
        *trans = 0;
        return ORACLE_OK;
    }
    if (m->cs == 1) {
        *ld = m->rs;
        *trans = 1;
        return ORACLE_OK;
    }
    return ORACLE_STRIDES_NOT_SUPPORT;
}

/*
 * Args::layout, operators/src/mat_mul/args.rs:64-121: every operand becomes a
 * Matrix{batch, stride, r, c, rs, cs} in elements; a row-major C transposes the
 * whole product and swaps A and B; the result is a column-major strided-batched
 * GEMM descriptor.
 * Pinned by: hand cases in the tests (row-major C => ab_swap, the four
 * transposition combinations, broadcast batch => stride 0, error kinds).
 */
ORACLE_API int oracle_mat_mul_layout(oracle_mm_layout *out, size_t elem_size, size_t c_ndim,
                                     const size_t *c_shape, const ptrdiff_t *c_strides,
                                     size_t a_ndim, const size_t *a_shape,
                                     const ptrdiff_t *a_strides, size_t b_ndim,
                                     const size_t *b_shape, const ptrdiff_t *b_strides) {
    mtx_t c, a, b;
    int e;
    if ((e = mtx_from(&c, c_ndim, c_shape, c_strides, elem_size))) return e;
    if ((e = mtx_from(&a, a_ndim, a_shape, a_strides, elem_size))) return e;
    if ((e = mtx_from(&b, b_ndim, b_shape, b_strides, elem_size))) return e;
    if (c.r != a.r || c.c != b.c || a.c != b.r) return ORACLE_SHAPE_MISMATCH;
    size_t batch = c.batch;
    if (!(a.batch == 1 || a.batch == batch) || !(b.batch == 1 || b.batch == batch))
        return ORACLE_SHAPE_MISMATCH;
    int ab_swap;
    if (c.rs == 1 && c.cs != 1) {
        ab_swap = 0;
    } else if (c.cs == 1) {
        mtx_transpose(&c);
        mtx_transpose(&a);
        mtx_transpose(&b);
        mtx_t t = a;
        a = b;
        b = t;
        ab_swap = 1;
    } else {
        return ORACLE_STRIDES_NOT_SUPPORT;
    }
    memset(out, 0, sizeof(*out));
    if ((e = mtx_ld_trans(&a, &out->a_ld, &out->a_trans))) return e;
    if ((e = mtx_ld_trans(&b, &out->b_ld, &out->b_trans))) return e;
    out->ab_swap = ab_swap;
    out->batch = batch;
    out->m = c.r;
    out->n = c.c;
    out->k = a.c;
    out->c_stride = c.stride;
    out->c_ld = c.cs;
    out->a_stride = a.stride;
    out->b_stride = b.stride;
    return ORACLE_OK;
}

/*
 * launch, operators/src/mat_mul/common_cpu/mod.rs:60-105.  Per batch
 *   C = (beta != 0 ? beta' * C : 0) + alpha' * (A . B)
 * where for f16 data alpha' and beta' are alpha and beta rounded to f16 (:101)
 * and `beta != 0` is tested on the f32 argument (:80).  Products and sums are
 * f32 (f64 for f64 data), k ascending, one rounding to the storage type at the end.
 * PARITY UNPINNED at bit level: the reference delegates the arithmetic to the
 * un-vendored `gemm` 0.18 crate whose f16 blocking order is not readable here;
 * any f32-accumulating order agrees within K * 2^-24 relative plus one f16 rounding.
 * a_base / b_base are the ORIGINAL operands; the swap is applied here as in :60-66.
 */
ORACLE_API int oracle_mat_mul(void *c_base, float beta, const void *a_base, const void *b_base,
                              float alpha, const oracle_mm_layout *L, int dt) {
    if (dt != ORACLE_F16 && dt != ORACLE_F32 && dt != ORACLE_F64) return ORACLE_TYPE_NOT_SUPPORT;
    const void *a = L->ab_swap ? b_base : a_base;
    const void *b = L->ab_swap ? a_base : b_base;
    ptrdiff_t lhs_cs = L->a_trans ? 1 : L->a_ld, lhs_rs = L->a_trans ? L->a_ld : 1;
    ptrdiff_t rhs_cs = L->b_trans ? 1 : L->b_ld, rhs_rs = L->b_trans ? L->b_ld : 1;
    ptrdiff_t M = (ptrdiff_t)L->m, N = (ptrdiff_t)L->n, K = (ptrdiff_t)L->k;
    float al = alpha, be = beta;
    if (dt == ORACLE_F16) {
        al = oracle_f16_to_f32(oracle_f32_to_f16(alpha));
        be = oracle_f16_to_f32(oracle_f32_to_f16(beta));
    }
    int read_dst = beta != 0.0f;
    if (dt == ORACLE_F16) {
        /* Tasks are (column j, block of IB rows); inside a task every C element is
         * still one k-ascending f32 running sum, so the result does not depend on
         * the blocking or on the loop order chosen for cache behaviour. */
        enum { IB = 256 };
        ptrdiff_t nib = (M + IB - 1) / IB;
        for (ptrdiff_t bi = 0; bi < (ptrdiff_t)L->batch; bi++) {
            uint16_t *C = (uint16_t *)c_base + bi * L->c_stride;
            const uint16_t *A = (const uint16_t *)a + bi * L->a_stride;
            const uint16_t *B = (const uint16_t *)b + bi * L->b_stride;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1) schedule(dynamic, 1)
            for (ptrdiff_t task = 0; task < N * nib; task++) {
                ptrdiff_t j = task / nib, i0 = (task % nib) * IB;
                ptrdiff_t i1 = i0 + IB < M ? i0 + IB : M;
                float acc[IB];
                for (ptrdiff_t i = i0; i < i1; i++) acc[i - i0] = 0.0f;
                if (lhs_rs == 1) { /* A is m-contiguous: sweep k outermost */
                    for (ptrdiff_t l = 0; l < K; l++) {
                        float bv = oracle_f16_to_f32(B[l * rhs_rs + j * rhs_cs]);
                        const uint16_t *acol = A + l * lhs_cs;
                        for (ptrdiff_t i = i0; i < i1; i++)
                            acc[i - i0] = acc[i - i0] + oracle_f16_to_f32(acol[i]) * bv;
                    }
                } else { /* A is k-contiguous: one dot product per row */
                    for (ptrdiff_t i = i0; i < i1; i++) {
                        float s = 0.0f;
                        const uint16_t *arow = A + i * lhs_rs;
                        for (ptrdiff_t l = 0; l < K; l++)
                            s = s + oracle_f16_to_f32(arow[l * lhs_cs]) *
                                        oracle_f16_to_f32(B[l * rhs_rs + j * rhs_cs]);
                        acc[i - i0] = s;
                    }
                }
                for (ptrdiff_t i = i0; i < i1; i++) {
                    uint16_t *pc = C + i + j * L->c_ld;
                    float r = al * acc[i - i0];
                    if (read_dst) r = be * oracle_f16_to_f32(*pc) + r;
                    *pc = oracle_f32_to_f16(r);
                }
            }
        }
        return ORACLE_OK;
    }
    for (ptrdiff_t bi = 0; bi < (ptrdiff_t)L->batch; bi++) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1) schedule(static)
        for (ptrdiff_t j = 0; j < N; j++) {
            if (dt == ORACLE_F32) {
                float *C = (float *)c_base + bi * L->c_stride;
                const float *A = (const float *)a + bi * L->a_stride;
                const float *B = (const float *)b + bi * L->b_stride;
                for (ptrdiff_t i = 0; i < M; i++) {
                    float acc = 0.0f;
                    for (ptrdiff_t l = 0; l < K; l++)
                        acc = acc + A[i * lhs_rs + l * lhs_cs] * B[l * rhs_rs + j * rhs_cs];
                    float *pc = C + i + j * L->c_ld;
                    float r = al * acc;
                    if (read_dst) r = be * *pc + r;
                    *pc = r;
                }
            } else {
                double *C = (double *)c_base + bi * L->c_stride;
                const double *A = (const double *)a + bi * L->a_stride;
                const double *B = (const double *)b + bi * L->b_stride;
                for (ptrdiff_t i = 0; i < M; i++) {
                    double acc = 0.0;
                    for (ptrdiff_t l = 0; l < K; l++)
                        acc = acc + A[i * lhs_rs + l * lhs_cs] * B[l * rhs_rs + j * rhs_cs];
                    double *pc = C + i + j * L->c_ld;
                    double r = (double)alpha * acc;
                    if (read_dst) r = (double)beta * *pc + r;
                    *pc = r;
                }
            }
        }
    }
    return ORACLE_OK;
}

/* ------------------------------------------------------------ layer_norm -- */
/* layer_norm/common_cpu/mod.rs:127-147 (Scheme::calculate), X = f32 for f16 / f32 data:
 *   sum, sum2 sequential in j; e = sum/d; e2 = sum2/d; std = sqrt(e2 - e*e);
 *   k = 1/(std + eps);  y = fma(x - e, s*k, b)  (mul_add is one fused operation).
 * (scale/bias, x/y) in {(f16,f16), (f32,f16), (f32,f32), (f64,f64)} (mod.rs:84-90).
 * Pinned by: f64 closed form, constant row gives bias exactly, scale 1 / bias 0 gives zero
 * mean, explicit numpy-f32 replay of the rounding points.
 */
ORACLE_API int oracle_layer_norm(void *y, ptrdiff_t nsy, ptrdiff_t dsy, const void *x, ptrdiff_t nsx,
                                 ptrdiff_t dsx, const void *s, ptrdiff_t dss, const void *b, ptrdiff_t dsb,
                                 size_t n, size_t d, float epsilon, int dt_a, int dt_w) {
    const int f64 = dt_a == ORACLE_F64 && dt_w == ORACLE_F64;
    const int ok = (dt_a == ORACLE_F16 && (dt_w == ORACLE_F16 || dt_w == ORACLE_F32)) ||
                   (dt_a == ORACLE_F32 && dt_w == ORACLE_F32) || f64;
    if (!ok) return ORACLE_TYPE_NOT_SUPPORT;
    for (ptrdiff_t i = 0; i < (ptrdiff_t)n; i++) {
        const char *xr = (const char *)x + i * nsx;
        char *yr = (char *)y + i * nsy;
        if (f64) {
            double sum = 0.0, sum2 = 0.0;
            for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
                double v = ld_f64(xr + j * dsx);
                sum += v;
                sum2 += v * v;
            }
            double nn = (double)d, e = sum / nn, e2 = sum2 / nn;
            double k = 1.0 / (sqrt(e2 - e * e) + (double)epsilon);
            for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++)
                st_f64(yr + j * dsy, fma(ld_f64(xr + j * dsx) - e, ld_f64((const char *)s + j * dss) * k,
                                         ld_f64((const char *)b + j * dsb)));
        } else {
            float sum = 0.0f, sum2 = 0.0f;
            for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
                float v = dt_a == ORACLE_F16 ? ld_f16(xr + j * dsx) : ld_f32(xr + j * dsx);
                sum += v;
                sum2 += v * v;
            }
            float nn = (float)d, e = sum / nn, e2 = sum2 / nn;
            float k = 1.0f / (sqrtf(e2 - e * e) + epsilon);
            for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
                float v = dt_a == ORACLE_F16 ? ld_f16(xr + j * dsx) : ld_f32(xr + j * dsx);
                float sc = dt_w == ORACLE_F16 ? ld_f16((const char *)s + j * dss) : ld_f32((const char *)s + j * dss);
                float bi = dt_w == ORACLE_F16 ? ld_f16((const char *)b + j * dsb) : ld_f32((const char *)b + j * dsb);
                float r = fmaf(v - e, sc * k, bi);
                if (dt_a == ORACLE_F16) st_f16(yr + j * dsy, r);
                else st_f32(yr + j * dsy, r);
            }
        }
    }
    return ORACLE_OK;
}

/* ------------------------------------------------------------------ gelu -- */
/* gelu/common_cpu/mod.rs:112-123:  0.5 * x * (1 + tanh(sqrt(2/pi) * (x + 0.044715 * x^3))),
 * evaluated left to right in the element's arithmetic type (f32 for f16 data); powi(3) is
 * x * x * x; FRAC_2_PI.sqrt() is the correctly rounded square root of the f32 constant.
 * Pinned by: f64 closed form, gelu(0) = 0, large |x| saturates to x and -0, odd part identity
 * gelu(x) - gelu(-x) = x.
 */
ORACLE_API int oracle_gelu(void *base, ptrdiff_t sn, ptrdiff_t sd, size_t n, size_t d, int dt) {
    if (dt != ORACLE_F16 && dt != ORACLE_F32 && dt != ORACLE_F64) return ORACLE_TYPE_NOT_SUPPORT;
    const float c32 = sqrtf(0.636619772367581343076f);
    const double c64 = sqrt(0.636619772367581343076);
    for (ptrdiff_t i = 0; i < (ptrdiff_t)n; i++)
        for (ptrdiff_t j = 0; j < (ptrdiff_t)d; j++) {
            char *p = (char *)base + i * sn + j * sd;
            if (dt == ORACLE_F64) {
                double v = ld_f64(p);
                st_f64(p, 0.5 * v * (1.0 + tanh(c64 * (v + 0.044715 * (v * v * v)))));
            } else {
                float v = dt == ORACLE_F16 ? ld_f16(p) : ld_f32(p);
                float r = 0.5f * v * (1.0f + tanhf(c32 * (v + 0.044715f * (v * v * v))));
                if (dt == ORACLE_F16) st_f16(p, r);
                else st_f32(p, r);
            }
        }
    return ORACLE_OK;
}

/* ------------------------------------------------------------------- add -- */
/* add/args.rs:42-167 (validation) + add/common_cpu/mod.rs:29-75: c = a + b element-wise.
 * The reference's Scheme only chooses the visiting order (merged dimensions); the sum of two
 * f16 is formed in f32 and rounded once (half's Add).  Checks in the reference's order:
 * types, ranks, per-dimension shapes, zero c stride on a dimension longer than 1.
 * Pinned by: numpy on random strided / broadcast layouts (f16 sums of f16 are exact in f32,
 * so numpy's float16 add rounds identically).
 */
ORACLE_API int oracle_add(void *c, const void *a, const void *b, size_t ndim_c, size_t ndim_a, size_t ndim_b,
                          const size_t *shape_c, const size_t *shape_a, const size_t *shape_b,
                          const ptrdiff_t *sc, const ptrdiff_t *sa, const ptrdiff_t *sb, int dt_c, int dt_a,
                          int dt_b) {
    if (dt_c != dt_a || dt_c != dt_b) return ORACLE_TYPE_MISMATCH;
    if (ndim_a != ndim_c || ndim_b != ndim_c) return ORACLE_RANK_MISMATCH;
    size_t total = 1;
    for (size_t i = 0; i < ndim_c; i++) {
        if (shape_c[i] == SIZE_MAX || shape_a[i] == SIZE_MAX || shape_b[i] == SIZE_MAX ||
            sc[i] == PTRDIFF_MAX || sa[i] == PTRDIFF_MAX || sb[i] == PTRDIFF_MAX)
            return ORACLE_DYNAMIC_NOT_SUPPORT;
        if (shape_a[i] != shape_c[i] || shape_b[i] != shape_c[i]) return ORACLE_SHAPE_MISMATCH;
        if (shape_c[i] != 1 && sc[i] == 0) return ORACLE_SHAPE_NOT_SUPPORT;
        total *= shape_c[i];
    }
    if (dt_c != ORACLE_F16 && dt_c != ORACLE_F32 && dt_c != ORACLE_F64) return ORACLE_TYPE_NOT_SUPPORT;
    for (size_t f = 0; f < total; f++) {
        size_t rem = f;
        ptrdiff_t oc = 0, oa = 0, ob = 0;
        for (size_t q = ndim_c; q-- > 0;) {
            ptrdiff_t k = (ptrdiff_t)(rem % shape_c[q]);
            rem /= shape_c[q];
            oc += k * sc[q];
            oa += k * sa[q];
            ob += k * sb[q];
        }
        if (dt_c == ORACLE_F16) st_f16((char *)c + oc, ld_f16((const char *)a + oa) + ld_f16((const char *)b + ob));
        else if (dt_c == ORACLE_F32) st_f32((char *)c + oc, ld_f32((const char *)a + oa) + ld_f32((const char *)b + ob));
        else st_f64((char *)c + oc, ld_f64((const char *)a + oa) + ld_f64((const char *)b + ob));
    }
    return ORACLE_OK;
}

/* -------------------------------------------------------------- add_rows -- */
/* add_rows/common_cpu/mod.rs:131-147: dst[b, m, :] += src[idx[b, m], :]; the reference
 * asserts idx < k (here: ORACLE_ARGS_NOT_SUPPORT, nothing of that row is written).
 * Pinned by: numpy fancy indexing with repeated and boundary indices.
 */
ORACLE_API int oracle_add_rows(void *dst, ptrdiff_t bsd, ptrdiff_t msd, ptrdiff_t nsd, const void *src,
                               ptrdiff_t kss, ptrdiff_t nss, const void *idx, ptrdiff_t bsi, ptrdiff_t msi,
                               size_t batch, size_t m, size_t n, size_t k, int dt, int dt_idx) {
    if (dt_idx != ORACLE_U32 && dt_idx != ORACLE_U64) return ORACLE_TYPE_NOT_SUPPORT;
    if (dt != ORACLE_F16 && dt != ORACLE_F32 && dt != ORACLE_F64) return ORACLE_TYPE_NOT_SUPPORT;
    int bad = 0;
    for (ptrdiff_t bi = 0; bi < (ptrdiff_t)batch; bi++)
        for (ptrdiff_t mi = 0; mi < (ptrdiff_t)m; mi++) {
            const char *ip = (const char *)idx + bi * bsi + mi * msi;
            uint64_t r;
            if (dt_idx == ORACLE_U32) {
                uint32_t t;
                memcpy(&t, ip, 4);
                r = t;
            } else {
                memcpy(&r, ip, 8);
            }
            if (r >= k) {
                bad = 1;
                continue;
            }
            char *d = (char *)dst + bi * bsd + mi * msd;
            const char *s = (const char *)src + (ptrdiff_t)r * kss;
            for (ptrdiff_t j = 0; j < (ptrdiff_t)n; j++) {
                char *pd = d + j * nsd;
                const char *ps = s + j * nss;
                if (dt == ORACLE_F16) st_f16(pd, ld_f16(pd) + ld_f16(ps));
                else if (dt == ORACLE_F32) st_f32(pd, ld_f32(pd) + ld_f32(ps));
                else st_f64(pd, ld_f64(pd) + ld_f64(ps));
            }
        }
    return bad ? ORACLE_ARGS_NOT_SUPPORT : ORACLE_OK;
}
