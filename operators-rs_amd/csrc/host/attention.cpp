// attention and attention_kv_cached on the HIP backend: the two composites that sit
// directly on top of mat_mul, fuesd_softmax and rearrange in the reference
// (attention/operator.rs:1-278, attention_kv_cached/operator.rs:1-184).  They own no
// kernels: they plan workspace, build views and launch the three operators in the
// reference's order, so the work lands on the queue exactly as the crate would put it.
#include <algorithm>
#include <cmath>
#include <cstdlib>

#include "../kernels/params.h"
#include "handle.hpp"

using namespace ophip;

namespace {

// a sub-operator's status code back into an Error, keeping its message
void sub(int code) {
    if (code != OPHIP_OK) throw Error{code, ophip_last_error()};
}

// rank-3 layout with owned shape / strides (bytes), viewable as ophip_tensor_layout
struct Lay3 {
    size_t shape[3];
    ptrdiff_t strides[3];
    ophip_tensor_layout tl(uint64_t dt) const { return ophip_tensor_layout{dt, 3, shape, strides}; }
    static Lay3 contiguous(uint64_t dt, size_t a, size_t b, size_t c) {  // TensorLayout::new_contiguous
        const ptrdiff_t e = (ptrdiff_t)ophip_dtype_nbytes(dt);
        return Lay3{{a, b, c}, {(ptrdiff_t)(b * c) * e, (ptrdiff_t)c * e, e}};
    }
    // rows of c elements, each starting on a 16-byte boundary: what the MFMA mat_mul kernels need of a
    // K-contiguous operand.  The score matrix lives in the operator's own workspace, so its row pitch is
    // the operator's choice (the reference keeps it dense).
    static size_t padded_row(uint64_t dt, size_t c) {
        const size_t e = ophip_dtype_nbytes(dt), per16 = e && 16 % e == 0 ? 16 / e : 1;
        return (c + per16 - 1) / per16 * per16;
    }
    static Lay3 padded_rows(uint64_t dt, size_t a, size_t b, size_t c) {
        const ptrdiff_t e = (ptrdiff_t)ophip_dtype_nbytes(dt), ld = (ptrdiff_t)padded_row(dt, c);
        return Lay3{{a, b, c}, {(ptrdiff_t)b * ld * e, ld * e, e}};
    }
    static Lay3 dyn(size_t a, size_t b, size_t c) {  // TensorLayout::new_dyn with dynamic strides
        return Lay3{{a, b, c}, {OPHIP_DYN_ISIZE, OPHIP_DYN_ISIZE, OPHIP_DYN_ISIZE}};
    }
    static Lay3 of(const ophip_tensor_layout &l) {
        return Lay3{{l.shape[0], l.shape[1], l.shape[2]}, {l.strides[0], l.strides[1], l.strides[2]}};
    }
};

// WorkspaceCollector (common/workspace.rs:54-90): bases first, then the largest sub-operator
// need, each taken only while the running total still fits.
struct WorkspaceCollector {
    std::vector<size_t> base;
    size_t sub_need = 0;
    void push_base(size_t b) { base.push_back(b); }
    void push_sub(size_t s) { sub_need = std::max(sub_need, s); }
    size_t calculate(size_t max_ws) {
        base.push_back(sub_need);
        size_t ans = 0;
        for (size_t s : base) {
            if (s <= max_ws && ans <= max_ws - s) ans += s;
            else return ans;
        }
        return ans;
    }
};

struct AttentionMeta {
    uint64_t dt;
    size_t nh, nkvh, seq, att, dh;
};

// attention/args.rs:60-90
AttentionMeta attention_meta(const ophip_attention_args &a) {
    expect_rank(a.q_layout, "q", 3);
    expect_rank(a.k_layout, "k", 3);
    expect_rank(a.v_layout, "v", 3);
    expect_rank(a.o_layout, "o", 3);
    AttentionMeta m;
    m.dt = type_distinct({a.q_layout.dt, a.k_layout.dt, a.v_layout.dt, a.o_layout.dt});
    m.nh = dim_distinct({a.q_layout.shape[0], a.o_layout.shape[0]});
    m.nkvh = dim_distinct({a.k_layout.shape[0], a.v_layout.shape[0]});
    m.seq = dim_distinct({a.q_layout.shape[1], a.o_layout.shape[1]});
    m.att = dim_distinct({a.k_layout.shape[1], a.v_layout.shape[1]});
    m.dh = dim_distinct({a.q_layout.shape[2], a.k_layout.shape[2], a.v_layout.shape[2], a.o_layout.shape[2]});
    return m;
}

}  // namespace

struct ophip_attention {
    ophip_device *dev;
    ophip_mat_mul *mat_mul = nullptr;
    ophip_fused_softmax *softmax = nullptr;
    ophip_rearrange *rearrange = nullptr;
    // the one-pass kernel for many query rows: [f16 / bf16][dh 64 / 128][4 waves on all key tiles / 8 waves, even and odd key tiles]
    hipFunction_t prefill[2][2][2] = {};
    int key_split = -1;  // OPHIP_ATTN_KEYSPLIT=0|1 keeps one of the two builds (sweeps); read once, here
    // OPHIP_ATTN_FUSED=0 keeps the composite (tests, comparisons), =1 takes the one-pass kernel wherever it applies;
    // read once, here.  Otherwise an estimate of the two times decides (attention_one_pass).
    int fused = -1;
    // the one-pass kernels for decode shapes (few query rows per kv head against many keys; attention_kv_cached uses them
    // through its own attention operator): [f16 / bf16][16 * {1, 2, 4} query rows per kv head][dh 64 / 128]
    hipFunction_t decode[2][3][2][2], combine[2][3][2];  // decode: [..][..][..][256 / 128 keys per workgroup]
    bool one_pass = true;  // OPHIP_ATTN_ONE_PASS=0 keeps the composite (tests, comparisons); read once, here
    int force_chunk = 0;   // OPHIP_ATTN_CHUNK=256|128 keeps one chunk size (sweeps)
    explicit ophip_attention(ophip_device *d) : dev(d) {
        ophip_device_retain(d);
        try {
            sub(ophip_mat_mul_create(d, &mat_mul));
            sub(ophip_fused_softmax_create(d, &softmax));
            sub(ophip_rearrange_create(d, &rearrange));
            for (int e = 0; e < 2; ++e) {
                const std::string mod = e ? "attention_prefill_bf16" : "attention_prefill", tag = e ? "_bf16" : "";
                prefill[e][0][0] = d->kernel(mod.c_str(), ("attn_prefill_d64" + tag).c_str());
                prefill[e][1][0] = d->kernel(mod.c_str(), ("attn_prefill_d128" + tag).c_str());
                prefill[e][0][1] = d->kernel(mod.c_str(), ("attn_prefill_d64_g2" + tag).c_str());
                prefill[e][1][1] = d->kernel(mod.c_str(), ("attn_prefill_d128_g2" + tag).c_str());
            }
            static const char *mt_tag[3] = {"m1", "m2", "m4"}, *dh_tag[2] = {"d64", "d128"};
            for (int e = 0; e < 2; ++e)
                for (int i = 0; i < 3; ++i)
                    for (int j = 0; j < 2; ++j) {
                        const std::string mod = e ? "attention_decode_bf16" : "attention_decode", tag = e ? "_bf16" : "";
                        const std::string tail = std::string(mt_tag[i]) + "_" + dh_tag[j];
                        decode[e][i][j][0] = d->kernel(mod.c_str(), ("attn_decode_" + tail + "_k64" + tag).c_str());
                        decode[e][i][j][1] = d->kernel(mod.c_str(), ("attn_decode_" + tail + "_k32" + tag).c_str());
                        combine[e][i][j] = d->kernel(mod.c_str(), ("attn_decode_combine_" + tail + tag).c_str());
                    }
            if (const char *e = std::getenv("OPHIP_ATTN_ONE_PASS")) one_pass = std::atoi(e) != 0;
            if (const char *e = std::getenv("OPHIP_ATTN_CHUNK")) force_chunk = std::atoi(e);
            if (const char *e = std::getenv("OPHIP_ATTN_FUSED")) fused = std::atoi(e) != 0;
            if (const char *e = std::getenv("OPHIP_ATTN_KEYSPLIT")) key_split = std::atoi(e) != 0;
        } catch (...) {
            release();
            throw;
        }
    }
    void release() {
        ophip_mat_mul_destroy(mat_mul);
        ophip_fused_softmax_destroy(softmax);
        ophip_rearrange_destroy(rearrange);
        ophip_device_release(dev);
    }
    ~ophip_attention() { release(); }
    ophip_attention(const ophip_attention &) = delete;
    ophip_attention &operator=(const ophip_attention &) = delete;
};

namespace {

// Keys per workgroup of the one-pass kernel: 256, or 128 when that leaves CUs without a workgroup (measured: the
// decode layer, 32 kv heads x 2048 keys, 15.5 us with 256 keys against 17.0; 8 kv heads x 4096 keys 12.3 against 10.7).
size_t decode_chunk(size_t nkvh, size_t att, unsigned cus, int force) {
    if (force == 256 || force == 128) return (size_t)force;
    return (att + 255) / 256 * nkvh < (size_t)cus ? 128 : 256;
}

// Workspace of the one-pass kernel for these sizes, or SIZE_MAX when it does not serve them (the shapes alone
// decide here; launch also looks at strides and alignment).
size_t one_pass_workspace(uint64_t dt, size_t nh, size_t nkvh, size_t seq, size_t att, size_t dh, size_t chunk) {
    if ((dt != OPHIP_DT_F16 && dt != OPHIP_DT_BF16) || (dh != 64 && dh != 128) || nkvh == 0 || nh % nkvh != 0 || seq == 0 || att == 0) return SIZE_MAX;
    const size_t rows = nh / nkvh * seq;
    if (rows > 64 || att > 0x7fffffffu) return SIZE_MAX;
    const size_t nchunk = (att + chunk - 1) / chunk, rp = rows <= 16 ? 16 : rows <= 32 ? 32 : 64;
    return nchunk == 1 ? 0 : nkvh * nchunk * rp * (dh + 2) * sizeof(float);
}

// Operator::scheme (attention/operator.rs:46-141)
size_t attention_scheme(ophip_attention *op, const ophip_attention_args &args, size_t max_ws) {
    const AttentionMeta m = attention_meta(args);
    size_t need = 0;
    WorkspaceCollector wc;
    if (is_dyn(m.nh) || is_dyn(m.seq) || is_dyn(m.att) || is_dyn(m.dh)) {
        // not all of nh, seq, att, dh known: initialise the operators with placeholders
        const Lay3 any = Lay3::dyn(OPHIP_DYN_USIZE, OPHIP_DYN_USIZE, OPHIP_DYN_USIZE);
        const ophip_mat_mul_args mm{any.tl(m.dt), nullptr, 1.f, any.tl(m.dt), nullptr, any.tl(m.dt), nullptr, 1.f};
        sub(ophip_mat_mul_scheme(op->mat_mul, &mm, max_ws, &need));
        wc.push_sub(need);
        const Lay3 att = Lay3::dyn(m.nh, m.seq, m.att);
        const ophip_fused_softmax_args sm{args.mask, att.tl(m.dt), nullptr};
        sub(ophip_fused_softmax_scheme(op->softmax, &sm, max_ws, &need));
        wc.push_sub(need);
        const ophip_rearrange_args re{any.tl(m.dt), nullptr, any.tl(m.dt), nullptr};
        sub(ophip_rearrange_scheme(op->rearrange, &re, max_ws, &need));
        wc.push_sub(need);
        return wc.calculate(max_ws);
    }
    const size_t ele = ophip_dtype_nbytes(m.dt);
    const Lay3 att = Lay3::padded_rows(m.dt, m.nh, m.seq, m.att);
    const size_t q_size = m.nh * m.seq * m.dh * ele, att_size = m.nh * m.seq * Lay3::padded_row(m.dt, m.att) * ele;
    const size_t rest = max_ws > q_size + att_size ? max_ws - (q_size + att_size) : 0;  // saturating_sub
    wc.push_base(q_size);
    wc.push_base(att_size);
    // att = q . k^T
    const ophip_mat_mul_args qk{att.tl(m.dt), nullptr, 0.f, args.q_layout, nullptr, args.k_layout, nullptr, 1.f};
    sub(ophip_mat_mul_scheme(op->mat_mul, &qk, rest, &need));
    wc.push_sub(need);
    // att = softmax(att)
    const ophip_fused_softmax_args sm{args.mask, att.tl(m.dt), nullptr};
    sub(ophip_fused_softmax_scheme(op->softmax, &sm, rest, &need));
    wc.push_sub(need);
    // q = att . v
    const ophip_mat_mul_args pv{args.q_layout, nullptr, 0.f, att.tl(m.dt), nullptr, args.v_layout, nullptr, 1.f};
    sub(ophip_mat_mul_scheme(op->mat_mul, &pv, rest, &need));
    wc.push_sub(need);
    // o = rearrange(q)
    const ophip_rearrange_args re{args.o_layout, nullptr, args.q_layout, nullptr};
    sub(ophip_rearrange_scheme(op->rearrange, &re, rest, &need));
    wc.push_sub(need);
    size_t ans = wc.calculate(max_ws);
    // a launch of these sizes may run on the decode kernel instead: a workspace that serves either
    if (op->one_pass && !is_dyn(m.nkvh)) {
        const size_t fused = one_pass_workspace(m.dt, m.nh, m.nkvh, m.seq, m.att, m.dh,
                                                decode_chunk(m.nkvh, m.att, (unsigned)op->dev->props.multiProcessorCount, op->force_chunk));
        if (fused != SIZE_MAX && fused <= max_ws) ans = std::max(ans, fused);
    }
    return ans;
}

// The bytes a rank-3 view can touch, as [first, last) addresses (strides in bytes, of either sign; an empty view
// touches nothing).
struct ByteSpan {
    const char *lo, *hi;
};
ByteSpan span_of(const void *base, const size_t (&shape)[3], const ptrdiff_t (&strides)[3], size_t ele) {
    const char *b = static_cast<const char *>(base);
    if (shape[0] == 0 || shape[1] == 0 || shape[2] == 0) return {b, b};
    ptrdiff_t lo = 0, hi = 0;
    for (int i = 0; i < 3; ++i) {
        const ptrdiff_t reach = (ptrdiff_t)(shape[i] - 1) * strides[i];
        (reach < 0 ? lo : hi) += reach;
    }
    return {b + lo, b + hi + (ptrdiff_t)ele};
}
bool spans_apart(const ByteSpan &x, const ByteSpan &y) { return x.lo == x.hi || y.lo == y.hi || x.hi <= y.lo || y.hi <= x.lo; }


// The one-pass kernel (attention_prefill.hip) when it serves this call; false, with nothing done, otherwise.
// `merged`: the reference would use q in place and leave att . v in it.
bool attention_one_pass(const ophip_attention *op, const ophip_attention_args &args, const AttentionMeta &m, bool merged,
                        const ophip_queue_alloc *qa) {
    if (op->fused == 0 || (m.dt != OPHIP_DT_F16 && m.dt != OPHIP_DT_BF16)) return false;
    const size_t nh = static_of(m.nh), nkvh = static_of(m.nkvh), seq = static_of(m.seq), att = static_of(m.att), dh = static_of(m.dh);
    if ((dh != 64 && dh != 128) || nh == 0 || seq == 0 || att == 0 || nh > 0x7fffffffu || seq > 0x7fffffffu || att > 0x7fffffffu) return false;
    if (args.mask != OPHIP_MASK_NONE && args.mask != OPHIP_MASK_CAUSAL) return false;
    if (args.mask == OPHIP_MASK_CAUSAL && att < seq) return false;  // rows that keep no column: the softmax of the composite refuses them
    // A workgroup walks its keys tile after tile (two tiles of 64 per 2.7 us in the eight-wave build at dh 128), so with
    // fewer workgroups than CUs the longest walk is the kernel's time, while the composite pays five launches and
    // four passes over the score matrix (about 24 us + 1.25 us per MB of it: 32 heads of 256 x 4096 108 us, where the
    // eight-wave build takes 88; 8 heads 40 us against 81).  Measured, 32 heads, dh 128, causal, one
    // pass against composite: 16 rows x 2048 keys 42 / 21 us, 128 x 2048 47 / 41, 64 x 64 7 / 16, 256 x 256 13 / 23,
    // 512 x 512 19 / 35, 2048 x 2048 68 / 326.
    const size_t cus = (size_t)op->dev->props.multiProcessorCount;
    const size_t wgs = nh * ((seq + 127) / 128), tiles = (att + 63) / 64;
    if (op->fused < 0 && wgs <= cus) {
        const double walk = 4.0 + (double)((tiles + 1) / 2) * (dh == 128 ? 2.7 : 1.6);
        const double composite = 24.0 + 1.25 * (double)nh * (double)seq * (double)att * 2.0 / 1e6;
        if (walk >= composite) return false;
    }
    struct View {
        const ophip_tensor_layout &l;
        const void *base;
    };
    const View q{args.q_layout, args.q_base}, k{args.k_layout, args.k_base}, v{args.v_layout, args.v_base}, o{args.o_layout, args.o_base};
    // dh contiguous, rows and heads on 16-byte boundaries, no negative strides
    for (const View *t : {&q, &k, &v, &o}) {
        if (!t->base || !aligned16(t->base)) return false;
        const ptrdiff_t s0 = static_of(t->l.strides[0]), s1 = static_of(t->l.strides[1]), s2 = static_of(t->l.strides[2]);
        if (s2 != 2 || s0 < 0 || s1 < 0 || !mult16(s0) || !mult16(s1)) return false;
        if (s1 >= ((ptrdiff_t)1 << 24)) return false;  // the kernel adds 32-bit byte offsets inside a tile of 64 rows
    }
    // o must not lie over anything the other workgroups still read: apart from q itself in q's own layout
    auto span = [](const View &t) {
        return span_of(t.base, {static_of(t.l.shape[0]), static_of(t.l.shape[1]), static_of(t.l.shape[2])},
                       {static_of(t.l.strides[0]), static_of(t.l.strides[1]), static_of(t.l.strides[2])}, 2);
    };
    auto apart = [&](const View &a, const View &b) { return spans_apart(span(a), span(b)); };
    const bool o_is_q = o.base == q.base && static_of(o.l.strides[0]) == static_of(q.l.strides[0]) &&
                        static_of(o.l.strides[1]) == static_of(q.l.strides[1]);
    if (!o_is_q && !apart(o, q)) return false;
    if (!apart(o, k) || !apart(o, v)) return false;
    if (merged && (!apart(q, k) || !apart(q, v))) return false;

    AttnPrefillParams p{};
    p.q = args.q_base;
    p.q_out = merged && !o_is_q ? args.q_base : nullptr;
    p.o = args.o_base;
    p.k = args.k_base;
    p.v = args.v_base;
    p.q_sh = static_of(args.q_layout.strides[0]) / 2;
    p.q_ss = static_of(args.q_layout.strides[1]) / 2;
    p.o_sh = static_of(args.o_layout.strides[0]) / 2;
    p.o_ss = static_of(args.o_layout.strides[1]) / 2;
    p.k_sh = static_of(args.k_layout.strides[0]) / 2;
    p.k_ss = static_of(args.k_layout.strides[1]) / 2;
    p.v_sh = static_of(args.v_layout.strides[0]) / 2;
    p.v_ss = static_of(args.v_layout.strides[1]) / 2;
    p.nh = (uint32_t)nh;
    p.group = (uint32_t)(nh / nkvh);
    p.seq = (uint32_t)seq;
    p.att = (uint32_t)att;
    p.causal = args.mask == OPHIP_MASK_CAUSAL;
    p.nblocks = (uint32_t)((seq + 127) / 128);
    // the reference's mat_mul rounds alpha to the data type
    p.scale = m.dt == OPHIP_DT_BF16 ? round_to_bf16(1.0f / std::sqrt((float)dh)) : round_to_f16(1.0f / std::sqrt((float)dh));
    if (p.nblocks > 65535) return false;
    op->dev->make_current();
    // Under a causal mask the block with the most keys decides once there are no more workgroups than places for
    // them (two per CU): then the eight-wave build, whose workgroups take half as long (32 heads, causal: 2048 x 2048
    // 67.9 against 73.1 us, 512 x 512 19.5 against 21.3; 4096 x 4096 232 against 203, and without a mask it always loses)
    // (and whenever there are fewer workgroups than CUs: a lone workgroup's walk takes 2.7 us per two tiles against 1.75 us per tile)
    const bool split = op->key_split >= 0 ? op->key_split != 0 : wgs <= cus || (p.causal && wgs <= 2 * cus);
    launch(op->prefill[m.dt == OPHIP_DT_BF16 ? 1 : 0][dh == 64 ? 0 : 1][split], Dim3{(unsigned)nh, p.nblocks}, Dim3{split ? 512u : 256u}, 0, stream_of(qa), p);
    return true;
}

// One call of the one-pass decode kernel (attention_decode.hip): q against the first `pos` rows of the caches followed by
// the rows of k_new / v_new, which the kernel also appends to the caches at `pos`; att = keys in all.  With pos = att
// nothing is new and nothing is appended: plain attention over k and v.  As in the reference's attention_kv_cached the
// v-cache is addressed with the k-cache's strides.
struct DecodeCall {
    uint64_t dt;
    int mask;
    size_t nh, nkvh, seq, dh, att, pos;
    const ophip_tensor_layout *q, *o, *k_new, *v_new, *k_cache;
    void *q_base, *o_base;
    const void *k_new_base, *v_new_base;
    void *k_cache_base, *v_cache_base;
};

// The kernel when it serves this call; false, with nothing done, otherwise.
bool decode_one_pass(const ophip_attention *op, const DecodeCall &c, void *workspace, size_t workspace_len, const ophip_queue_alloc *qa) {
    if (!op->one_pass) return false;
    const size_t nh = c.nh, nkvh = c.nkvh, seq = c.seq, dh = c.dh, att = c.att;
    const size_t chunk = decode_chunk(nkvh, att, (unsigned)op->dev->props.multiProcessorCount, op->force_chunk);
    const size_t need = one_pass_workspace(c.dt, nh, nkvh, seq, att, dh, chunk);
    if (need == SIZE_MAX || (c.mask != OPHIP_MASK_NONE && c.mask != OPHIP_MASK_CAUSAL)) return false;
    if (c.mask == OPHIP_MASK_CAUSAL && att < seq) return false;  // rows that keep no column: the softmax of the composite refuses them
    // every tensor: dh contiguous, rows and heads on 16-byte boundaries
    auto fits = [](const ophip_tensor_layout &l, const void *base) {
        for (int i = 0; i < 3; ++i)
            if (is_dyn(l.strides[i])) return false;
        return l.strides[2] == 2 && mult16(l.strides[0]) && mult16(l.strides[1]) && aligned16(base);
    };
    if (!fits(*c.q, c.q_base) || !fits(*c.o, c.o_base) || !fits(*c.k_new, c.k_new_base) || !fits(*c.v_new, c.v_new_base) ||
        !fits(*c.k_cache, c.k_cache_base) || !aligned16(c.v_cache_base))
        return false;
    const size_t group = nh / nkvh, rows = group * seq;
    AttnDecodeParams p{};
    p.q = c.q_base;
    p.o = c.o_base;
    // the reference overwrites q with the result when q's heads and tokens merge (attention/operator.rs:186-239)
    const ptrdiff_t nh_sq = c.q->strides[0], seq_sq = c.q->strides[1];
    const bool merged = nh == 1 || seq == 1 || nh_sq == (ptrdiff_t)seq * seq_sq;
    // A kv head's workgroup writes o (and q, when the reference would) while the workgroups of other kv heads may
    // still read q, the appended rows and the caches: the composite reads all of them before it writes, so a call
    // whose o (or overwritten q) lies over any of them is left to it.  o over q itself, in q's own layout, is fine:
    // a workgroup reads the rows it writes, and no other.
    {
        const size_t fresh = att - c.pos;  // rows of k_new / v_new
        const ByteSpan qs = span_of(c.q_base, {nh, seq, dh}, {c.q->strides[0], c.q->strides[1], 2}, 2);
        const ByteSpan os = span_of(c.o_base, {nh, seq, dh}, {c.o->strides[0], c.o->strides[1], 2}, 2);
        const ByteSpan kn = span_of(c.k_new_base, {nkvh, fresh, dh}, {c.k_new->strides[0], c.k_new->strides[1], 2}, 2);
        const ByteSpan vn = span_of(c.v_new_base, {nkvh, fresh, dh}, {c.v_new->strides[0], c.v_new->strides[1], 2}, 2);
        const ByteSpan kc = span_of(c.k_cache_base, {nkvh, att, dh}, {c.k_cache->strides[0], c.k_cache->strides[1], 2}, 2);
        const ByteSpan vc = span_of(c.v_cache_base, {nkvh, att, dh}, {c.k_cache->strides[0], c.k_cache->strides[1], 2}, 2);
        const bool o_is_q = c.o_base == c.q_base && c.o->strides[0] == c.q->strides[0] && c.o->strides[1] == c.q->strides[1];
        if (!o_is_q && !spans_apart(os, qs)) return false;
        for (const ByteSpan *t : {&kn, &vn, &kc, &vc})
            if (!spans_apart(os, *t) || (merged && !spans_apart(qs, *t))) return false;
    }
    p.q_out = merged && c.q_base != c.o_base ? c.q_base : nullptr;
    p.k_new = c.k_new_base;
    p.v_new = c.v_new_base;
    p.k_cache = c.k_cache_base;
    p.v_cache = c.v_cache_base;
    p.q_sh = nh_sq / 2, p.q_ss = seq_sq / 2;
    p.o_sh = c.o->strides[0] / 2, p.o_ss = c.o->strides[1] / 2;
    p.kn_sh = c.k_new->strides[0] / 2, p.kn_ss = c.k_new->strides[1] / 2;
    p.vn_sh = c.v_new->strides[0] / 2, p.vn_ss = c.v_new->strides[1] / 2;
    p.kc_sh = c.k_cache->strides[0] / 2, p.kc_ss = c.k_cache->strides[1] / 2;
    p.nkvh = (uint32_t)nkvh, p.group = (uint32_t)group, p.seq = (uint32_t)seq, p.att = (uint32_t)att, p.pos = (uint32_t)c.pos;
    p.nchunk = (uint32_t)((att + chunk - 1) / chunk);
    p.causal = c.mask == OPHIP_MASK_CAUSAL;
    // the reference's mat_mul rounds alpha to the data type
    p.scale = c.dt == OPHIP_DT_BF16 ? round_to_bf16(1.0f / std::sqrt((float)dh)) : round_to_f16(1.0f / std::sqrt((float)dh));
    if (p.nchunk > 65535 || nkvh > 65535) return false;
    Workspace ws(qa, workspace, workspace_len, need);
    p.partial = static_cast<float *>(ws.ptr());
    const int mi = rows <= 16 ? 0 : rows <= 32 ? 1 : 2, di = dh == 64 ? 0 : 1, ei = c.dt == OPHIP_DT_BF16 ? 1 : 0;
    op->dev->make_current();
    launch(op->decode[ei][mi][di][chunk == 256 ? 0 : 1], Dim3{p.nchunk, (unsigned)nkvh}, Dim3{256}, 0, stream_of(qa), p);
    if (p.nchunk > 1) launch(op->combine[ei][mi][di], Dim3{(unsigned)(nkvh * rows)}, Dim3{256}, 0, stream_of(qa), p);
    return true;
}

// Operator::launch (attention/operator.rs:143-277).  q is overwritten with att . v, as in
// the reference, unless it had to be copied into the workspace first.
void attention_launch(const ophip_attention *op, const ophip_attention_args &args, void *workspace,
                      size_t workspace_len, const ophip_queue_alloc *qa) {
    const AttentionMeta m = attention_meta(args);
    const uint64_t dt = m.dt;
    const size_t ele = ophip_dtype_nbytes(dt);
    const size_t nh = static_of(m.nh), seq = static_of(m.seq), dh = static_of(m.dh);
    const ptrdiff_t nh_sq = static_of(args.q_layout.strides[0]), seq_sq = static_of(args.q_layout.strides[1]),
                    dh_sq = static_of(args.q_layout.strides[2]);
    const size_t nkvh = static_of(m.nkvh), att = static_of(m.att);
    const ptrdiff_t nkvh_sk = static_of(args.k_layout.strides[0]), att_sk = static_of(args.k_layout.strides[1]),
                    dh_sk = static_of(args.k_layout.strides[2]);
    if (nkvh == 0 || nh % nkvh != 0) throw shape_mismatch("nh must be a multiple of nkvh");
    if (nh != 0 && seq != 0 && dh != 0 && att != 0 && (!args.q_base || !args.k_base || !args.v_base || !args.o_base))
        throw args_not_support("null base address");  // (the one-pass kernels would take them as they are)

    // ArrayLayout::merge_be(0, 2) of ndarray-layout: heads and tokens fold into one dimension
    // when the head stride is seq * token stride (a dimension of length 1 folds with anything)
    const bool merged = nh == 1 || seq == 1 || nh_sq == (ptrdiff_t)seq * seq_sq;
    const ptrdiff_t row_sq = seq == 1 ? nh_sq : seq_sq;  // stride of the merged [nh * seq] dimension
    // Few rows per kv head against k and v of one layout: the decode kernel with nothing to append (unless a knob asks
    // for the composite or for the prefill kernel).
    if (op->fused == -1 && !is_dyn(args.v_layout.strides[0]) && args.v_layout.strides[0] == args.k_layout.strides[0] &&
        args.v_layout.strides[1] == args.k_layout.strides[1]) {
        DecodeCall c{};
        c.dt = dt, c.mask = args.mask;
        c.nh = nh, c.nkvh = nkvh, c.seq = seq, c.dh = dh, c.att = att, c.pos = att;
        c.q = &args.q_layout, c.q_base = args.q_base;
        c.o = &args.o_layout, c.o_base = args.o_base;
        c.k_new = &args.k_layout, c.k_new_base = args.k_base;
        c.v_new = &args.v_layout, c.v_new_base = args.v_base;
        c.k_cache = &args.k_layout, c.k_cache_base = const_cast<void *>(args.k_base);
        c.v_cache_base = const_cast<void *>(args.v_base);
        if (decode_one_pass(op, c, workspace, workspace_len, qa)) return;
    }
    if (attention_one_pass(op, args, m, merged, qa)) return;
    // k^T: ArrayLayout::transpose(&[2, 1])
    const Lay3 kt{{nkvh, dh, att}, {nkvh_sk, dh_sk, att_sk}};

    const size_t q_size = merged ? 0 : nh * seq * dh * ele;
    const size_t att_size = nh * seq * Lay3::padded_row(dt, att) * ele;
    Workspace ws(qa, workspace, workspace_len, q_size + att_size);
    char *q_buf = static_cast<char *>(ws.ptr());
    char *att_buf = q_buf + q_size;
    // what is left of a caller-provided workspace goes to the sub-operators
    const bool ext = ws.ptr() == workspace && workspace_len >= q_size + att_size;
    void *rest = ext ? att_buf + att_size : nullptr;
    const size_t rest_len = ext ? workspace_len - (q_size + att_size) : 0;

    const size_t head_group = nh / nkvh;
    Lay3 q_lay, qx_lay;
    void *q_base;
    if (!merged) {
        q_lay = Lay3::contiguous(dt, nh, seq, dh);
        qx_lay = Lay3::contiguous(dt, nkvh, head_group * seq, dh);
        q_base = q_buf;
        const ophip_rearrange_args re{q_lay.tl(dt), q_base, args.q_layout, args.q_base};
        sub(ophip_rearrange_launch(op->rearrange, &re, rest, rest_len, qa));
    } else {
        // tile_be(0, &[nkvh, head_group * seq]) of the merged dimension
        q_lay = Lay3::of(args.q_layout);
        qx_lay = Lay3{{nkvh, head_group * seq, dh}, {(ptrdiff_t)(head_group * seq) * row_sq, row_sq, dh_sq}};
        q_base = args.q_base;
    }
    const Lay3 att_mm = Lay3::padded_rows(dt, nkvh, head_group * seq, att);
    const Lay3 att_sm = Lay3::padded_rows(dt, nh, seq, att);

    // att = q . k^T
    const ophip_mat_mul_args qk{att_mm.tl(dt), att_buf, 0.f, qx_lay.tl(dt), q_base, kt.tl(dt), args.k_base,
                                1.0f / std::sqrt((float)dh)};
    sub(ophip_mat_mul_launch(op->mat_mul, &qk, rest, rest_len, qa));
    // att = softmax(att)
    const ophip_fused_softmax_args sm{args.mask, att_sm.tl(dt), att_buf};
    sub(ophip_fused_softmax_launch(op->softmax, &sm, rest, rest_len, qa));
    // q = att . v
    const ophip_mat_mul_args pv{qx_lay.tl(dt), q_base, 0.f, att_mm.tl(dt), att_buf, args.v_layout, args.v_base, 1.f};
    sub(ophip_mat_mul_launch(op->mat_mul, &pv, rest, rest_len, qa));
    // o = rearrange(q)
    if (q_base != args.o_base) {
        const ophip_rearrange_args re{args.o_layout, args.o_base, q_lay.tl(dt), q_base};
        sub(ophip_rearrange_launch(op->rearrange, &re, rest, rest_len, qa));
    }
}

}  // namespace

struct ophip_attention_kv_cached {
    ophip_device *dev;
    ophip_rearrange *rearrange = nullptr;
    ophip_attention *attention = nullptr;
    explicit ophip_attention_kv_cached(ophip_device *d) : dev(d) {
        ophip_device_retain(d);
        try {
            sub(ophip_rearrange_create(d, &rearrange));
            sub(ophip_attention_create(d, &attention));
        } catch (...) {
            release();
            throw;
        }
    }
    void release() {
        ophip_rearrange_destroy(rearrange);
        ophip_attention_destroy(attention);
        ophip_device_release(dev);
    }
    ~ophip_attention_kv_cached() { release(); }
    ophip_attention_kv_cached(const ophip_attention_kv_cached &) = delete;
    ophip_attention_kv_cached &operator=(const ophip_attention_kv_cached &) = delete;
};

namespace {

struct KvCachedMeta {
    uint64_t dt;
    size_t nh, nkvh, dh, seq;
};

// attention_kv_cached/args.rs:72-115
KvCachedMeta kv_cached_meta(const ophip_attention_kv_cached_args &a) {
    expect_rank(a.q_layout, "q", 3);
    expect_rank(a.k_layout, "k", 3);
    expect_rank(a.v_layout, "v", 3);
    expect_rank(a.o_layout, "o", 3);
    expect_rank(a.k_cache_layout, "k_cache", 3);
    expect_rank(a.v_cache_layout, "v_cache", 3);
    KvCachedMeta m;
    m.dt = type_distinct({a.q_layout.dt, a.k_layout.dt, a.v_layout.dt, a.o_layout.dt, a.k_cache_layout.dt,
                          a.v_cache_layout.dt});
    m.nh = dim_distinct({a.q_layout.shape[0], a.o_layout.shape[0]});
    m.nkvh = dim_distinct({a.k_layout.shape[0], a.v_layout.shape[0], a.k_cache_layout.shape[0],
                           a.v_cache_layout.shape[0]});
    m.dh = dim_distinct({a.q_layout.shape[2], a.k_layout.shape[2], a.v_layout.shape[2], a.o_layout.shape[2],
                         a.k_cache_layout.shape[2], a.v_cache_layout.shape[2]});
    m.seq = dim_distinct({a.q_layout.shape[1], a.k_layout.shape[1], a.v_layout.shape[1], a.o_layout.shape[1]});
    return m;
}

// Operator::scheme (attention_kv_cached/operator.rs:42-77)
size_t kv_cached_scheme(ophip_attention_kv_cached *op, const ophip_attention_kv_cached_args &args, size_t max_ws) {
    const KvCachedMeta m = kv_cached_meta(args);
    WorkspaceCollector wc;
    size_t need = 0;
    const Lay3 any = Lay3::dyn(OPHIP_DYN_USIZE, OPHIP_DYN_USIZE, OPHIP_DYN_USIZE);
    const ophip_rearrange_args re{any.tl(m.dt), nullptr, any.tl(m.dt), nullptr};
    sub(ophip_rearrange_scheme(op->rearrange, &re, max_ws, &need));
    wc.push_sub(need);
    const size_t att = (!is_dyn(m.seq) && !is_dyn(args.pos)) ? args.pos + m.seq : OPHIP_DYN_USIZE;
    // attention::Args::new_null(mask, dt, nh, nkvh, seq, att, dh): every stride dynamic
    const Lay3 qo = Lay3::dyn(m.nh, m.seq, m.dh), kv = Lay3::dyn(m.nkvh, att, m.dh);
    ophip_attention_args at{};
    at.q_layout = at.o_layout = qo.tl(m.dt);
    at.k_layout = at.v_layout = kv.tl(m.dt);
    at.mask = args.mask;
    need = attention_scheme(op->attention, at, max_ws);
    wc.push_sub(need);
    size_t ans = wc.calculate(max_ws);
    // a launch of these sizes may run on the one-pass kernel instead: a workspace that serves either
    if (op->attention->one_pass && !is_dyn(m.nh) && !is_dyn(m.nkvh) && !is_dyn(m.dh) && !is_dyn(att)) {
        const size_t fused = one_pass_workspace(m.dt, m.nh, m.nkvh, m.seq, att, m.dh,
                                                decode_chunk(m.nkvh, att, (unsigned)op->dev->props.multiProcessorCount, op->attention->force_chunk));
        if (fused != SIZE_MAX && fused <= max_ws) ans = std::max(ans, fused);
    }
    return ans;
}

// The one-pass kernel (attention_decode.hip) when it serves this call; false, with nothing done, otherwise.
bool kv_cached_one_pass(const ophip_attention_kv_cached *op, const ophip_attention_kv_cached_args &args, const KvCachedMeta &m,
                        size_t pos, size_t att, void *workspace, size_t workspace_len, const ophip_queue_alloc *qa) {
    DecodeCall c{};
    c.dt = m.dt, c.mask = args.mask;
    c.nh = static_of(m.nh), c.nkvh = static_of(m.nkvh), c.seq = static_of(m.seq), c.dh = static_of(m.dh), c.att = att, c.pos = pos;
    c.q = &args.q_layout, c.q_base = args.q_base;
    c.o = &args.o_layout, c.o_base = args.o_base;
    c.k_new = &args.k_layout, c.k_new_base = args.k_base;
    c.v_new = &args.v_layout, c.v_new_base = args.v_base;
    c.k_cache = &args.k_cache_layout, c.k_cache_base = args.k_cache_base;
    c.v_cache_base = args.v_cache_base;
    return decode_one_pass(op->attention, c, workspace, workspace_len, qa);
}

// Operator::launch (attention_kv_cached/operator.rs:79-183).  As in the reference, the
// v-cache view takes its strides from k_cache_layout (operator.rs:114) and the appended v
// rows land at the k-cache's byte offset (operator.rs:156): the two caches are expected to
// share one layout.
void kv_cached_launch(const ophip_attention_kv_cached *op, const ophip_attention_kv_cached_args &args,
                      void *workspace, size_t workspace_len, const ophip_queue_alloc *qa) {
    const KvCachedMeta m = kv_cached_meta(args);
    const size_t pos = static_of(args.pos), seq = static_of(m.seq);
    const size_t buf_k = static_of(args.k_cache_layout.shape[1]);
    const size_t nkvh = static_of(m.nkvh), buf_v = static_of(args.v_cache_layout.shape[1]), dh = static_of(m.dh);
    const ptrdiff_t nkvh_skc = static_of(args.k_cache_layout.strides[0]),
                    buf_skc = static_of(args.k_cache_layout.strides[1]),
                    dh_skc = static_of(args.k_cache_layout.strides[2]);
    const ptrdiff_t nkvh_svc = nkvh_skc, buf_svc = buf_skc, dh_svc = dh_skc;

    // cache capacity
    const size_t att = pos + seq;
    if (buf_k < att || buf_v < att) throw shape_mismatch("Out of cache buffer");
    if (nkvh != 0 && seq != 0 && dh != 0 && static_of(m.nh) != 0 &&
        (!args.q_base || !args.k_base || !args.v_base || !args.o_base || !args.k_cache_base || !args.v_cache_base))
        throw args_not_support("null base address");  // (the one-pass kernel would take them as they are)
    if (kv_cached_one_pass(op, args, m, pos, att, workspace, workspace_len, qa)) return;
    // concatenate the new rows onto the caches: slice(1, pos, 1, seq)
    const Lay3 k_cat{{nkvh, seq, dh}, {nkvh_skc, buf_skc, dh_skc}};
    const Lay3 v_cat{{nkvh, seq, dh}, {nkvh_svc, buf_svc, dh_svc}};
    const ptrdiff_t cat_offset = (ptrdiff_t)pos * buf_skc;
    const ophip_rearrange_args rk{k_cat.tl(m.dt), static_cast<char *>(args.k_cache_base) + cat_offset, args.k_layout,
                                  args.k_base};
    sub(ophip_rearrange_launch(op->rearrange, &rk, workspace, workspace_len, qa));
    const ophip_rearrange_args rv{v_cat.tl(m.dt), static_cast<char *>(args.v_cache_base) + cat_offset, args.v_layout,
                                  args.v_base};
    sub(ophip_rearrange_launch(op->rearrange, &rv, workspace, workspace_len, qa));
    // attention over rows [0, att) of the caches
    const Lay3 k_all{{nkvh, att, dh}, {nkvh_skc, buf_skc, dh_skc}};
    const Lay3 v_all{{nkvh, att, dh}, {nkvh_svc, buf_svc, dh_svc}};
    ophip_attention_args at{};
    at.q_layout = args.q_layout;
    at.q_base = args.q_base;
    at.k_layout = k_all.tl(m.dt);
    at.k_base = args.k_cache_base;
    at.v_layout = v_all.tl(m.dt);
    at.v_base = args.v_cache_base;
    at.o_layout = args.o_layout;
    at.o_base = args.o_base;
    at.mask = args.mask;
    attention_launch(op->attention, at, workspace, workspace_len, qa);
}

}  // namespace

extern "C" {

int ophip_attention_create(ophip_device *dev, ophip_attention **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_attention(dev);
    });
}
void ophip_attention_destroy(ophip_attention *op) { delete op; }

int ophip_attention_scheme(ophip_attention *op, const ophip_attention_args *args, size_t max_ws, size_t *ws) {
    return guard([&] {
        if (ws) *ws = 0;
        if (!op || !args) throw args_not_support("null argument");
        const size_t need = attention_scheme(op, *args, max_ws);
        if (ws) *ws = need;
    });
}

int ophip_attention_launch(const ophip_attention *op, const ophip_attention_args *args, void *workspace,
                           size_t workspace_len, const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        attention_launch(op, *args, workspace, workspace_len, qa);
    });
}

int ophip_attention_kv_cached_create(ophip_device *dev, ophip_attention_kv_cached **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_attention_kv_cached(dev);
    });
}
void ophip_attention_kv_cached_destroy(ophip_attention_kv_cached *op) { delete op; }

int ophip_attention_kv_cached_scheme(ophip_attention_kv_cached *op, const ophip_attention_kv_cached_args *args,
                                     size_t max_ws, size_t *ws) {
    return guard([&] {
        if (ws) *ws = 0;
        if (!op || !args) throw args_not_support("null argument");
        const size_t need = kv_cached_scheme(op, *args, max_ws);
        if (ws) *ws = need;
    });
}

int ophip_attention_kv_cached_launch(const ophip_attention_kv_cached *op, const ophip_attention_kv_cached_args *args,
                                     void *workspace, size_t workspace_len, const ophip_queue_alloc *qa) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        kv_cached_launch(op, *args, workspace, workspace_len, qa);
    });
}

}  // extern "C"
