// Kernel parameter blocks shared by the host library and the gfx950 kernels.
// Every kernel takes exactly one of these structs by value; the host fills it
// and hands it to hipModuleLaunchKernel as the raw argument buffer.
// Plain C layout only: this header is compiled by g++ (host) and hipcc (device).
#pragma once
#include <stdint.h>

// Unsigned 32-bit division by a launch-time constant: q = n / d for any n.
//   t = mulhi(m, n);  q = (t + ((n - t) >> s1)) >> s2
struct FastDivU32 {
    uint32_t m, s1, s2, d;
};

struct RmsNormParams {
    void *y;
    const void *x;
    const void *w;
    int64_t nsy, nsx;  // row strides in bytes
    uint32_t n, d;
    float epsilon;
    uint32_t _pad;
};

struct SwigluParams {
    void *gate;
    const void *up;
    int64_t sgn, sun;  // row strides in bytes
    uint32_t n, d;
    uint32_t total;      // the `_nt` kernels: 16-byte vectors in all, numbered row by row ...
    FastDivU32 per_row;  // ... this many to a row
};

struct RopeParams {
    void *t;
    const void *pos;
    int64_t st, sh, sp;  // token / head / position strides in bytes
    uint32_t nt, nh, dh;
    float theta;
    uint32_t pos_is_u64;
    uint32_t heads_per_block;
    uint32_t tokens_per_block;  // the `_multi` kernels: consecutive tokens a workgroup takes
    // theta^(k / (dh/2)) for k < dh/2, evaluated by the host's powf (what the reference's CPU backend divides by) when
    // dh <= 256; has_den = 0: the kernel evaluates powf itself
    uint32_t has_den;
    float den[128];
};

struct SoftmaxParams {
    void *att;
    int64_t sh, ss;  // head / row strides in bytes
    uint32_t nh, seq, att_len;
    uint32_t causal;
};

#define OPHIP_REARRANGE_MAXD 8
struct RearrangeParams {
    void *dst;
    const void *src;
    uint64_t total;  // number of chunks = count * chunks_per_unit
    uint32_t ndim;
    uint32_t chunks_per_unit;
    FastDivU32 cpu_div;
    FastDivU32 idx_div[OPHIP_REARRANGE_MAXD];
    uint64_t idx[OPHIP_REARRANGE_MAXD];      // idx_strides (units per step of dim q)
    int64_t dst_s[OPHIP_REARRANGE_MAXD];     // bytes
    int64_t src_s[OPHIP_REARRANGE_MAXD];     // bytes
};

// rearrange where the destination is contiguous along one dimension (A) and the source along another (B), unit 2 / 4 / 8
// bytes: tiles of 64 x 64 units through LDS.  Workgroup ids enumerate (outer index, tile of A, tile of B).
struct TransposeParams {
    void *dst;
    const void *src;
    uint32_t len_a, len_b;        // units along A and B
    int64_t dst_b, src_a;         // bytes: destination stride along B, source stride along A (the other two are the unit)
    uint32_t tiles_a, tiles_b;
    uint32_t nouter;              // outer dimensions
    FastDivU32 tiles_div;         // tiles_a * tiles_b
    FastDivU32 tb_div;            // tiles_b
    FastDivU32 outer_div[OPHIP_REARRANGE_MAXD];  // units per step of outer dimension q (innermost outer = 1)
    int64_t outer_dst[OPHIP_REARRANGE_MAXD], outer_src[OPHIP_REARRANGE_MAXD];  // bytes
};

struct SampleParams {
    void *kv;            // ophip_kv_pair*, one per row
    const void *logits;  // rows x n
    void *workspace;     // general path only
    const float *seeds;  // optional per-row draws (device memory); null = `seed` for every row
    int64_t row_stride;  // bytes between rows of logits
    uint32_t n;
    uint32_t k_eff;      // min(top_k, n)
    float temperature, top_p, seed;
    uint32_t npow2;      // general path: n rounded up to a power of two
    // top_k beyond what the single-workgroup kernels sort (or no top_k at all): they try first, with 64, 1024 and then
    // 8192 candidates, and report in the first word of the row's workspace whether those candidates already
    // hold top_p of the probability (0: the result is written; 1: the next kernel in line has to do the row).
    // Bit 0: write that word; bit 1: read it first and leave the row alone if it is 0.
    uint32_t verify_cover;
};

// attention_kv_cached in one pass (attention_decode.hip).  Strides in elements; the v-cache is addressed with the
// k-cache's strides, as in the reference.
struct AttnDecodeParams {
    const void *q;
    void *q_out;  // q again when the reference would overwrite it with the result (its heads and tokens merge), else null
    void *o;
    const void *k_new, *v_new;  // the rows being appended: [nkvh, seq, dh]
    void *k_cache, *v_cache;
    float *partial;  // several chunks: [nkvh][nchunk] blocks of 16 * MT rows x (dh + 2) floats
    int64_t q_sh, q_ss, o_sh, o_ss, kn_sh, kn_ss, vn_sh, vn_ss, kc_sh, kc_ss;
    uint32_t nkvh, group, seq, att, pos, nchunk, causal;
    float scale;
};

// attention in one pass for prefill shapes (attention_prefill.hip).  Strides in elements; dh is contiguous everywhere.
struct AttnPrefillParams {
    const void *q;
    void *q_out;  // q again when the reference would overwrite it with the result (its heads and tokens merge), else null
    void *o;
    const void *k, *v;
    int64_t q_sh, q_ss, o_sh, o_ss, k_sh, k_ss, v_sh, v_ss;
    uint32_t nh, group, seq, att, causal, nblocks;
    float scale;
};

// Canonical GEMM seen by the kernels:
//   D[i, j] = alpha * sum_l P[i, l] * Q[l, j] + beta * D[i, j]
// element strides; exactly one of each operand's two strides is 1.
struct GemmParams {
    void *d;
    const void *p;
    const void *q;
    void *partial;   // f32 [split_k][batch][M][N] when split_k > 1
    void *counters;  // u32 per (batch, column tile), zero between launches; null = separate reduce kernel
    int64_t d_si, d_sj, d_sb;
    int64_t p_si, p_sl, p_sb;
    int64_t q_sl, q_sj, q_sb;
    uint32_t M, N, K, batch;
    float alpha, beta;
    uint32_t read_dst;  // the reference reads C only when beta != 0
    uint32_t split_k;
    uint32_t k_per_split;  // multiple of 32
    // gemm_stream only: strips whose first 256-byte granule has its class (address bits 8..10) in `slow_mask` are cut
    // into `split_slow` K ranges of ceil(K / 32 / split_slow) steps, the others into `split_k`; mask 0: all alike
    uint32_t slow_mask;
    uint32_t split_slow;
};

// gemm_stream's work units, numbered the same way by the kernel (blockIdx.x -> unit) and by the host (grid size; a
// CPU test walks every unit of a launch through this function before any launch does).
#if defined(__HIPCC__)
#define OPHIP_HD __host__ __device__
#else
#define OPHIP_HD
#endif
struct GemmStreamUnit {
    uint32_t strip;         // 128-column strip
    uint32_t range;         // which of the strip's K ranges
    uint32_t ranges;        // how many K ranges the strip has
    uint32_t kbeg, kend;    // the range: rows [kbeg, kend), in whole steps of 32; empty if kend <= kbeg
    uint32_t valid;         // 0: the block has no unit (the last group of eight strips is short)
};
// K ranges of a strip whose first 256-byte granule has class `cls` (address bits 8..10)
static inline OPHIP_HD uint32_t gemm_stream_ranges(const struct GemmParams *p, uint32_t cls) {
    return (p->slow_mask >> (cls & 7)) & 1 ? p->split_slow : p->split_k;
}
// Unit of workgroup `block` (blockIdx.x); `q_addr` = address of Q's first element for the batch entry.
// Mask 0: strip-major inside each K range (block = range * strips + strip), every strip in split_k ranges of
// k_per_split rows.  Otherwise: groups of eight consecutive strips, inside a group strip by strip, a strip's ranges
// next to each other; a strip in n ranges has ranges of ceil(K / 32 / n) steps.
static inline OPHIP_HD struct GemmStreamUnit gemm_stream_unit(const struct GemmParams *p, uint64_t q_addr, uint32_t block) {
    struct GemmStreamUnit u;
    const uint32_t nstrips = (p->N + 127) / 128;
    uint32_t k_per = p->k_per_split;
    u.valid = 1;
    if (p->slow_mask == 0) {
        u.strip = block % nstrips;
        u.range = block / nstrips;
        u.ranges = p->split_k;
    } else {
        const uint32_t g0 = (uint32_t)(q_addr >> 8);  // class of strip 0's first granule (strips are 256 bytes wide)
        uint32_t per8 = 0;
        for (uint32_t c = 0; c < 8; ++c) per8 += gemm_stream_ranges(p, g0 + c);
        uint32_t r = block % per8;
        u.strip = block / per8 * 8;
        u.ranges = 1;
        for (uint32_t c = 0; c < 8; ++c) {
            u.ranges = gemm_stream_ranges(p, g0 + c);
            if (r < u.ranges) break;
            r -= u.ranges;
            ++u.strip;
        }
        u.range = r;
        if (u.strip >= nstrips) u.valid = 0;
        k_per = (p->K / 32 + u.ranges - 1) / u.ranges * 32;
    }
    if (u.range >= u.ranges) u.valid = 0;  // (a grid larger than the units)
    const uint64_t kb = (uint64_t)u.range * k_per;
    u.kbeg = kb < p->K ? (uint32_t)kb : p->K;
    u.kend = (uint64_t)u.kbeg + k_per < p->K ? u.kbeg + k_per : p->K;
    return u;
}
// Workgroups per batch entry of a launch
static inline OPHIP_HD uint32_t gemm_stream_units(const struct GemmParams *p, uint64_t q_addr) {
    const uint32_t nstrips = (p->N + 127) / 128;
    if (p->slow_mask == 0) return nstrips * p->split_k;
    uint32_t per8 = 0;
    for (uint32_t c = 0; c < 8; ++c) per8 += gemm_stream_ranges(p, (uint32_t)(q_addr >> 8) + c);
    return (nstrips + 7) / 8 * per8;
}

// dst[0 .. size) = value, bytes: the first `head` bytes (up to 16-byte alignment) and the last `tail` bytes one at a
// time, `body` 16-byte units between them
struct FillBytesParams {
    void *dst;
    uint64_t body;
    uint32_t head, tail;
    uint32_t value;  // the byte, repeated four times
    uint32_t _pad;
};

// dst[0 .. count) = value, 32-bit words (the split-K arrival counters start at zero)
struct FillU32Params {
    void *dst;
    uint32_t count;
    uint32_t value;
};

struct LayerNormParams {
    void *y;
    const void *x;
    const void *scale;
    const void *bias;
    int64_t nsy, nsx;  // row strides in bytes
    uint32_t n, d;
    float epsilon;
    uint32_t _pad;
};

struct GeluParams {
    void *base;
    int64_t sn;  // row stride in bytes
    uint32_t n, d;
};

// c = a + b over up to OPHIP_REARRANGE_MAXD merged dimensions; item g decodes into one index per
// dimension through idx_div (items per step of that dimension), strides in bytes.
struct AddParams {
    void *c;
    const void *a;
    const void *b;
    uint32_t total;  // items: elements, or 16-byte vectors when `vec`
    uint32_t ndim;
    FastDivU32 idx_div[OPHIP_REARRANGE_MAXD];
    int64_t c_s[OPHIP_REARRANGE_MAXD];
    int64_t a_s[OPHIP_REARRANGE_MAXD];
    int64_t b_s[OPHIP_REARRANGE_MAXD];
};

// dst[b, m, :] += src[idx[b, m], :]
struct AddRowsParams {
    void *dst;
    const void *src;
    const void *idx;
    int64_t bsd, msd, kss, bsi, msi;  // bytes
    uint32_t batch, m, n, k;
    uint32_t idx_is_u64;
    uint32_t _pad;
};
