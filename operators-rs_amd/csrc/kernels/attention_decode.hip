// attention_kv_cached in one pass over the caches, for the decode shapes (few query rows per kv head).
//
// The reference builds the operator from seven launches (two cache appends, q . k^T, softmax, att . v and up to two
// copies; attention_kv_cached/operator.rs:79-183, attention/operator.rs:143-277) with the [nh, seq, att] score matrix
// in a workspace between them.  At decode shapes the two caches are all the traffic there is, so here every key and
// value is read exactly once and the scores never leave the chip:
//
//   grid (chunk, kv head); a workgroup of 4 waves owns 256 (or 128) keys of one kv head, a wave 64 (32) of them.  The query rows
//   of the kv head's group (head_group * seq rows, up to 64) are the A operands of v_mfma_f32_16x16x32_f16, the keys
//   come from the cache 16 bytes per lane straight into B operands.  The rows' maxima are shared between the waves
//   through LDS, so that all four use one maximum; exp2, the row sums, then the probabilities go through a
//   wave-private LDS tile from the MFMA result layout to the A-operand layout, the values are transposed in the
//   lane's registers (as gemm_skinny does for a weight stored [K, N]) and the second product runs.  The waves' partial
//   outputs are summed through LDS in wave order.
//   One chunk: the workgroup divides by the row sums and writes o (and q, which the reference overwrites when its heads
//   and tokens merge).  Several chunks: it writes its maximum, sum and unnormalised output to the workspace and
//   attn_decode_combine, a second launch, merges them in a fixed order.  (Merging inside the first launch, by the
//   workgroup that arrives last as gemm_skinny's split-K does, was tried: 15.7 against 16.1 us at the decode layer's
//   shape, 22 against 18 us with 56 rows per kv head: not worth the counters.)
//   The rows being appended ([pos, pos + seq) of the caches) are read from k and v themselves, and the wave that holds
//   them writes them to the caches bit for bit; no workgroup reads a cache row that another one writes.
//
// As in the reference the v-cache is addressed with the k-cache's strides (operator.rs:114, 156).
//
// Compiled twice, like the MFMA GEMMs (gemm_elem.h): on f16 elements as it stands, and with -DGEMM_ELEM_BF16 on bf16
// elements (module `attention_decode_bf16`, kernel names with `_bf16` appended).
#include "gemm_elem.h"

constexpr int AD_WAVES = 4;
// KPW, keys per wave (64 or 32; a workgroup takes 4 * KPW keys), is a template parameter: few kv heads or a short
// cache give too few workgroups of 256 keys to keep every CU busy with two of them.

__device__ __forceinline__ void ad_transpose8x8(const u32x4 (&w)[8], u32x4 (&b)[8]) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t lo = w[2 * d][t / 2], hi = w[2 * d + 1][t / 2];
            b[t][d] = (t & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
        }
    }
}

template <int MT, int DH, int AD_KPW>
__device__ __forceinline__ void attn_decode(const AttnDecodeParams &p) {
    constexpr int KS = DH / 32;   // K-steps of q . k^T
    constexpr int NCG = DH / 8;   // 8-column groups of an output row
    constexpr int AD_CHUNK = AD_WAVES * AD_KPW;  // keys per workgroup
    constexpr int AD_P_PITCH = AD_KPW + 8;       // halves per row of the probability tile (an odd number of 16-byte units)
    __shared__ float red[AD_WAVES][32][WAVE];
    __shared__ float s_max[AD_WAVES][16 * MT], s_sum[AD_WAVES][16 * MT];
    __shared__ __attribute__((aligned(16))) elem s_p[AD_WAVES][16 * MT][AD_P_PITCH];

    const uint32_t wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const uint32_t j16 = lane % 16, g = lane / 16;
    const uint32_t chunk = blockIdx.x, kvh = blockIdx.y;
    const uint32_t rows = p.group * p.seq;  // query rows of this kv head: row = head-in-group * seq + token
    const uint32_t key0 = chunk * AD_CHUNK + wave * AD_KPW;

    const elem *qb = reinterpret_cast<const elem *>(p.q);
    const elem *kn = reinterpret_cast<const elem *>(p.k_new) + (int64_t)kvh * p.kn_sh;
    const elem *vn = reinterpret_cast<const elem *>(p.v_new) + (int64_t)kvh * p.vn_sh;
    elem *kc = reinterpret_cast<elem *>(p.k_cache) + (int64_t)kvh * p.kc_sh;
    elem *vc = reinterpret_cast<elem *>(p.v_cache) + (int64_t)kvh * p.kc_sh;
    auto q_row = [&](uint32_t r) {  // r < rows
        const uint32_t hg = r / p.seq, s = r - hg * p.seq;
        return (int64_t)(kvh * p.group + hg) * p.q_sh + (int64_t)s * p.q_ss;
    };

    // q as A operands: lane (j16, g) holds row mt * 16 + j16, dh slots ks * 32 + 8g .. + 7
    u32x4 qa[MT][KS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const elem *src = qb + q_row(min((uint32_t)mt * 16 + j16, rows - 1)) + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qa[mt][ks] = ld128(src + 32 * ks);
    }
    // keys as B operands: MFMA ct covers keys key0 + ct * 16 + j16.  Rows [pos, att) come from k itself and are
    // written to the cache by the lane that holds them.
    u32x4 kb[AD_KPW / 16][KS];
#pragma unroll
    for (int ct = 0; ct < AD_KPW / 16; ++ct) {
        const uint32_t key = key0 + ct * 16 + j16, keyc = min(key, p.att - 1);
        const elem *src = (keyc >= p.pos ? kn + (int64_t)(keyc - p.pos) * p.kn_ss : kc + (int64_t)keyc * p.kc_ss) + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kb[ct][ks] = ld128(src + 32 * ks);
        if (key >= p.pos && key < p.att) {
            elem *dst = kc + (int64_t)key * p.kc_ss + 8 * g;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) st128(dst + 32 * ks, kb[ct][ks]);
        }
    }
    // values, requested now so that they travel while the scores are worked out: lane (j16, g) holds keys
    // key0 + kk * 32 + 8g + r, columns 8 * (j16 % NCG) .. + 7
    const uint32_t cg = j16 % NCG;
    u32x4 vw[AD_KPW / 32][8];
#pragma unroll
    for (int kk = 0; kk < AD_KPW / 32; ++kk)
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const uint32_t key = key0 + kk * 32 + 8 * g + r, keyc = min(key, p.att - 1);
            const elem *src = (keyc >= p.pos ? vn + (int64_t)(keyc - p.pos) * p.vn_ss : vc + (int64_t)keyc * p.kc_ss) + 8 * cg;
            vw[kk][r] = ld128(src);
            if (key >= p.pos && key < p.att && j16 < NCG) st128(vc + (int64_t)key * p.kc_ss + 8 * cg, vw[kk][r]);
        }

    // scores: lane (j16, g) gets rows mt * 16 + 4g + i, key key0 + ct * 16 + j16
    f32x4 sc[MT][AD_KPW / 16];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int ct = 0; ct < AD_KPW / 16; ++ct) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                PackE a, b;
                a.u = qa[mt][ks];
                b.u = kb[ct][ks];
                acc = mfma_16x16x32(a.h, b.h, acc);
            }
            sc[mt][ct] = acc;
        }
    // scale, mask, row maxima of this wave's keys (the 16 lanes of a g hold one row's 64 keys)
    constexpr float LOG2E = 1.44269504088896340736f;
    const float scale2 = p.scale * LOG2E;  // scores in units of log2: exp(x - m) = exp2(x' - m')
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t r = mt * 16 + 4 * g + i, tok = r % p.seq;
            const uint32_t keep = p.causal ? p.att - p.seq + tok + 1 : p.att;  // row r keeps keys [0, keep)
            float m = -INFINITY;
#pragma unroll
            for (int ct = 0; ct < AD_KPW / 16; ++ct) {
                const uint32_t key = key0 + ct * 16 + j16;
                const float v = key < keep ? sc[mt][ct][i] * scale2 : -INFINITY;
                sc[mt][ct][i] = v;
                m = fmaxf(m, v);
            }
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, WAVE));
            if (j16 == 0) s_max[wave][r] = m;
        }
    __syncthreads();
    // one maximum per row for the whole workgroup; probabilities, their sums, and the tile for the second product
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t r = mt * 16 + 4 * g + i;
            float m = s_max[0][r];
#pragma unroll
            for (int w = 1; w < AD_WAVES; ++w) m = fmaxf(m, s_max[w][r]);
            if (m == -INFINITY) m = 0.f;  // no key of this chunk is kept by the row: every term is exp2(-inf) = 0
            float l = 0.f;
#pragma unroll
            for (int ct = 0; ct < AD_KPW / 16; ++ct) {
                const float e = __builtin_amdgcn_exp2f(sc[mt][ct][i] - m);
                l += e;
                s_p[wave][r][ct * 16 + j16] = f2e(e);
            }
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) l += __shfl_xor(l, o, WAVE);
            if (j16 == 0) s_sum[wave][r] = l;
        }
    // (the tile is wave-private and LDS operations of one wave stay in order: no barrier before reading it back)
    f32x4 oc[MT][8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 8; ++t) oc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < AD_KPW / 32; ++kk) {
        u32x4 vb[8];
        ad_transpose8x8(vw[kk], vb);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            PackE a;
            a.u = ld128(&s_p[wave][mt * 16 + j16][kk * 32 + 8 * g]);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                PackE b;
                b.u = vb[t];
                oc[mt][t] = mfma_16x16x32(a.h, b.h, oc[mt][t]);
            }
        }
    }

    // the four waves' outputs summed in wave order; thread (wave, g, j16) then owns row mt * 16 + 4g + wave,
    // columns 8 * j16 .. + 7
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        __syncthreads();
#pragma unroll
        for (int t = 0; t < 8; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][t * 4 + i][lane] = oc[mt][t][i];
        __syncthreads();
        const uint32_t r = mt * 16 + 4 * g + wave;
        if (r >= rows || j16 >= NCG) continue;
        float out[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < AD_WAVES; ++w) s += red[w][t * 4 + wave][lane];
            out[t] = s;
        }
        float m = s_max[0][r], l = 0.f;
#pragma unroll
        for (int w = 1; w < AD_WAVES; ++w) m = fmaxf(m, s_max[w][r]);
#pragma unroll
        for (int w = 0; w < AD_WAVES; ++w) l += s_sum[w][r];
        if (p.nchunk == 1) {
            const float inv = 1.0f / l;
            PackE o;
#pragma unroll
            for (int t = 0; t < 8; ++t) o.e[t] = f2e(out[t] * inv);
            const uint32_t hg = r / p.seq, s = r - hg * p.seq;
            const int64_t h = kvh * p.group + hg;
            st128(reinterpret_cast<elem *>(p.o) + h * p.o_sh + (int64_t)s * p.o_ss + 8 * j16, o.u);
            if (p.q_out) st128(reinterpret_cast<elem *>(p.q_out) + h * p.q_sh + (int64_t)s * p.q_ss + 8 * j16, o.u);
        } else {
            // [kv head][chunk]: 16 * MT rows of DH floats, then per row the pair (maximum, sum)
            float *base = p.partial + ((size_t)kvh * p.nchunk + chunk) * (size_t)(16 * MT) * (DH + 2);
            float *dst = base + (size_t)r * DH + 8 * j16;
            *reinterpret_cast<f32x4 *>(dst) = f32x4{out[0], out[1], out[2], out[3]};
            *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{out[4], out[5], out[6], out[7]};
            if (j16 == 0) *reinterpret_cast<f32x2 *>(base + (size_t)(16 * MT) * DH + 2 * r) = f32x2{m, l};
        }
    }
}

// Merges the chunks of a row: M = max m_c, o = sum_c 2^(m_c - M) o_c / sum_c 2^(m_c - M) l_c.  One workgroup per
// (kv head, row): thread (cl, cg) folds the chunks cl, cl + 16, ... for 8 columns (all its loads of a round in flight
// together), then the 16 partial results of a column group are merged through LDS in a fixed order.
template <int MT, int DH>
__device__ __forceinline__ void attn_decode_combine(const AttnDecodeParams &p) {
    constexpr int NCG = DH / 8, RP = 16 * MT, CL = 16;
    __shared__ float s_part[CL][NCG][10];
    const uint32_t rows = p.group * p.seq;
    const uint32_t r = blockIdx.x % rows, kvh = blockIdx.x / rows;
    const uint32_t cgi = threadIdx.x % 16, cl = threadIdx.x / 16;
    const float *base = p.partial + (size_t)kvh * p.nchunk * (size_t)RP * (DH + 2);
    const size_t cstride = (size_t)RP * (DH + 2);
    float M = -INFINITY, L = 0.f, acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (cgi < NCG) {
        for (uint32_t c = cl; c < p.nchunk; c += CL) {
            const float *b = base + c * cstride;
            const float m = b[(size_t)RP * DH + 2 * r], l = b[(size_t)RP * DH + 2 * r + 1];
            const f32x4 lo = *reinterpret_cast<const f32x4 *>(b + (size_t)r * DH + 8 * cgi);
            const f32x4 hi = *reinterpret_cast<const f32x4 *>(b + (size_t)r * DH + 8 * cgi + 4);
            const float Mn = fmaxf(M, m);
            const float wo = M == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(M - Mn);
            const float wn = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - Mn);
            L = wo * L + wn * l;
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[t] = wo * acc[t] + wn * lo[t], acc[4 + t] = wo * acc[4 + t] + wn * hi[t];
            M = Mn;
        }
        float *mine = s_part[cl][cgi];
        mine[0] = M, mine[1] = L;
#pragma unroll
        for (int t = 0; t < 8; ++t) mine[2 + t] = acc[t];
    }
    __syncthreads();
    if (cl != 0 || cgi >= NCG) return;
    for (uint32_t o = 1; o < CL && o < p.nchunk; ++o) {
        const float *other = s_part[o][cgi];
        const float m = other[0];
        const float Mn = fmaxf(M, m);
        const float wo = M == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(M - Mn);
        const float wn = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - Mn);
        L = wo * L + wn * other[1];
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = wo * acc[t] + wn * other[2 + t];
        M = Mn;
    }
    const float inv = 1.0f / L;
    PackE o;
#pragma unroll
    for (int t = 0; t < 8; ++t) o.e[t] = f2e(acc[t] * inv);
    const uint32_t hg = r / p.seq, s = r - hg * p.seq;
    const int64_t h = kvh * p.group + hg;
    st128(reinterpret_cast<elem *>(p.o) + h * p.o_sh + (int64_t)s * p.o_ss + 8 * cgi, o.u);
    if (p.q_out) st128(reinterpret_cast<elem *>(p.q_out) + h * p.q_sh + (int64_t)s * p.q_ss + 8 * cgi, o.u);
}

#define ATTN_DECODE(MT, DH)                                                                                  \
    extern "C" __global__ void __launch_bounds__(256) GEMM_KERNEL(attn_decode_m##MT##_d##DH##_k64)(AttnDecodeParams p) {   \
        attn_decode<MT, DH, 64>(p);                                                                          \
    }                                                                                                        \
    extern "C" __global__ void __launch_bounds__(256) GEMM_KERNEL(attn_decode_m##MT##_d##DH##_k32)(AttnDecodeParams p) {   \
        attn_decode<MT, DH, 32>(p);                                                                          \
    }                                                                                                        \
    extern "C" __global__ void __launch_bounds__(256) GEMM_KERNEL(attn_decode_combine_m##MT##_d##DH)(AttnDecodeParams p) { \
        attn_decode_combine<MT, DH>(p);                                                                      \
    }
ATTN_DECODE(1, 64)
ATTN_DECODE(2, 64)
ATTN_DECODE(4, 64)
ATTN_DECODE(1, 128)
ATTN_DECODE(2, 128)
ATTN_DECODE(4, 128)
