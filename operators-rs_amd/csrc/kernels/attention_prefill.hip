// attention in one pass for prefill shapes (many query rows per head): o = softmax(q . k^T / sqrt(dh), causal) . v
// with the [nh, seq, att] score matrix never leaving the chip.
//
// The reference builds the operator from up to five launches (attention/operator.rs:143-277: q . k^T into a workspace,
// softmax over it, att . v, copies), and at prefill shapes the score matrix is most of the memory traffic: 268 MB
// written, read, written and read again for 32 heads of 2048 x 2048.  Here a workgroup of four waves owns 128 query rows
// of one head, a wave 32 of them, and walks the keys in tiles of 64 with the running maximum and sum of the rows
// (the usual online softmax):
//
//   * K and V tiles (64 keys x dh) go from global memory through registers into LDS, double-buffered; the next tile's
//     loads are in flight while the current one is multiplied.  One barrier per tile.
//   * Scores are computed transposed, S^T = K . Q^T with v_mfma_f32_32x32x16_f16: A operands are key rows read from LDS
//     16 bytes per lane, B operands the wave's 32 query rows, which stay in registers for the whole kernel.  In the
//     result a lane holds ONE query (lane % 32) and 32 of the tile's 64 keys, so the row maximum and sum are sums over
//     the lane's own registers plus one exchange with lane ^ 32, and every per-row factor is a per-lane scalar.
//   * The probabilities (f16) are packed straight from that result layout into B operands of the second product,
//     O^T = V^T . P^T: which of a lane's keys go to which contraction slot is free as long as V^T uses the same order,
//     and V^T fragments come from the row-major V tile through the transposing LDS read (ds_read_b64_tr_b16): a lane
//     gets four consecutive keys of one dh column per read.  No transposition in registers, no LDS round trip for P.
//   * Causal mask: row i keeps keys <= att - seq + i; tiles beyond the block's last row are never visited.  Blocks are
//     launched last-block-first (the longest first), heads along grid x so that the blocks of a head meet in one XCD's L2.
//
// Results agree with the composite within the f16 bar (scores and probabilities are not rounded to f16 in between;
// the scale is rounded to f16 as the reference's mat_mul rounds alpha).
//
// Compiled twice, like the MFMA GEMMs (gemm_elem.h): on f16 elements as it stands, and with -DGEMM_ELEM_BF16 on bf16
// elements (module `attention_prefill_bf16`, kernel names with `_bf16` appended): the element type decides the two MFMA
// instructions and the rounding of the probabilities and of the output, nothing else.
#include "gemm_elem.h"

typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int AP_BM = 128, AP_BN = 64;

// G = 1: a workgroup of 4 waves walks all key tiles of its 128 rows; two such workgroups share a CU.
// G = 2: a workgroup of 8 waves, two groups of 4 on the same 128 rows: group 0 takes the even key tiles, group 1 the odd
// ones, each with its own LDS buffers and its own threads loading them; at the end group 1 hands its maxima, sums and
// output to group 0 through LDS.  One such workgroup fills a CU.  A workgroup's time halves, which is what a causal
// mask wants when there are about as many workgroups as places for them: the block with the most keys decides.
template <int DH, int G>
__device__ __forceinline__ void attn_prefill(const AttnPrefillParams &p) {
    constexpr int KP = DH + 8;        // halves per K row in LDS: an odd number of 16-byte units, so 16-byte reads of consecutive rows spread
    constexpr int VP = DH + 32;       // halves per V row in LDS: 64 bytes past a multiple of 256, so four consecutive rows cover all banks
    constexpr int CPR = DH / 8;       // 16-byte chunks per row
    constexpr int NCH = AP_BN * CPR / 256;  // chunks per thread and tile
    constexpr int DS = DH / 16, DB = DH / 32;
    constexpr int TILE_HALVES = AP_BN * (KP + VP);
    __shared__ __attribute__((aligned(16))) elem lds[G * 2 * TILE_HALVES];

    const uint32_t grp = G == 1 ? 0 : threadIdx.x / 256;
    const uint32_t tid = threadIdx.x % 256, wave = tid / WAVE, lane = tid % WAVE;
    const uint32_t n32 = lane % 32, h = lane / 32, s16 = lane % 16, b16 = (lane / 16) % 2;
    // blocks go out longest first (the last block of rows has the most keys under a causal mask), heads along x
    const uint32_t head = blockIdx.x, qblock = p.nblocks - 1 - blockIdx.y;
    const uint32_t kvh = head / p.group;
    const uint32_t i0 = qblock * AP_BM;
    const uint32_t row = i0 + wave * 32 + n32, rowc = min(row, p.seq - 1);
    elem *const k_lds = lds + grp * 2 * TILE_HALVES;          // [2][AP_BN * KP]
    elem *const v_lds = k_lds + 2 * AP_BN * KP;               // [2][AP_BN * VP]

    const elem *qb = reinterpret_cast<const elem *>(p.q) + (int64_t)head * p.q_sh;
    const elem *kb = reinterpret_cast<const elem *>(p.k) + (int64_t)kvh * p.k_sh;
    const elem *vb = reinterpret_cast<const elem *>(p.v) + (int64_t)kvh * p.v_sh;

    // the wave's queries as B operands: lane (n32, h) holds query row n32, dh slots 16 ds + 8 h .. + 7
    PackE qf[DS];
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) qf[ds].u = ld128(qb + (int64_t)rowc * p.q_ss + 16 * ds + 8 * h);

    // keys this block needs: up to the last row's limit
    const uint32_t last_row = min(i0 + AP_BM, p.seq) - 1;
    const uint32_t keys = p.causal ? min(p.att, p.att - p.seq + last_row + 1) : p.att;
    const uint32_t ntiles = (keys + AP_BN - 1) / AP_BN;
    // the last key this lane's row keeps
    const int32_t lim = p.causal ? (int32_t)(p.att - p.seq + rowc) : (int32_t)p.att - 1;
    const int32_t lim_first = __builtin_amdgcn_readfirstlane(lim);  // the wave's smallest: its first row's

    // The thread's chunks of a tile: byte offsets from the tile's first key (32 bits: the host checks that 64 rows of k
    // and v span less than 2 GiB), so that a load is a uniform base plus a lane offset.  Only a last tile that reaches
    // past att clamps its rows.
    u32x4 kreg[NCH], vreg[NCH];
    uint32_t koff[NCH], voff[NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = tid + 256 * i, r = c / CPR, cc = c % CPR;
        koff[i] = (r * (uint32_t)p.k_ss + 8 * cc) * 2;
        voff[i] = (r * (uint32_t)p.v_ss + 8 * cc) * 2;
    }
    auto fetch = [&](uint32_t t) {
        const char *kt = reinterpret_cast<const char *>(kb + (int64_t)(t * AP_BN) * p.k_ss);
        const char *vt = reinterpret_cast<const char *>(vb + (int64_t)(t * AP_BN) * p.v_ss);
        if (t * AP_BN + AP_BN <= p.att) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                kreg[i] = ld128(kt + koff[i]);
                vreg[i] = ld128(vt + voff[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const uint32_t c = tid + 256 * i, r = min(c / CPR, p.att - 1 - t * AP_BN), cc = c % CPR;
                kreg[i] = ld128(kt + (r * (uint32_t)p.k_ss + 8 * cc) * 2);
                vreg[i] = ld128(vt + (r * (uint32_t)p.v_ss + 8 * cc) * 2);
            }
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const uint32_t c = tid + 256 * i, r = c / CPR, cc = c % CPR;
            st128(k_lds + buf * (AP_BN * KP) + r * KP + 8 * cc, kreg[i]);
            st128(v_lds + buf * (AP_BN * VP) + r * VP + 8 * cc, vreg[i]);
        }
    };

    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    constexpr float LOG2E = 1.4426950408889634f;
    const float sc2 = p.scale * LOG2E;  // scores in units of log2 (positive: maxima commute with it)

    // this group's tiles: grp, grp + G, ...  (a group without tiles still meets every barrier)
    if (grp < ntiles) {
        fetch(grp);
        commit(0);
    }
    __syncthreads();
    for (uint32_t u = 0; u * G < ntiles; ++u) {
        const uint32_t t = u * G + grp;
        const int buf = u & 1;
        if (t < ntiles) {
            const bool more = t + G < ntiles;
            if (more) fetch(t + G);
            const elem *kt = k_lds + buf * (AP_BN * KP), *vt = v_lds + buf * (AP_BN * VP);

            // S^T = K . Q^T: sacc[kb][e] is key 32 kb + 8 (e / 4) + 4 h + e % 4 of the tile, query n32
            f32x16 sacc[2];
#pragma unroll
            for (int kb2 = 0; kb2 < 2; ++kb2) {
#pragma unroll
                for (int e = 0; e < 16; ++e) sacc[kb2][e] = 0.f;
#pragma unroll
                for (int ds = 0; ds < DS; ++ds) {
                    PackE a;
                    a.u = ld128(kt + (32 * kb2 + n32) * KP + 16 * ds + 8 * h);
                    sacc[kb2] = mfma_32x32x16(a.h, qf[ds].h, sacc[kb2]);
                }
            }
            // mask (only a tile that reaches past the wave's first limit has anything to mask), the tile's maximum for
            // this lane's query
            if ((int32_t)(t * AP_BN) + AP_BN - 1 > lim_first) {
#pragma unroll
                for (int kb2 = 0; kb2 < 2; ++kb2)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int32_t key = (int32_t)(t * AP_BN) + 32 * kb2 + 8 * (e / 4) + 4 * (int32_t)h + (e % 4);
                        if (key > lim) sacc[kb2][e] = -INFINITY;
                    }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int kb2 = 0; kb2 < 2; ++kb2)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sacc[kb2][e]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
            const float m_new = fmaxf(m_run, mx * sc2);
            const float m_ref = m_new == -INFINITY ? 0.f : m_new;  // (a row with nothing kept so far: every term below is 0)
            // a new maximum in any of the wave's rows: the sums and the output so far shrink by 2^(old - new)
            if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
                l_run *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int e = 0; e < 16; ++e) oacc[db][e] *= alpha;
                m_run = m_new;
            }
            float psum = 0.f;
            // probabilities, packed for the second product: MFMA j covers the tile's keys 16 j .. 16 j + 15; the lane's eight
            // contraction slots 8 h .. 8 h + 7 hold keys 16 j + 4 h + {0..3} and 16 j + 8 + 4 h + {0..3}
            PackE pb[4];
#pragma unroll
            for (int kb2 = 0; kb2 < 2; ++kb2)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb2][e], sc2, -m_ref));
                    psum += pr;
                    pb[2 * kb2 + e / 8].e[e % 8] = f2e(pr);
                }
            l_run += psum;

            // O^T += V^T . P^T: the A operand's row is dh column 32 db + lane % 32; a transposing read hands a lane four
            // consecutive keys of that column (the lanes of a 16-lane group address key s16 / 4, columns 4 (s16 % 4) .. + 3)
            typedef __attribute__((address_space(3))) s16x4 *lds_s16x4;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const elem *src = vt + (16 * j + 4 * h + s16 / 4) * VP + 32 * db + 16 * b16 + 4 * (s16 % 4);
                    union {
                        s16x4 q[2];
                        elem8 hv;
                    } a;
                    a.q[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)src);
                    a.q[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)(src + 8 * VP));
                    oacc[db] = mfma_32x32x16(a.hv, pb[j].h, oacc[db]);
                }

            if (more) commit(buf ^ 1);
        }
        __syncthreads();
    }

    float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
    if constexpr (G == 2) {
        // group 1 hands over through LDS (the tiles are done with: the loop ended on a barrier): value j of lane l of wave
        // w at float (w * (2 + 16 DB) + j) * 64 + l
        float *x = reinterpret_cast<float *>(lds) + wave * (2 + 16 * DB) * WAVE + lane;
        if (grp == 1) {
            x[0] = m_run;
            x[WAVE] = l_tot;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int e = 0; e < 16; ++e) x[(2 + 16 * db + e) * WAVE] = oacc[db][e];
        }
        __syncthreads();
        if (grp == 1) return;
        const float m1 = x[0], l1 = x[WAVE];
        const float m = fmaxf(m_run, m1);  // finite: group 0 has the first tile, in which every row keeps key 0
        const float a0 = __builtin_amdgcn_exp2f(m_run - m), a1 = __builtin_amdgcn_exp2f(m1 - m);
        l_tot = l_tot * a0 + l1 * a1;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[db][e] = oacc[db][e] * a0 + x[(2 + 16 * db + e) * WAVE] * a1;
    }

    // o = O^T / l: the lane holds, for its query, columns 32 db + 8 (e / 4) + 4 h + e % 4: four adjacent ones per e / 4
    const float inv = 1.0f / l_tot;
    if (row < p.seq) {
        elem *orow = reinterpret_cast<elem *>(p.o) + (int64_t)head * p.o_sh + (int64_t)row * p.o_ss;
        elem *qrow = p.q_out ? reinterpret_cast<elem *>(p.q_out) + (int64_t)head * p.q_sh + (int64_t)row * p.q_ss : nullptr;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                union {
                    elem e[4];
                    u32x2 u;
                } o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o.e[r] = f2e(oacc[db][4 * g + r] * inv);
                const uint32_t col = 32 * db + 8 * g + 4 * h;
                *reinterpret_cast<u32x2 *>(orow + col) = o.u;
                if (qrow) *reinterpret_cast<u32x2 *>(qrow + col) = o.u;
            }
    }
}

// (two waves per SIMD: two workgroups of four waves per CU, or one of eight; one wave multiplies while the other does its
// exponentials)
extern "C" __global__ void __launch_bounds__(256, 2) GEMM_KERNEL(attn_prefill_d128)(AttnPrefillParams p) { attn_prefill<128, 1>(p); }
extern "C" __global__ void __launch_bounds__(256, 2) GEMM_KERNEL(attn_prefill_d64)(AttnPrefillParams p) { attn_prefill<64, 1>(p); }
extern "C" __global__ void __launch_bounds__(512) GEMM_KERNEL(attn_prefill_d128_g2)(AttnPrefillParams p) { attn_prefill<128, 2>(p); }
extern "C" __global__ void __launch_bounds__(512) GEMM_KERNEL(attn_prefill_d64_g2)(AttnPrefillParams p) { attn_prefill<64, 2>(p); }
