// mat_mul kernels for gfx950 (f16 storage, f32 accumulation; compiled a second time on bf16 elements, see
// gemm_elem.h: `elem` below is the element type of the build).
//
// Canonical problem (the host maps the reference's column-major descriptor onto it):
//     D[i, j] = alpha * sum_l P[i, l] * Q[l, j] + (read_dst ? beta * D[i, j] : 0)
//
//  gemm_skinny_*  : M <= 64 rows (decode: a handful of tokens against a weight
//                   matrix).  HBM-bound: Q is streamed exactly once with 16-byte
//                   loads straight into MFMA operand registers, P (tiny) comes
//                   from L2, the product runs on v_mfma_f32_16x16x32_f16 (_bf16).
//  gemm_stream_m1 : the same product for M <= 16 against an N-contiguous Q with K in whole steps of 32 (a decode
//                   step's weight GEMMs): 126 registers, so four workgroups fit a CU; loads through buffer
//                   resources (scalar base, scalar row offset, one 32-bit lane offset); no tail code.
//  gemm_generic_* : any strides / alignment, LDS-tiled FMA; the safety net.
//  gemm_splitk_reduce : sums the f32 partials of a split-K skinny launch in a
//                   fixed order and applies alpha / beta.
#include <type_traits>

#include "gemm_elem.h"

// ----------------------------------------------------------- skinny (MFMA) --
//
// Wave tile: 16*MT rows x 128 columns x 32 of K per step.  Lane (j, g) with
// j = lane % 16, g = lane / 16 owns columns n0 + 8j .. 8j+7 and the K-slots
// 8g .. 8g+7 of the step.
//   QMODE 0 (Q is j-contiguous, e.g. W[K, N]): the lane loads 8 rows x 16 bytes,
//     i.e. an 8(k) x 8(j) block, and transposes it inside its own registers
//     (byte-permutes, no LDS, no cross-lane traffic) into eight B operands, one
//     per column offset t.
//   QMODE 1 (Q is l-contiguous, e.g. K-cache used as K^T): one 16-byte load per
//     column offset t already is the B operand.
//   QMODE 2 (Q is l-contiguous and long in l, e.g. a weight stored [N, K]): QMODE 1 reads 64
//     bytes per column and instruction.  Here a wave step is 128 of K x 32 columns: the 16 lanes
//     l % 16 read 256 contiguous bytes of one column, an instruction covers 4 columns, and the
//     tile goes through a wave-private LDS buffer to reach the MFMA operand layout (8 writes and
//     8 reads of 16 bytes per lane and step; LDS operations of one wave stay in order, so the
//     buffer needs no barrier).  Step cg of a K-chunk holds the columns 8n + 2cg + {0, 1},
//     n = 0..15, so the accumulators end up exactly as in the other modes.
// MFMA number t multiplies the 16 rows of P with the 16 columns {n0 + 8j + t};
// after the eight of them a lane holds, for 4 rows, 8 consecutive columns: one
// 16-byte store per row.
// The block's 4 waves take interleaved K-steps and are summed through LDS; with
// split_k > 1 the block writes f32 partials instead of the final tile.

constexpr int SK_WAVES = 4;

// Loads the lane's 8 x 16 bytes of one K-step.  `colc` is the lane's first column
// clamped into the matrix (lanes past N load valid memory and their results are
// dropped at the store), so the steady-state loop carries no branches.
template <int QMODE>
__device__ __forceinline__ void skinny_load_q(const GemmParams &p, const elem *qb, uint32_t kb, uint32_t colc,
                                              uint32_t g, u32x4 (&w)[8]) {
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        if constexpr (QMODE == 0) {
            w[r] = ld128_nt(qb + (int64_t)(kb + 8 * g + r) * p.q_sl + colc);
        } else {
            const uint32_t col = min(colc + r, p.N - 1);
            w[r] = ld128_nt(qb + (int64_t)col * p.q_sj + (kb + 8 * g));
        }
    }
}
// Same, for a final K-step that reaches past kend: rows beyond it read as zero.
template <int QMODE>
__device__ __forceinline__ void skinny_load_q_tail(const GemmParams &p, const elem *qb, uint32_t kb, uint32_t kend,
                                                   uint32_t colc, uint32_t g, u32x4 (&w)[8]) {
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        w[r] = u32x4{0, 0, 0, 0};
        if constexpr (QMODE == 0) {
            const uint32_t k = kb + 8 * g + r;
            if (k < kend) w[r] = ld128_nt(qb + (int64_t)k * p.q_sl + colc);
        } else {
            const uint32_t k = kb + 8 * g, col = min(colc + r, p.N - 1);
            if (k < kend) w[r] = ld128_nt(qb + (int64_t)col * p.q_sj + k);
        }
    }
}

// b[t] = column t of the lane's 8x8 block: (w[0][t], ..., w[7][t])
__device__ __forceinline__ void transpose8x8(const u32x4 (&w)[8], u32x4 (&b)[8]) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t lo = w[2 * d][t / 2], hi = w[2 * d + 1][t / 2];
            b[t][d] = (t & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
        }
    }
}
// The same with each output register written as one byte permute of its two sources (gemm_stream: 32 instructions
// per K-step instead of the shift / mask / or sequences the expression above compiles to, and fewer temporaries).
__device__ __forceinline__ void transpose8x8_perm(const u32x4 (&w)[8], u32x4 (&b)[8]) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
#pragma unroll
        for (int d = 0; d < 4; ++d)
            b[t][d] = __builtin_amdgcn_perm(w[2 * d + 1][t / 2], w[2 * d][t / 2], (t & 1) ? 0x07060302u : 0x05040100u);
    }
}

// Split-K partials cross workgroups that may sit on different XCDs (each with its
// own L2), inside one kernel.  They are moved with write-through / L2-bypassing accesses
// (the sc1 cache policy the compiler gives device-scope relaxed atomics) instead of plain
// accesses plus device-scope fences: a device-scope fence writes back and invalidates the whole
// L2, which is ruinous while the same L2 is streaming weights.
// They go 16 bytes at a time through buffer instructions, which take the cache policy as an operand: a lane's 8
// partial sums are two stores, and 16 lanes write 512 contiguous bytes (as four 64-bit atomic stores per lane the
// hardware counted four times the bytes written).  Offsets are 32-bit: the host keeps this path for workspaces
// below 4 GiB.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t partial_rsrc(void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(base, 0, 0xffffffff, 0x00020000);
}
constexpr int PARTIAL_SC1 = 16;  // the cache-policy operand of the buffer builtins: bit 4 = sc1
__device__ __forceinline__ void partial_store4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, float a, float b, float c, float d) {
    const u32x4 v = {__float_as_uint(a), __float_as_uint(b), __float_as_uint(c), __float_as_uint(d)};
    __builtin_amdgcn_raw_buffer_store_b128(v, r, byte_off, 0, PARTIAL_SC1);
}
__device__ __forceinline__ void partial_load4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, float (&out)[4]) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, PARTIAL_SC1);
#pragma unroll
    for (int t = 0; t < 4; ++t) out[t] = __uint_as_float(v[t]);
}

// D[i, col0 .. col0+7] = alpha * sum + beta * D, rounded once to f16
__device__ __forceinline__ void skinny_store(const GemmParams &p, uint32_t bat, uint32_t i, uint32_t col0,
                                             const float (&sum)[8]) {
    elem *dst = reinterpret_cast<elem *>(p.d) + (int64_t)bat * p.d_sb + (int64_t)i * p.d_si;
    if (p.d_sj == 1) {
        PackE o;
        if (p.read_dst) {
            PackE c;
            c.u = ld128(dst + col0);
#pragma unroll
            for (int t = 0; t < 8; ++t) o.e[t] = f2e(p.beta * e2f(c.e[t]) + p.alpha * sum[t]);
        } else {
#pragma unroll
            for (int t = 0; t < 8; ++t) o.e[t] = f2e(p.alpha * sum[t]);
        }
        st128(dst + col0, o.u);
    } else {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            elem *e = dst + (int64_t)(col0 + t) * p.d_sj;
            float r = p.alpha * sum[t];
            if (p.read_dst) r = p.beta * e2f(*e) + r;
            *e = f2e(r);
        }
    }
}

constexpr int SK_TR_PITCH = 272;  // bytes per LDS row of the QMODE 2 transposition buffer: 256 + 16 (an odd number of 16-byte units)

template <int MT, int QMODE, bool PAIRED>
__device__ __forceinline__ void gemm_skinny(const GemmParams &p) {
    __shared__ float red[SK_WAVES][32][WAVE];
    __shared__ __attribute__((aligned(16))) char tr_all[QMODE == 2 ? SK_WAVES * 32 * SK_TR_PITCH : 16];

    const uint32_t wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const uint32_t j16 = lane % 16, g = lane / 16;
    const uint32_t n0 = blockIdx.x * 128;
    const uint32_t split = blockIdx.y, bat = blockIdx.z;
    const uint32_t kbeg = split * p.k_per_split;
    const uint32_t kend = min(p.K, kbeg + p.k_per_split);
    const uint32_t col0 = n0 + 8 * j16;

    const elem *qb = reinterpret_cast<const elem *>(p.q) + (int64_t)bat * p.q_sb;
    const elem *pb = reinterpret_cast<const elem *>(p.p) + (int64_t)bat * p.p_sb;

    f32x4 acc[MT][8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // rows of P this lane feeds (clamped: rows past M only produce output rows that are never stored)
    const elem *prow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) prow[mt] = pb + (int64_t)min(mt * 16 + j16, p.M - 1) * p.p_si + 8 * g;
    const uint32_t colc = min(col0, p.N - 8);

    if constexpr (QMODE == 2) {
        // The host guarantees: Q l-contiguous, N a multiple of 128, this split's K range a multiple of 128.
        char *tr = tr_all + wave * (32 * SK_TR_PITCH);
        const uint32_t chunks = (kend - kbeg) / 128;
        const uint32_t cnt = chunks > wave ? (chunks - wave + SK_WAVES - 1) / SK_WAVES : 0;  // K-chunks of this wave
        // load t of a step: local column lc = 4t + g = (n, cb) = (lc / 2, lc % 2) -> column n0 + 8n + cb (+ 2cg),
        // 8 of K at 8 * j16; LDS row cb * 16 + n
        const elem *qrow[8];
        uint32_t wr_off[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t lc = 4 * t + g, n = lc / 2, cb = lc % 2;
            qrow[t] = qb + (int64_t)(n0 + 8 * n + cb) * p.q_sj + 8 * j16;
            wr_off[t] = (cb * 16 + n) * SK_TR_PITCH + j16 * 16;
        }
        const uint32_t rd_off = j16 * SK_TR_PITCH + g * 16;  // + cb * 16 rows + kb4 * 64 bytes
        const int64_t cg_stride = 2 * p.q_sj;
        u32x4 wbuf[4][8], a_cur[MT][4], a_nxt[MT][4];
        auto kc_of = [&](uint32_t i) { return kbeg + 128 * (wave + SK_WAVES * min(i, cnt - 1)); };
        auto issue_w = [&](auto U, uint32_t i, int cg) {
            constexpr int u = decltype(U)::value;
            const uint32_t kc = kc_of(i);
#pragma unroll
            for (int t = 0; t < 8; ++t) wbuf[u][t] = ld128_nt(qrow[t] + cg * cg_stride + kc);
        };
        auto issue_a = [&](u32x4(&a)[MT][4], uint32_t i) {
            const uint32_t kc = kc_of(i);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int kb4 = 0; kb4 < 4; ++kb4) a[mt][kb4] = ld128(prow[mt] + kc + 32 * kb4);
        };
        auto compute = [&](auto U, int cg) {
            constexpr int u = decltype(U)::value;
#pragma unroll
            for (int t = 0; t < 8; ++t) st128(tr + wr_off[t], wbuf[u][t]);
            OPHIP_WAVE_LOCKSTEP();
#pragma unroll
            for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                for (int kb4 = 0; kb4 < 4; ++kb4) {
                    PackE bt;
                    bt.u = ld128(tr + rd_off + cb * (16 * SK_TR_PITCH) + kb4 * 64);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        PackE at;
                        at.u = a_cur[mt][kb4];
                        acc[mt][2 * cg + cb] = mfma_16x16x32(at.h, bt.h, acc[mt][2 * cg + cb]);
                    }
                }
        };
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        using I3 = std::integral_constant<int, 3>;
        if (cnt > 0) {
            issue_a(a_cur, 0);
            issue_w(I0{}, 0, 0);
            issue_w(I1{}, 0, 1);
            issue_w(I2{}, 0, 2);
            // Four steps (one K-chunk) per trip; the loads of the next three steps are in flight.  Past the
            // last chunk the loads fetch it again and nobody uses them.
            for (uint32_t i = 0; i < cnt; ++i) {
                issue_w(I3{}, i, 3);
                issue_a(a_nxt, i + 1);
                compute(I0{}, 0);
                issue_w(I0{}, i + 1, 0);
                compute(I1{}, 1);
                issue_w(I1{}, i + 1, 1);
                compute(I2{}, 2);
                issue_w(I2{}, i + 1, 2);
                compute(I3{}, 3);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int kb4 = 0; kb4 < 4; ++kb4) a_cur[mt][kb4] = a_nxt[mt][kb4];
            }
        }
    } else {
    auto step = [&](const u32x4(&w)[8], const u32x4(&a)[MT]) {
            u32x4 b[8];
            if constexpr (QMODE == 0) {
                transpose8x8(w, b);
            } else {
#pragma unroll
                for (int t = 0; t < 8; ++t) b[t] = w[t];
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                PackE bt;
                bt.u = b[t];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    PackE at;
                    at.u = a[mt];
                    acc[mt][t] = mfma_16x16x32(at.h, bt.h, acc[mt][t]);
                }
            }
        };

        if constexpr (PAIRED) {
            // Full K-steps run through a ring of three register buffers: while one step is
            // being multiplied, the loads of the next two are in flight (16 KB per wave).
            // The full steps are dealt to the waves in pairs (steps 2i, 2i + 1 go to wave i % 4): a lane's two
            // 16-byte reads of P for a pair are the two halves of one 128-byte line.  (P comes from L2 and its
            // requests compete with the weight stream for the CU's outstanding misses: without them the
            // kernel runs 6 % faster at 16 rows and 20 % at 48.)
            const uint32_t nfull = (kend - kbeg) / 32, kfull = kbeg + nfull * 32;  // full steps, and where they end
            const uint32_t npair = nfull / 2;
            const uint32_t cnt = 2 * (npair > wave ? (npair - wave + SK_WAVES - 1) / SK_WAVES : 0) +
                                 ((nfull & 1) && npair % SK_WAVES == wave ? 1 : 0);  // full steps of this wave
            // P is requested a pair at a time, both halves of its 128-byte lines back to back (the second request
            // finds the line on its way; a ring slot later the weight stream would have pushed it out of L1 again),
            // and waits in its own ring of three pairs.
            u32x4 wbuf[3][8], abuf[3][2][MT];
            // step number S6 = idx % 6 of this wave: weight buffer S6 % 3, P pair (S6 / 2) % 3, half S6 % 2
            auto issue = [&](auto S6, uint32_t idx) {
                constexpr int s6 = decltype(S6)::value, u = s6 % 3, ps = (s6 / 2) % 3;
                const uint32_t kb = kbeg + 64 * wave + (64 * SK_WAVES) * (idx / 2) + 32 * (idx & 1);
                if constexpr (s6 % 2 == 0) {
    #pragma unroll
                    for (int mt = 0; mt < MT; ++mt) abuf[ps][0][mt] = ld128(prow[mt] + kb);
                    if (idx + 1 < cnt) {  // wave-uniform: the pair's second step exists
    #pragma unroll
                        for (int mt = 0; mt < MT; ++mt) abuf[ps][1][mt] = ld128(prow[mt] + kb + 32);
                    }
                }
                skinny_load_q<QMODE>(p, qb, kb, colc, g, wbuf[u]);
            };
            auto compute = [&](auto S6) {
                constexpr int s6 = decltype(S6)::value;
                step(wbuf[s6 % 3], abuf[(s6 / 2) % 3][s6 % 2]);
            };
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            using I3 = std::integral_constant<int, 3>;
            using I4 = std::integral_constant<int, 4>;
            using I5 = std::integral_constant<int, 5>;
            uint32_t done = 0;  // a multiple of 6 throughout; steps done and done + 1 are in flight
            if (cnt > 0) issue(I0{}, 0);
            if (cnt > 1) issue(I1{}, 1);
            while (done + 8 <= cnt) {
                issue(I2{}, done + 2); compute(I0{});
                issue(I3{}, done + 3); compute(I1{});
                issue(I4{}, done + 4); compute(I2{});
                issue(I5{}, done + 5); compute(I3{});
                issue(I0{}, done + 6); compute(I4{});
                issue(I1{}, done + 7); compute(I5{});
                done += 6;
            }
            // at most 7 steps are left: the same sequence, each part only if its step exists
            const uint32_t left = cnt - done;
            if (left > 2) issue(I2{}, done + 2);
            if (left > 0) compute(I0{});
            if (left > 3) issue(I3{}, done + 3);
            if (left > 1) compute(I1{});
            if (left > 4) issue(I4{}, done + 4);
            if (left > 2) compute(I2{});
            if (left > 5) issue(I5{}, done + 5);
            if (left > 3) compute(I3{});
            if (left > 6) issue(I0{}, done + 6);
            if (left > 4) compute(I4{});
            if (left > 5) compute(I5{});
            if (left > 6) compute(I0{});

            if (kfull < kend && (nfull / 2) % SK_WAVES == wave) {  // the ragged last step belongs to exactly one wave
                const uint32_t kb = kfull;
    #pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    abuf[0][0][mt] = u32x4{0, 0, 0, 0};
                    if (kb + 8 * g + 8 <= kend) {
                        abuf[0][0][mt] = ld128(prow[mt] + kb);
                    } else if (kb + 8 * g < kend) {  // K cuts this group of 8 (K % 8 != 0): element by element
                        const uint16_t *h = reinterpret_cast<const uint16_t *>(prow[mt] + kb);
    #pragma unroll
                        for (int e = 0; e < 7; ++e)
                            if (kb + 8 * g + e < kend) abuf[0][0][mt][e / 2] |= (uint32_t)h[e] << (16 * (e & 1));
                    }
                }
                skinny_load_q_tail<QMODE>(p, qb, kb, kend, colc, g, wbuf[0]);
                step(wbuf[0], abuf[0][0]);
            }
        } else {
            // Full K-steps run through a ring of three register buffers: while one step is
            // being multiplied, the loads of the next two are in flight (16 KB per wave).
            const uint32_t kfull = kbeg + (kend - kbeg) / 32 * 32;  // end of the full steps
            constexpr uint32_t STRIDE = 32 * SK_WAVES;
            const uint32_t kb0 = kbeg + 32 * wave;
            const uint32_t cnt = kfull > kb0 ? (kfull - kb0 + STRIDE - 1) / STRIDE : 0;  // full steps of this wave
            u32x4 wbuf[3][8], abuf[3][MT];
            auto issue = [&](auto U, uint32_t idx) {
                constexpr int u = decltype(U)::value;
                const uint32_t kb = kb0 + idx * STRIDE;
    #pragma unroll
                for (int mt = 0; mt < MT; ++mt) abuf[u][mt] = ld128(prow[mt] + kb);
                skinny_load_q<QMODE>(p, qb, kb, colc, g, wbuf[u]);
            };
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            uint32_t issued = 0, done = 0;
            if (cnt > 0) { issue(I0{}, 0); issued = 1; }
            if (cnt > 1) { issue(I1{}, 1); issued = 2; }
            while (issued + 3 <= cnt) {
                issue(I2{}, issued);
                step(wbuf[0], abuf[0]);
                issue(I0{}, issued + 1);
                step(wbuf[1], abuf[1]);
                issue(I1{}, issued + 2);
                step(wbuf[2], abuf[2]);
                issued += 3;
                done += 3;
            }
            const uint32_t rem = cnt - issued;  // 0, 1 or 2 steps still to load
            if (done < cnt) {
                if (rem >= 1) issue(I2{}, issued);
                step(wbuf[0], abuf[0]);
            }
            if (done + 1 < cnt) {
                if (rem >= 2) issue(I0{}, issued + 1);
                step(wbuf[1], abuf[1]);
            }
            if (rem >= 1) step(wbuf[2], abuf[2]);
            if (rem >= 2) step(wbuf[0], abuf[0]);

            if (kfull < kend && kb0 + cnt * STRIDE == kfull) {  // the ragged last step belongs to exactly one wave
                const uint32_t kb = kfull;
    #pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    abuf[0][mt] = u32x4{0, 0, 0, 0};
                    if (kb + 8 * g + 8 <= kend) {
                        abuf[0][mt] = ld128(prow[mt] + kb);
                    } else if (kb + 8 * g < kend) {  // K cuts this group of 8 (K % 8 != 0): element by element
                        const uint16_t *h = reinterpret_cast<const uint16_t *>(prow[mt] + kb);
    #pragma unroll
                        for (int e = 0; e < 7; ++e)
                            if (kb + 8 * g + e < kend) abuf[0][mt][e / 2] |= (uint32_t)h[e] << (16 * (e & 1));
                    }
                }
                skinny_load_q_tail<QMODE>(p, qb, kb, kend, colc, g, wbuf[0]);
                step(wbuf[0], abuf[0]);
            }
        }

    }

    // combine the 4 waves, then row = mt*16 + 4g + wave, columns col0 .. col0+7
    __shared__ uint32_t s_last;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        __syncthreads();
#pragma unroll
        for (int t = 0; t < 8; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) red[wave][t * 4 + q][lane] = acc[mt][t][q];
        __syncthreads();
        float sum[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w) s += red[w][t * 4 + wave][lane];
            sum[t] = s;
        }
        const uint32_t i = mt * 16 + 4 * g + wave;
        if (i < p.M && col0 < p.N) {
            if (p.split_k > 1) {
                const size_t first = (((size_t)split * p.batch + bat) * p.M + i) * p.N + col0;
                float *dst = reinterpret_cast<float *>(p.partial) + first;
                if (p.counters) {
                    const __amdgpu_buffer_rsrc_t r = partial_rsrc(p.partial);
                    partial_store4(r, (uint32_t)(first * 4), sum[0], sum[1], sum[2], sum[3]);
                    partial_store4(r, (uint32_t)(first * 4 + 16), sum[4], sum[5], sum[6], sum[7]);
                } else {
                    *reinterpret_cast<f32x4 *>(dst) = f32x4{sum[0], sum[1], sum[2], sum[3]};
                    *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{sum[4], sum[5], sum[6], sum[7]};
                }
            } else {
                skinny_store(p, bat, i, col0, sum);
            }
        }
    }
    if (p.split_k > 1 && p.counters) {
        // Split-K without a second kernel: every workgroup publishes its partial tile,
        // then bumps the tile's counter; the workgroup that arrives last sums all
        // partials in ascending split order (so the result does not depend on
        // arrival order) and resets the counter for the next launch.
        // The partials were written with device-scope (write-through) stores; once
        // every thread has seen its stores acknowledged the count may be published.
        // A workgroup-scope fence does not wait for them (within one CU memory operations stay in
        // order without that), and the count travels to another L2 channel than the partials: without
        // the explicit wait it can overtake them, and a workgroup that arrives last right then sums
        // whatever the buffer held before.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        OPHIP_WAIT_VMEM();
        __syncthreads();
        uint32_t *counter = reinterpret_cast<uint32_t *>(p.counters) + (size_t)bat * gridDim.x + blockIdx.x;
        if (threadIdx.x == 0) s_last = atomicAdd(counter, 1u) == p.split_k - 1 ? 1u : 0u;
        __syncthreads();
        if (s_last) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint32_t i = mt * 16 + 4 * g + wave;
                if (i < p.M && col0 < p.N) {
                    float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                    const size_t sstride = (size_t)p.batch * p.M * p.N;  // floats between splits
                    const size_t elem0 = ((size_t)bat * p.M + i) * p.N + col0;
                    const __amdgpu_buffer_rsrc_t r = partial_rsrc(p.partial);
                    constexpr int FLY = MT == 1 ? 8 : 4;  // splits whose loads are in flight together, summed in order
                    for (uint32_t s0 = 0; s0 < p.split_k; s0 += FLY) {
                        float v[FLY][8];
#pragma unroll
                        for (int u = 0; u < FLY; ++u) {
                            float lo[4] = {0.f, 0.f, 0.f, 0.f}, hi[4] = {0.f, 0.f, 0.f, 0.f};
                            if (s0 + u < p.split_k) {
                                const uint32_t off = (uint32_t)((elem0 + (s0 + u) * sstride) * 4);
                                partial_load4(r, off, lo);
                                partial_load4(r, off + 16, hi);
                            }
#pragma unroll
                            for (int t = 0; t < 4; ++t) v[u][t] = lo[t], v[u][4 + t] = hi[t];
                        }
#pragma unroll
                        for (int u = 0; u < FLY; ++u)
                            if (s0 + u < p.split_k) {
#pragma unroll
                                for (int t = 0; t < 8; ++t) sum[t] += v[u][t];
                            }
                    }
                    skinny_store(p, bat, i, col0, sum);
                }
            }
            if (threadIdx.x == 0) *counter = 0;
        }
    }
}

// ------------------------------------------------------- stream (MFMA, M <= 16) --
//
// The same wave tile as gemm_skinny with MT = 1 and QMODE 0, built for residency instead of depth: two register
// buffers per wave (126 registers: four workgroups per CU), every address a scalar base plus one 32-bit lane offset
// (buffer loads: the resource carries the base of the wave's K-step, the scalar offset the row inside it), and no
// tail: a step past the wave's last one loads through a resource of zero records, for which the hardware returns
// zeros without touching memory, and multiplies zeros.
//
// Work units.  A unit is (128-column strip, K range); one workgroup takes one unit.  HBM does not serve every
// 256-byte granule of the address space at the same rate when a workgroup walks down one granule column (a strip
// of an N-contiguous weight whose rows are whole granules apart stays in one or two granule classes, address
// bits 8..10): strips in classes 1 and 5 stream about a quarter slower than the others, and a launch ends with
// its slowest strip.  `slow_mask` marks the classes whose strips are cut into `split_slow` K ranges instead of
// `split_k`; the host chooses both so that all units end together (mask 0: every strip is cut alike).
// Units are numbered by gemm_stream_unit (params.h), which the host uses for the grid as well.
template <int NW>
__device__ __forceinline__ void gemm_stream(const GemmParams &p) {
    __shared__ float red[NW][32][WAVE];
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), lane = threadIdx.x % WAVE;
    const uint32_t j16 = lane % 16, g = lane / 16;
    const uint32_t bat = blockIdx.z;
    const uint32_t nstrips = (p.N + 127) / 128;
    const elem *qbat = reinterpret_cast<const elem *>(p.q) + (int64_t)bat * p.q_sb;

    // unit -> (strip, K range, ranges of this strip): params.h, shared with the host
    const GemmStreamUnit unit = gemm_stream_unit(&p, reinterpret_cast<uint64_t>(qbat), blockIdx.x);
    if (!unit.valid) return;
    const uint32_t strip = unit.strip, split = unit.range, nsplit = unit.ranges;
    const uint32_t n0 = strip * 128;
    const uint32_t kbeg = unit.kbeg, kend = unit.kend;
    const uint32_t col0 = n0 + 8 * j16;
    const uint32_t colc = min(col0, p.N - 8);  // lanes past N load valid memory; their results are dropped at the store

    const uint32_t nsteps = kend > kbeg ? (kend - kbeg) / 32 : 0;  // (a K range past the end is empty)
    const uint32_t cnt = nsteps > wave ? (nsteps - wave + NW - 1) / NW : 0;  // steps wave, wave + NW, ... of the range

    const char *qs = reinterpret_cast<const char *>(qbat) + (int64_t)(kbeg + 32 * wave) * p.q_sl * 2;
    const char *ps = reinterpret_cast<const char *>(p.p) + ((int64_t)bat * p.p_sb + (int64_t)(kbeg + 32 * wave)) * 2;
    const uint32_t qoff = (uint32_t)((8 * g) * p.q_sl + colc) * 2;
    const uint32_t poff = (uint32_t)(min(j16, p.M - 1) * p.p_si + 8 * g) * 2;
    const uint32_t rowb = (uint32_t)p.q_sl * 2;     // bytes between K rows
    const int64_t stepb = (int64_t)32 * NW * rowb;  // bytes between this wave's steps
    // What is left of either operand from the wave's first step on: the records of the buffer resources, so that a
    // load can never reach past the operand (it would read zeros), whatever the arguments.
    const int64_t qleft = ((int64_t)(p.K - 1) * p.q_sl + p.N) * 2 - (int64_t)(kbeg + 32 * wave) * p.q_sl * 2;
    const int64_t pleft = ((int64_t)(p.M - 1) * p.p_si + p.K) * 2 - (int64_t)(kbeg + 32 * wave) * 2;

    f32x4 acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    u32x4 wbuf[2][8], abuf[2];
    auto issue = [&](auto U, uint32_t idx) {
        constexpr int u = decltype(U)::value;
        const int64_t qrem = qleft - (int64_t)idx * stepb, prem = pleft - (int64_t)idx * (64 * NW);
        const uint32_t qrec = idx < cnt && qrem > 0 ? (uint32_t)min(qrem, (int64_t)0xffffffff) : 0u;
        const uint32_t prec = idx < cnt && prem > 0 ? (uint32_t)min(prem, (int64_t)0xffffffff) : 0u;
        const __amdgpu_buffer_rsrc_t qr =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(qs + (int64_t)idx * stepb), 0, qrec, 0x00020000);
        const __amdgpu_buffer_rsrc_t pr =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(ps + (int64_t)idx * (64 * NW)), 0, prec, 0x00020000);
        abuf[u] = __builtin_amdgcn_raw_buffer_load_b128(pr, poff, 0, 0);
#pragma unroll
        for (int r = 0; r < 8; ++r) wbuf[u][r] = __builtin_amdgcn_raw_buffer_load_b128(qr, qoff, r * rowb, 2 /* nt */);
        __builtin_amdgcn_sched_barrier(0);  // the loads stay where they are written: ahead of the other buffer's products
    };
    auto compute = [&](auto U) {
        constexpr int u = decltype(U)::value;
        u32x4 b[8];
        transpose8x8_perm(wbuf[u], b);
        PackE at;
        at.u = abuf[u];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            PackE bt;
            bt.u = b[t];
            acc[t] = mfma_16x16x32(at.h, bt.h, acc[t]);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    issue(I0{}, 0);
    for (uint32_t i = 0; i < cnt; i += 2) {
        issue(I1{}, i + 1);
        compute(I0{});
        issue(I0{}, i + 2);
        compute(I1{});
    }

    // combine the waves: row 4g + wave, columns col0 .. col0 + 7, summed by the first four waves
    __shared__ uint32_t s_last;
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int q = 0; q < 4; ++q) red[wave][t * 4 + q][lane] = acc[t][q];
    __syncthreads();
    float sum[8];
    const uint32_t i = 4 * g + wave;
    const bool owner = wave < 4 && i < p.M && col0 < p.N;
    if (wave < 4) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += red[w][t * 4 + wave][lane];
            sum[t] = s;
        }
    }
    if (nsplit == 1) {
        if (owner) skinny_store(p, bat, i, col0, sum);
        return;
    }
    // The K ranges of a strip meet as in gemm_skinny: partials through write-through stores, one arrival counter per
    // strip, the last workgroup to arrive sums in ascending range order.
    const size_t first = (((size_t)split * p.batch + bat) * p.M + i) * p.N + col0;
    if (!p.counters) {  // no counters (more strips than the host keeps counters for): gemm_splitk_reduce sums
        if (owner) {
            float *dst = reinterpret_cast<float *>(p.partial) + first;
            *reinterpret_cast<f32x4 *>(dst) = f32x4{sum[0], sum[1], sum[2], sum[3]};
            *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{sum[4], sum[5], sum[6], sum[7]};
        }
        return;
    }
    const __amdgpu_buffer_rsrc_t r = partial_rsrc(p.partial);
    if (owner) {
        partial_store4(r, (uint32_t)(first * 4), sum[0], sum[1], sum[2], sum[3]);
        partial_store4(r, (uint32_t)(first * 4 + 16), sum[4], sum[5], sum[6], sum[7]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    OPHIP_WAIT_VMEM();
    __syncthreads();
    uint32_t *counter = reinterpret_cast<uint32_t *>(p.counters) + (size_t)bat * nstrips + strip;
    if (threadIdx.x == 0) s_last = atomicAdd(counter, 1u) == nsplit - 1 ? 1u : 0u;
    __syncthreads();
    if (s_last) {
        if (owner) {
            float tot[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            const size_t sstride = (size_t)p.batch * p.M * p.N;  // floats between ranges
            const size_t elem0 = ((size_t)bat * p.M + i) * p.N + col0;
            constexpr int FLY = 8;  // ranges whose loads are in flight together, summed in order
            for (uint32_t s0 = 0; s0 < nsplit; s0 += FLY) {
                float v[FLY][8];
#pragma unroll
                for (int u = 0; u < FLY; ++u) {
                    float lo[4] = {0.f, 0.f, 0.f, 0.f}, hi[4] = {0.f, 0.f, 0.f, 0.f};
                    if (s0 + u < nsplit) {
                        const uint32_t off = (uint32_t)((elem0 + (s0 + u) * sstride) * 4);
                        partial_load4(r, off, lo);
                        partial_load4(r, off + 16, hi);
                    }
#pragma unroll
                    for (int t = 0; t < 4; ++t) v[u][t] = lo[t], v[u][4 + t] = hi[t];
                }
#pragma unroll
                for (int u = 0; u < FLY; ++u)
                    if (s0 + u < nsplit) {
#pragma unroll
                        for (int t = 0; t < 8; ++t) tot[t] += v[u][t];
                    }
            }
            skinny_store(p, bat, i, col0, tot);
        }
        if (threadIdx.x == 0) *counter = 0;
    }
}

extern "C" __global__ void __launch_bounds__(256, 4) GEMM_KERNEL(gemm_stream_m1)(GemmParams p) { gemm_stream<4>(p); }

#define GEMM_SKINNY(MT, QMODE)                                                                   \
    extern "C" __global__ void __launch_bounds__(256) GEMM_KERNEL(gemm_skinny_m##MT##_q##QMODE)(GemmParams p) { \
        gemm_skinny<MT, QMODE, false>(p);                                                        \
    }
// `q0p`: K-steps dealt to the waves in pairs.  For a split whose steps come in whole groups of 8 (two per
// wave) and are many: with an odd number of pairs per wave the longest wave decides, and on short K ranges
// (split 8 of K = 4096) the plain dealing is 3 % faster.
#define GEMM_SKINNY_PAIRED(MT)                                                                   \
    extern "C" __global__ void __launch_bounds__(256) GEMM_KERNEL(gemm_skinny_m##MT##_q0p)(GemmParams p) {    \
        gemm_skinny<MT, 0, true>(p);                                                             \
    }
GEMM_SKINNY_PAIRED(1)
GEMM_SKINNY_PAIRED(2)
GEMM_SKINNY_PAIRED(4)
GEMM_SKINNY(1, 0)
GEMM_SKINNY(2, 0)
GEMM_SKINNY(4, 0)
GEMM_SKINNY(1, 1)
GEMM_SKINNY(2, 1)
GEMM_SKINNY(4, 1)
GEMM_SKINNY(1, 2)
GEMM_SKINNY(2, 2)
GEMM_SKINNY(4, 2)

// One thread per (batch, row, 8 columns): partial sums in ascending split order.
extern "C" __global__ void __launch_bounds__(256) GEMM_KERNEL(gemm_splitk_reduce)(GemmParams p) {
    const uint32_t nvec = p.N / 8;
    const size_t total = (size_t)p.batch * p.M * nvec;
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const uint32_t v = gid % nvec;
    const uint32_t i = (gid / nvec) % p.M;
    const uint32_t bat = gid / ((size_t)nvec * p.M);
    const uint32_t col0 = v * 8;
    float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t s = 0; s < p.split_k; ++s) {
        const float *src = reinterpret_cast<const float *>(p.partial) +
                           (((size_t)s * p.batch + bat) * p.M + i) * p.N + col0;
        const f32x4 lo = *reinterpret_cast<const f32x4 *>(src);
        const f32x4 hi = *reinterpret_cast<const f32x4 *>(src + 4);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            sum[t] += lo[t];
            sum[4 + t] += hi[t];
        }
    }
    skinny_store(p, bat, i, col0, sum);
}

// ------------------------------------------------------------ generic (FMA) --
// 64 x 64 tile per 256-thread block, 4 x 4 outputs per thread, K-step 16.
// Element-wise loads with arbitrary strides; used when the fast kernels'
// alignment or contiguity requirements are not met.
template <typename T>
__device__ __forceinline__ void gemm_generic(const GemmParams &p) {
    constexpr int BM = 64, BN = 64, BK = 16;
    using Acc = std::conditional_t<sizeof(T) == 8, double, float>;  // f64 data multiplies and adds in f64
    __shared__ Acc Ps[BK][BM + 4];
    __shared__ Acc Qs[BK][BN + 4];
    const uint32_t bat = blockIdx.z;
    const uint32_t i0 = blockIdx.y * BM, j0 = blockIdx.x * BN;
    const T *pb = reinterpret_cast<const T *>(p.p) + (int64_t)bat * p.p_sb;
    const T *qb = reinterpret_cast<const T *>(p.q) + (int64_t)bat * p.q_sb;
    T *db = reinterpret_cast<T *>(p.d) + (int64_t)bat * p.d_sb;
    const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    Acc acc[4][4] = {};
    for (uint32_t k0 = 0; k0 < p.K; k0 += BK) {
        for (uint32_t e = threadIdx.x; e < BM * BK; e += 256) {
            uint32_t li, ll;
            if (p.p_sl == 1) { ll = e % BK; li = e / BK; } else { li = e % BM; ll = e / BM; }
            const uint32_t i = i0 + li, l = k0 + ll;
            Ps[ll][li] = (i < p.M && l < p.K) ? (Acc)pb[(int64_t)i * p.p_si + (int64_t)l * p.p_sl] : (Acc)0;
        }
        for (uint32_t e = threadIdx.x; e < BN * BK; e += 256) {
            uint32_t lj, ll;
            if (p.q_sl == 1) { ll = e % BK; lj = e / BK; } else { lj = e % BN; ll = e / BN; }
            const uint32_t j = j0 + lj, l = k0 + ll;
            Qs[ll][lj] = (j < p.N && l < p.K) ? (Acc)qb[(int64_t)l * p.q_sl + (int64_t)j * p.q_sj] : (Acc)0;
        }
        __syncthreads();
#pragma unroll
        for (int l = 0; l < BK; ++l) {
            Acc a[4], b[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) a[r] = Ps[l][ty * 4 + r];
#pragma unroll
            for (int c = 0; c < 4; ++c) b[c] = Qs[l][tx * 4 + c];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[r][c] += a[r] * b[c];
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t i = i0 + ty * 4 + r, j = j0 + tx * 4 + c;
            if (i < p.M && j < p.N) {
                T *e = db + (int64_t)i * p.d_si + (int64_t)j * p.d_sj;
                Acc v = (Acc)p.alpha * acc[r][c];
                if (p.read_dst) v = (Acc)p.beta * (Acc)*e + v;
                *e = (T)v;
            }
        }
}

#ifdef GEMM_ELEM_BF16
extern "C" __global__ void __launch_bounds__(256) gemm_generic_bf16(GemmParams p) { gemm_generic<bf16>(p); }
#else
// (the kernels that do not depend on the build's element type are part of the f16 build only)
// Clears a fresh buffer of arrival counters.  A kernel rather than a memset: it can be recorded into a launch graph
// like any other launch when an operator's first split-K product on a stream happens during recording.
extern "C" __global__ void __launch_bounds__(256) gemm_fill_u32(FillU32Params p) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < p.count) reinterpret_cast<uint32_t *>(p.dst)[i] = p.value;
}

extern "C" __global__ void __launch_bounds__(256) gemm_generic_f64(GemmParams p) { gemm_generic<double>(p); }
extern "C" __global__ void __launch_bounds__(256) gemm_generic_f16(GemmParams p) { gemm_generic<f16>(p); }
extern "C" __global__ void __launch_bounds__(256) gemm_generic_f32(GemmParams p) { gemm_generic<float>(p); }
#endif
