// Compute-bound mat_mul for gfx950: LDS-tiled MFMA kernel (f16 in, f32 accumulate).
//
//     D[i, j] = alpha * sum_l P[i, l] * Q[l, j] + (read_dst ? beta * D[i, j] : 0)
//
// A 256-thread workgroup (4 waves, 2 x 2) owns a BM x BN tile of D and walks K in
// steps of 32.  Both operands are staged in LDS as K-contiguous rows (one row per
// i for P, one per j for Q, padded to 40 halves so that 16-byte reads of 32
// consecutive rows hit distinct banks), which is the layout MFMA wants: every
// lane reads its 8 consecutive k with one ds_read_b128.  An operand that is
// K-contiguous in memory is copied 16 bytes at a time; one that is contiguous
// along i / j (e.g. a weight stored [K, N]) is loaded as 16-byte rows of 8
// columns and transposed inside the lane's registers before the LDS store.
// Global loads for step s+1 are issued before the MFMAs of step s and written to
// the other LDS buffer afterwards: one barrier per step.
// Workgroup ids are remapped so that the 8 XCDs (ids are dealt round-robin to
// them) each work on a compact block of tiles and share operand panels in
// their own L2.
//
// Requirements checked by the host: M % BM == 0, N % BN == 0, K % 32 == 0,
// 16-byte aligned bases and strides.  Everything else runs on the generic kernel.
#include "device_util.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TK = 32;       // K per step
constexpr int LDK = TK + 8;  // LDS row pitch in halves (80 bytes)

// Copies one R x 32 operand tile from global memory to registers (`fetch`) and
// from registers to LDS (`commit`).  KCONTIG: rows are K-contiguous in memory.
//
// LDS row order.  A K-contiguous operand keeps its rows in order.  A row-contiguous
// operand is written by threads that each own 8 adjacent rows (the 8 columns of
// their 16-byte loads); storing "row r at slot r" would make all lanes of a store
// hit rows 8 apart, i.e. the same few banks.  Its rows are therefore kept in the
// order  slot(r) = (r % 8) * (R / 8) + r / 8 : lanes of one store now touch
// consecutive slots.  MFMA does not care which rows a tile holds, so the readers
// simply take 32 consecutive slots and the epilogue maps slots back to rows with
// row(s) = (s % (R / 8)) * 8 + s / (R / 8).
template <int R, bool KCONTIG>
struct TileLoader {
    static constexpr bool PERMUTED = !KCONTIG;
    __device__ static __forceinline__ uint32_t row_of_slot(uint32_t s) {
        return PERMUTED ? (s % (R / 8)) * 8 + s / (R / 8) : s;
    }
    // Slot read by MFMA row/column r (0..31) of tile t in wave-half w.  For a permuted
    // operand the choice makes one lane's tiles t = 0, 1, .. adjacent rows of the matrix.
    __device__ static __forceinline__ uint32_t reader_slot(uint32_t w, uint32_t t, uint32_t r) {
        if constexpr (PERMUTED && R == 128) return (w * 4 + 2 * (r / 16) + t) * 16 + r % 16;
        return w * (R / 2) + t * 32 + r;
    }
    // K-contiguous: R * 4 vectors of 8 halves, R / 64 per thread.
    // Row-contiguous: thread (cb, kb) takes KR = R / 64 k-rows x 8 columns.
    static constexpr int NV = R / 64;
    u32x4 reg[NV];

    __device__ __forceinline__ void fetch(const f16 *base, int64_t s_row, int64_t s_k, uint32_t row0, uint32_t k0) {
        const uint32_t t = threadIdx.x;
        if constexpr (KCONTIG) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const uint32_t idx = t + v * 256, row = idx / 4, kv = idx % 4;
                reg[v] = ld128(base + (int64_t)(row0 + row) * s_row + (k0 + kv * 8));
            }
        } else {
            const uint32_t cb = t % (R / 8), kb = t / (R / 8);
#pragma unroll
            for (int v = 0; v < NV; ++v)
                reg[v] = ld128(base + (int64_t)(k0 + kb * NV + v) * s_k + (row0 + cb * 8));
        }
    }

    __device__ __forceinline__ void commit(f16 *lds) const {
        const uint32_t t = threadIdx.x;
        if constexpr (KCONTIG) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const uint32_t idx = t + v * 256, row = idx / 4, kv = idx % 4;
                st128(lds + row * LDK + kv * 8, reg[v]);
            }
        } else {
            const uint32_t cb = t % (R / 8), kb = t / (R / 8);
            // reg[v] holds k-row (kb*NV + v), columns cb*8 .. +8: write column c's NV halves together
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                f16 *dst = lds + (c * (R / 8) + cb) * LDK + kb * NV;
                if constexpr (NV == 4) {
                    uint32_t lo, hi;
                    const uint32_t a0 = reg[0][c / 2], a1 = reg[1][c / 2], a2 = reg[2][c / 2], a3 = reg[3][c / 2];
                    if (c & 1) {
                        lo = (a0 >> 16) | (a1 & 0xffff0000u);
                        hi = (a2 >> 16) | (a3 & 0xffff0000u);
                    } else {
                        lo = (a0 & 0xffffu) | (a1 << 16);
                        hi = (a2 & 0xffffu) | (a3 << 16);
                    }
                    *reinterpret_cast<u32x2 *>(dst) = u32x2{lo, hi};
                } else {
                    static_assert(NV == 2, "");
                    const uint32_t a0 = reg[0][c / 2], a1 = reg[1][c / 2];
                    *reinterpret_cast<uint32_t *>(dst) =
                        (c & 1) ? ((a0 >> 16) | (a1 & 0xffff0000u)) : ((a0 & 0xffffu) | (a1 << 16));
                }
            }
        }
    }
};

template <int BM, int BN, bool PK, bool QK>
__device__ __forceinline__ void gemm_tile(const GemmParams &p) {
    constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;
    __shared__ f16 lds[2][(BM + BN) * LDK];

    // XCD-aware tile order: ids are dealt round-robin over 8 XCDs; give each XCD a
    // contiguous run of tiles, walked in groups of 8 tile-rows so panels are reused.
    const uint32_t tiles_m = p.M / BM, tiles_n = p.N / BN, tiles = tiles_m * tiles_n;
    uint32_t id = blockIdx.x;
    {
        const uint32_t per_xcd = (tiles + 7) / 8;
        const uint32_t xcd = id % 8, local = id / 8;
        const uint32_t lin = xcd * per_xcd + local;
        id = (tiles % 8 == 0) ? lin : blockIdx.x;  // only remap when the tiles split evenly
    }
    constexpr uint32_t GROUP = 8;
    const uint32_t group_size = GROUP * tiles_n;
    const uint32_t group = id / group_size;
    const uint32_t first_m = group * GROUP;
    const uint32_t rows_in_group = min(tiles_m - first_m, GROUP);
    const uint32_t tile_m = first_m + (id % group_size) % rows_in_group;
    const uint32_t tile_n = (id % group_size) / rows_in_group;
    const uint32_t bat = blockIdx.z;

    const f16 *pb = reinterpret_cast<const f16 *>(p.p) + (int64_t)bat * p.p_sb;
    const f16 *qb = reinterpret_cast<const f16 *>(p.q) + (int64_t)bat * p.q_sb;
    const uint32_t i0 = tile_m * BM, j0 = tile_n * BN;

    const uint32_t wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const uint32_t wm = wave / 2, wn = wave % 2;
    const uint32_t l32 = lane % 32, lk = lane / 32;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

    typedef TileLoader<BM, PK> LP;
    typedef TileLoader<BN, QK> LQ;
    LP lp;
    LQ lq;
    const uint32_t ksteps = p.K / TK;
    lp.fetch(pb, p.p_si, p.p_sl, i0, 0);
    lq.fetch(qb, p.q_sj, p.q_sl, j0, 0);
    lp.commit(lds[0]);
    lq.commit(lds[0] + BM * LDK);
    __syncthreads();

    for (uint32_t ks = 0; ks < ksteps; ++ks) {
        const f16 *Ps = lds[ks & 1], *Qs = lds[ks & 1] + BM * LDK;
        if (ks + 1 < ksteps) {
            lp.fetch(pb, p.p_si, p.p_sl, i0, (ks + 1) * TK);
            lq.fetch(qb, p.q_sj, p.q_sl, j0, (ks + 1) * TK);
        }
#pragma unroll
        for (int kk = 0; kk < TK / 16; ++kk) {
            Pack8 a[TM], b[TN];
#pragma unroll
            for (int t = 0; t < TM; ++t) a[t].u = ld128(Ps + LP::reader_slot(wm, t, l32) * LDK + kk * 16 + lk * 8);
#pragma unroll
            for (int t = 0; t < TN; ++t) b[t].u = ld128(Qs + LQ::reader_slot(wn, t, l32) * LDK + kk * 16 + lk * 8);
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[tm].h, b[tn].h, acc[tm][tn], 0, 0, 0);
        }
        if (ks + 1 < ksteps) {
            lp.commit(lds[(ks + 1) & 1]);
            lq.commit(lds[(ks + 1) & 1] + BM * LDK);
        }
        __syncthreads();
    }

    // 32x32 accumulator tile: lane holds slot-column l32 and slot-rows 8*(e/4) + 4*lk + e%4.
    f16 *db = reinterpret_cast<f16 *>(p.d) + (int64_t)bat * p.d_sb;
    if (LQ::PERMUTED && p.d_sj == 1) {
        // the lane's TN tiles are TN adjacent columns of D: one 4*TN/2-byte store per row
        const uint32_t j = j0 + LQ::row_of_slot(LQ::reader_slot(wn, 0, l32));
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t i = i0 + LP::row_of_slot(LP::reader_slot(wm, tm, 8 * (e / 4) + 4 * lk + (e % 4)));
                f16 *dst = db + (int64_t)i * p.d_si + j;
                union { f16 h[TN]; uint32_t u[TN / 2]; } o, c;
                if (p.read_dst) {
#pragma unroll
                    for (int w = 0; w < TN / 2; ++w) c.u[w] = reinterpret_cast<const uint32_t *>(dst)[w];
                }
#pragma unroll
                for (int tn = 0; tn < TN; ++tn) {
                    float v = p.alpha * acc[tm][tn][e];
                    if (p.read_dst) v = p.beta * h2f(c.h[tn]) + v;
                    o.h[tn] = f2h(v);
                }
#pragma unroll
                for (int w = 0; w < TN / 2; ++w) reinterpret_cast<uint32_t *>(dst)[w] = o.u[w];
            }
    } else if (!LP::PERMUTED && p.d_si == 1) {
        // four consecutive accumulator rows are four adjacent rows of D: 8-byte stores
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const uint32_t j = j0 + LQ::row_of_slot(LQ::reader_slot(wn, tn, l32));
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t i = i0 + wm * WM + tm * 32 + 8 * q + 4 * lk;
                    f16 *dst = db + i + (int64_t)j * p.d_sj;
                    union { f16 h[4]; u32x2 u; } o, c;
                    if (p.read_dst) c.u = *reinterpret_cast<const u32x2 *>(dst);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float v = p.alpha * acc[tm][tn][4 * q + r];
                        if (p.read_dst) v = p.beta * h2f(c.h[r]) + v;
                        o.h[r] = f2h(v);
                    }
                    *reinterpret_cast<u32x2 *>(dst) = o.u;
                }
            }
    } else {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const uint32_t j = j0 + LQ::row_of_slot(LQ::reader_slot(wn, tn, l32));
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t i = i0 + LP::row_of_slot(LP::reader_slot(wm, tm, 8 * (e / 4) + 4 * lk + (e % 4)));
                    f16 *dst = db + (int64_t)i * p.d_si + (int64_t)j * p.d_sj;
                    float v = p.alpha * acc[tm][tn][e];
                    if (p.read_dst) v = p.beta * h2f(*dst) + v;
                    *dst = f2h(v);
                }
            }
    }
}

#define GEMM_TILE(BM, BN, PK, QK)                                                                        \
    extern "C" __global__ void __launch_bounds__(256) gemm_tile_##BM##x##BN##_p##PK##_q##QK(GemmParams p) { \
        gemm_tile<BM, BN, PK, QK>(p);                                                                    \
    }

GEMM_TILE(256, 256, 1, 1)
GEMM_TILE(256, 256, 1, 0)
GEMM_TILE(256, 256, 0, 1)
GEMM_TILE(256, 256, 0, 0)
GEMM_TILE(128, 128, 1, 1)
GEMM_TILE(128, 128, 1, 0)
GEMM_TILE(128, 128, 0, 1)
GEMM_TILE(128, 128, 0, 0)
