// Compute-bound mat_mul for gfx950: LDS-tiled MFMA kernel (f16 in, f32 accumulate; compiled a second time on bf16
// elements, see gemm_elem.h: `elem` below is the element type of the build).
//
//     D[i, j] = alpha * sum_l P[i, l] * Q[l, j] + (read_dst ? beta * D[i, j] : 0)
//
// A 256-thread workgroup (4 waves, 2 x 2) owns a BM x BN tile of D and walks K in
// steps of TK (64 for 256 x 256 tiles, 32 for 128 x 128).  Both operands are staged in LDS as
// K-contiguous rows (one row per i for P, one per j for Q; swizzled or padded, see TileRow,
// so that 16-byte reads of consecutive rows spread over the banks), which is the layout MFMA wants: every
// lane reads its 8 consecutive k with one ds_read_b128.  An operand that is
// K-contiguous in memory is copied 16 bytes at a time; one that is contiguous
// along i / j (e.g. a weight stored [K, N]) is loaded as 16-byte rows of 8
// columns and transposed inside the lane's registers before the LDS store.
// Tile s+1 waits in registers while tile s is multiplied and goes to the other LDS
// buffer under its MFMAs, the loads of tile s+2 refill the registers: one barrier per tile.
// Workgroup ids are remapped so that the 8 XCDs (ids are dealt round-robin to
// them) each work on a compact block of tiles and share operand panels in
// their own L2.
//
// Requirements checked by the host: 16-byte aligned bases and strides; for the plain kernels M and N
// in whole tiles and K % TK == 0 (TK = 64 for the 256 tiles, 64 or 32 for the 128 tiles); the `r`
// kernels take any M, N and K >= TK (M or N along which an operand is contiguous must be a multiple
// of 8).  Everything else runs on the generic kernel.
#include <type_traits>

#include "gemm_elem.h"


// Copies one R x TK operand tile from global memory to registers (`fetch`) and
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
//
// Within an LDS row.  Measured with SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE: a ds_read_b128
// is served 16 lanes per cycle over 64 banks of 4 bytes (4 cycles when conflict-free), a
// ds_write_b128 8 lanes per cycle over 128 bytes (8 cycles).  So 16 consecutive rows read at
// the same k must land on 16 different 16-byte groups modulo 256 bytes, and the 8 consecutive
// rows a transposing store touches on 8 different groups modulo 128 bytes.
// TK = 32: rows are padded to 40 halves (80 bytes).  TK = 64: rows are exactly 128 bytes and
// the eight 16-byte groups of row s are stored at position group ^ key(s),
// key(s) = (s & 7) ^ ((s >> 3) & 1): distinct over any 8 consecutive rows, and rows s, s + 8
// (same parity, hence the same 128-byte half of the 256-byte bank line) differ in the low
// bit.  The fragment reads, the 16-byte stores of K-contiguous operands (8 lanes per row) and
// the transposing stores are all conflict-free, and the tile needs 128 KiB instead of 144.
template <int TK>
struct TileRow {
    static constexpr bool SWIZZLE = TK == 64;
    static constexpr int LDK = SWIZZLE ? TK : TK + 8;  // row pitch in halves
    // offset in halves of 16-byte group `g` of LDS row `s`
    __device__ static __forceinline__ uint32_t at(uint32_t s, uint32_t g) {
        return s * LDK + (SWIZZLE ? (g ^ (s & 7) ^ ((s >> 3) & 1)) : g) * 8;
    }
};

template <int R, bool KCONTIG, int TK>
struct TileLoader {
    static constexpr int LDK = TileRow<TK>::LDK;
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
    // K-contiguous: R * TK/8 vectors of 8 halves, NV per thread.
    // Row-contiguous: thread (cb, kb) takes NV k-rows x 8 columns.
    static constexpr int KV = TK / 8;
    static constexpr int NV = R * KV / 256;
    // Row-contiguous operand: which 8 columns (cb) and which NV k-rows (kb) thread t holds.  With NV = 4 a thread's
    // transposing stores are 8 bytes wide and the hardware takes 16 lanes of such a store per cycle over 128 bytes: 16
    // lanes on 16 consecutive LDS rows would meet only 8 different swizzle keys (rows s and s + 8 collide; measured as
    // 1.3 conflict cycles per LDS instruction of the 128 tile).  So a group of 16 lanes takes 8 column groups of two
    // neighbouring kb instead: 8 rows x the two 8-byte halves of one 16-byte group.
    __device__ static __forceinline__ uint32_t cb_of(uint32_t t) {
        if constexpr (NV == 4 && R == 128 && TK == 64) return (t & 7) | ((t >> 1) & 8);
        return t % (R / 8);
    }
    __device__ static __forceinline__ uint32_t kb_of(uint32_t t) {
        if constexpr (NV == 4 && R == 128 && TK == 64) return ((t >> 3) & 1) | ((t >> 5) << 1);
        return t / (R / 8);
    }
    u32x4 reg[NV];
    uint32_t voff[NV];  // byte offset of each of the thread's vectors from the tile's first element

    // s_row: stride between rows (i or j), s_k: stride along K, in elements; one of them is 1.
    // The host guarantees that offsets inside a tile fit 32 bits.
    // CLAMP: only `rows` of the tile's R rows exist (the last tile of a dimension that is not a
    // multiple of R).  The threads of the missing rows load an existing row instead (the last one,
    // or for a row-contiguous operand the last group of 8: there the host guarantees rows % 8 == 0);
    // what they store to LDS only reaches accumulators that the epilogue drops.
    template <bool CLAMP>
    __device__ __forceinline__ void init(int64_t s_row, int64_t s_k, uint32_t rows) {
        const uint32_t t = threadIdx.x;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if constexpr (KCONTIG) {
                const uint32_t idx = t + v * 256, kv = idx % KV;
                const uint32_t row = CLAMP ? min(idx / KV, rows - 1) : idx / KV;
                voff[v] = (row * (uint32_t)s_row + kv * 8) * 2;
            } else {
                const uint32_t kb = kb_of(t);
                const uint32_t cb = CLAMP ? min(cb_of(t), rows / 8 - 1) : cb_of(t);
                voff[v] = ((kb * NV + v) * (uint32_t)s_k + cb * 8) * 2;
            }
        }
    }

    // `tile` (wave-uniform) points at element (row0, k0) of the operand.  The copy is cut
    // into NV pieces so that the main loop can place them one by one between MFMAs.
    // The empty asm keeps the compiler from widening the offset to 64 bits outside the loop: as
    // "uniform base + 32-bit lane offset" the load needs no address arithmetic.
    __device__ __forceinline__ void fetch_piece(const elem *tile, int v) {
        asm volatile("" : "+v"(voff[v]));
        reg[v] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(tile) + voff[v]);
    }
    __device__ __forceinline__ void fetch(const elem *tile) {
#pragma unroll
        for (int v = 0; v < NV; ++v) fetch_piece(tile, v);
    }
    // The last, partial K-step of a K that is no multiple of TK: only `kvalid` (< TK) of the tile's k exist,
    // the rest is filled with zeros.  Runs once per workgroup, outside the pipelined loop.
    __device__ __forceinline__ void fetch_tail(const elem *tile, uint32_t kvalid) {
        const uint32_t t = threadIdx.x;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const char *src = reinterpret_cast<const char *>(tile) + voff[v];
            reg[v] = u32x4{0, 0, 0, 0};
            if constexpr (KCONTIG) {
                const uint32_t k0 = ((t + v * 256) % KV) * 8;  // first k of this vector
                if (k0 + 8 <= kvalid) {
                    reg[v] = *reinterpret_cast<const u32x4 *>(src);
                } else if (k0 < kvalid) {
                    const uint16_t *h = reinterpret_cast<const uint16_t *>(src);
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (k0 + e < kvalid) reg[v][e / 2] |= (uint32_t)h[e] << (16 * (e & 1));
                }
            } else {
                const uint32_t k = kb_of(t) * NV + v;  // this register's k-row
                if (k < kvalid) reg[v] = *reinterpret_cast<const u32x4 *>(src);
            }
        }
    }

    // Piece v of the register -> LDS copy.  K-contiguous: vector v.  Row-contiguous: reg[v]
    // holds k-row (kb*NV + v), columns cb*8 .. +8, and piece v writes columns
    // v*8/NV .. (v+1)*8/NV, each as the NV halves the thread holds of it (so every piece
    // reads all NV registers: refill them only after the last piece).
    __device__ __forceinline__ void commit_piece(elem *lds, int v) const {
        const uint32_t t = threadIdx.x;
        if constexpr (KCONTIG) {
            const uint32_t idx = t + v * 256, row = idx / KV, kv = idx % KV;
            st128(lds + TileRow<TK>::at(row, kv), reg[v]);
        } else {
            const uint32_t cb = cb_of(t), kb = kb_of(t);
#pragma unroll
            for (int c = v * 8 / NV; c < (v + 1) * 8 / NV; ++c) {
                elem *dst = lds + TileRow<TK>::at(c * (R / 8) + cb, kb * NV / 8) + kb * NV % 8;
                uint32_t w[NV / 2];
#pragma unroll
                for (int d = 0; d < NV / 2; ++d) w[d] = pair(reg[2 * d][c / 2], reg[2 * d + 1][c / 2], c & 1);
                if constexpr (NV == 8) *reinterpret_cast<u32x4 *>(dst) = u32x4{w[0], w[1], w[2], w[3]};
                else if constexpr (NV == 4) *reinterpret_cast<u32x2 *>(dst) = u32x2{w[0], w[1]};
                else *reinterpret_cast<uint32_t *>(dst) = w[0];
            }
        }
    }
    // halves `hi` of a0 and a1 in one register: a single byte permute
    __device__ static __forceinline__ uint32_t pair(uint32_t a0, uint32_t a1, bool hi) {
        return __builtin_amdgcn_perm(a1, a0, hi ? 0x07060302u : 0x05040100u);
    }
    // A row-contiguous piece in two halves, so that the main loop can put the permutes and
    // the store behind different MFMAs (NV == 8: piece v is column v, one 16-byte store).
    __device__ __forceinline__ u32x4 pack_piece(int v) const {
        static_assert(KCONTIG || NV == 8 || NV <= 4, "pack_piece is for the 8-register case");
        u32x4 w;
#pragma unroll
        for (int d = 0; d < 4; ++d) w[d] = pair(reg[(2 * d) % NV][v / 2], reg[(2 * d + 1) % NV][v / 2], v & 1);
        return w;
    }
    __device__ __forceinline__ void store_packed(elem *lds, int v, u32x4 w) const {
        const uint32_t t = threadIdx.x;
        const uint32_t cb = cb_of(t), kb = kb_of(t);
        st128(lds + TileRow<TK>::at(v * (R / 8) + cb, kb * NV / 8) + kb * NV % 8, w);
    }
    __device__ __forceinline__ void commit(elem *lds) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) commit_piece(lds, v);
    }
};

// DEPTH: operand tiles kept in flight in registers (1: the next one; 2: the next two, in two register sets).
// RAGGED: M and N need not be multiples of the tile (the last tiles load clamped rows and the
// epilogue stores only what exists) nor K of TK (a last, partial K-step is loaded with zeros for
// the missing k and multiplied after the pipelined loop); K >= TK.
template <int BM, int BN, bool PK, bool QK, int TK, int DEPTH, bool RAGGED>
__device__ __forceinline__ void gemm_tile(const GemmParams &p) {
    constexpr int LDK = TileRow<TK>::LDK;
    constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;
    // LDS: P buffer 0, P buffer 1, Q buffer 0, Q buffer 1.  Both buffers of an operand are within
    // 64 KiB of each other, so one address register per lane serves both through the
    // instruction's immediate offset.
    __shared__ elem lds[2 * (BM + BN) * LDK];
    constexpr uint32_t Q_REGION = 2 * BM * LDK;
    auto p_buf = [&](int b) { return lds + b * (BM * LDK); };
    auto q_buf = [&](int b) { return lds + Q_REGION + b * (BN * LDK); };

    // XCD-aware tile order: ids are dealt round-robin over 8 XCDs; give each XCD a
    // contiguous run of tiles, walked in groups of 8 tile-rows so panels are reused.
    // (XCD x receives the ids x, x + 8, ...: one more than tiles / 8 of them when x < tiles % 8.)
    const uint32_t tiles_m = RAGGED ? (p.M + BM - 1) / BM : p.M / BM, tiles_n = RAGGED ? (p.N + BN - 1) / BN : p.N / BN;
    const uint32_t tiles = tiles_m * tiles_n;
    uint32_t id = blockIdx.x;
    {
        const uint32_t q8 = tiles / 8, r8 = tiles % 8;
        const uint32_t xcd = id % 8, local = id / 8;
        id = xcd < r8 ? xcd * (q8 + 1) + local : r8 * (q8 + 1) + (xcd - r8) * q8 + local;
    }
    constexpr uint32_t GROUP = 8;
    const uint32_t group_size = GROUP * tiles_n;
    const uint32_t group = id / group_size;
    const uint32_t first_m = group * GROUP;
    const uint32_t rows_in_group = min(tiles_m - first_m, GROUP);
    const uint32_t tile_m = first_m + (id % group_size) % rows_in_group;
    const uint32_t tile_n = (id % group_size) / rows_in_group;
    const uint32_t bat = blockIdx.z;

    const elem *pb = reinterpret_cast<const elem *>(p.p) + (int64_t)bat * p.p_sb;
    const elem *qb = reinterpret_cast<const elem *>(p.q) + (int64_t)bat * p.q_sb;
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

    typedef TileLoader<BM, PK, TK> LP;
    typedef TileLoader<BN, QK, TK> LQ;
    LP lp[DEPTH];
    LQ lq[DEPTH];
    // split K: workgroup blockIdx.y multiplies K-range [kbeg, kbeg + klen) and leaves f32 partials
    const uint32_t split = blockIdx.y;
    // (the last split also takes what is left of a K that is no multiple of TK; only the ragged builds see one)
    const uint32_t kbeg = split * p.k_per_split, klen = split + 1 == p.split_k ? p.K - kbeg : p.k_per_split;
    const uint32_t ksteps = klen / TK;
    constexpr int KK = TK / 16;  // MFMA k-steps per LDS tile
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        lp[d].template init<RAGGED>(p.p_si, p.p_sl, min((uint32_t)BM, p.M - i0));
        lq[d].template init<RAGGED>(p.q_sj, p.q_sl, min((uint32_t)BN, p.N - j0));
    }
    const elem *ptile = pb + (int64_t)i0 * p.p_si + (int64_t)kbeg * p.p_sl;
    const elem *qtile = qb + (int64_t)j0 * p.q_sj + (int64_t)kbeg * p.q_sl;
    const int64_t pstep = (int64_t)TK * p.p_sl, qstep = (int64_t)TK * p.q_sl;
    // One wave per SIMD: nothing hides a stall, so the loop is software-pipelined by hand.
    //   registers  : tile s+1 waits in `reg` while tile s is multiplied; MFMA fragments are
    //                double-buffered, the LDS reads of k-step kk+1 run under the MFMAs of kk
    //   stores     : tile s+1 goes from registers to the other LDS buffer, piece by piece
    //   loads      : the global loads of tile s+2 refill the registers behind the stores
    //   barrier    : before the last k-step (whose fragments are already in registers), so
    //                that step's MFMAs cover the first fragment reads of tile s+1
    // The code below is written in exactly that order, one memory operation after each MFMA,
    // and sched_barrier(0) after every such pair keeps the compiler from regrouping them.
    // Copy piece i in the order the main loop uses (the waits the compiler derives for the loop
    // merge the prologue's order with the loop's: they must agree or the loop waits too long).
    constexpr bool Q_FIRST = PK && !QK, ALTERNATE = PK && QK && LP::NV == LQ::NV;
    auto piece_is_q = [&](int i) { return ALTERNATE ? bool(i & 1) : (Q_FIRST ? i < LQ::NV : i >= LP::NV); };
    auto piece_v = [&](int i) { return ALTERNATE ? i / 2 : (Q_FIRST ? (i < LQ::NV ? i : i - LQ::NV) : (i < LP::NV ? i : i - LP::NV)); };
    auto fetch_all = [&](int set, const elem *pt, const elem *qt) {
#pragma unroll
        for (int i = 0; i < LP::NV + LQ::NV; ++i) {
            if (piece_is_q(i)) lq[set].fetch_piece(qt, piece_v(i));
            else lp[set].fetch_piece(pt, piece_v(i));
        }
    };
    // operand tile t travels through register set t % DEPTH
    fetch_all(0, ptile, qtile);
    lp[0].commit(p_buf(0));
    lq[0].commit(q_buf(0));
#pragma unroll
    for (int d = 1; d <= DEPTH; ++d) {
        const uint32_t kd = min((uint32_t)d, ksteps - 1);
        fetch_all(d % DEPTH, ptile + kd * pstep, qtile + kd * qstep);
    }
    __syncthreads();

    PackE a[2][TM], b[2][TN];
    // Fragment addresses.  Every slot a lane reads has the same low four bits (l32 & 15), so
    // the position of k-step kk's group inside the row is one value per kk for all fragments.
    uint32_t koff[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) koff[kk] = TileRow<TK>::at(l32 & 15, 2 * kk + lk) - (l32 & 15) * LDK;
    const uint32_t a_row = LP::reader_slot(wm, 0, l32) * LDK;
    const uint32_t b_row = Q_REGION + LQ::reader_slot(wn, 0, l32) * LDK;
    // fragment r of k-step kk of the tile at `tile`: r < TM is a P fragment, the rest are Q's
    // `from`: LDS buffer 0 or 1
    auto read_one = [&](int buf, int from, int kk, int r) {
        if (r < TM)
            a[buf][r].u = ld128(lds + (a_row + koff[kk]) + from * (BM * LDK) + (LP::reader_slot(wm, r, l32) - LP::reader_slot(wm, 0, l32)) * LDK);
        else
            b[buf][r - TM].u = ld128(lds + (b_row + koff[kk]) + from * (BN * LDK) + (LQ::reader_slot(wn, r - TM, l32) - LQ::reader_slot(wn, 0, l32)) * LDK);
    };
    auto mfma_one = [&](int buf, int m) {
        const int tm = m / TN, tn = m % TN;
        acc[tm][tn] = mfma_32x32x16(a[buf][tm].h, b[buf][tn].h, acc[tm][tn]);
    };
    constexpr int NMFMA = TM * TN, NREAD = TM + TN, NLOAD = LP::NV + LQ::NV;
    static_assert(NREAD <= NMFMA && NLOAD <= NMFMA * (KK / 2), "the copy pieces must fit the slots of half a tile");
    static_assert(KK >= 2 && KK % 2 == 0, "fragment buffers alternate per k-step");
    // Issue budget.  The wave issues in order and an MFMA occupies its pipe for 32 cycles, so
    // whatever stands between two MFMAs must issue in less than that or the pipe runs dry:
    // a ds_write_b128 alone takes about 20 cycles, a global load with its address arithmetic
    // about 16, a ds_read_b128 4.  Hence at most one memory operation per MFMA: fragment reads
    // after the even-numbered MFMAs of a tile, stores and loads after the odd-numbered ones.
    //   256 x 256 x 64 (4 k-steps of 16 MFMAs, 16 copy pieces): odd position o = 0..31 of a tile's
    //   loop holds the store of piece ST[i] = o or the load of piece LD[i] = o, pieces numbered
    //   in store order.  Stores end before the barrier (o < 24).  Both operands K-contiguous:
    //   two stores, then the load that refills the first of them, and so on, which leaves a
    //   load 19 to 30 positions (of 64 cycles) to arrive.  Otherwise: all stores, then all
    //   loads, the row-contiguous operand first, because each of its stores reads all of its
    //   registers.
    struct Sched { int st[16], ld[16]; };
    constexpr Sched SCH = (PK && QK) ? Sched{{0, 1, 3, 4, 6, 7, 9, 10, 12, 13, 15, 16, 18, 19, 21, 22},
                                             {2, 5, 8, 11, 14, 17, 20, 23, 24, 25, 26, 27, 28, 29, 30, 31}}
                                     : Sched{{0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15},
                                             {16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28, 29, 30, 31}};
    //   128 x 128 x 64 (4 k-steps of 4 MFMAs, 8 copy pieces, two such workgroups per CU so the other
    //   wave of the SIMD fills what one wave's issue leaves open): a fragment read after every
    //   MFMA, the stores after MFMAs 0..7, the loads after 8..15; with DEPTH = 2 a load has a
    //   tile and a half to arrive.
    //   128 x 128 x 32 (K not a multiple of 64): two k-steps, stores under the first, then the loads.
    constexpr bool BIG = NMFMA == 16 && KK == 4, MID = NMFMA == 4 && KK == 4;
    static_assert(KK == 2 || (BIG && LP::NV == 8 && LQ::NV == 8) || (MID && LP::NV == 4 && LQ::NV == 4), "no slot table for this tile");
    // fragments in the order the next k-step's MFMAs want them: a0 b0 b1 b2 b3 a1 a2 a3 (a0 b0 b1 a1)
    constexpr int RORDER[8] = {0, TM, TM + 1, BIG ? TM + 2 : 1, TM + 3, 1, 2, 3};
    // Every tile runs the same code: past the end of K the loads fetch the last tile again, the
    // stores put it into the buffer nobody reads any more and the fragment reads of a tile that
    // does not exist are not used.  (Separate code for the last two tiles costs more in
    // registers, through the extra control flow, than the few redundant copies.)
    auto step = [&](uint32_t ks, auto parity) {
        constexpr int cur = decltype(parity)::value, nxt = 1 - cur;  // = ks % 2
        constexpr int SET = DEPTH == 2 ? nxt : 0;  // register set of tile ks + 1, refilled with tile ks + 1 + DEPTH
        const uint32_t knext = min(ks + 1 + DEPTH, ksteps - 1);
        const elem *pnext = ptile + knext * pstep, *qnext = qtile + knext * qstep;
        u32x4 packed;
        // the permutes of a row-contiguous piece, one slot ahead of its store
        auto piece_pack = [&](int i) {
            const bool is_q = piece_is_q(i);
            const int v = piece_v(i);
            if (is_q) { if constexpr (!QK && LQ::NV == 8) packed = lq[SET].pack_piece(v); }
            else { if constexpr (!PK && LP::NV == 8) packed = lp[SET].pack_piece(v); }
        };
        auto piece_op = [&](int i, bool is_store) {
            const bool is_q = piece_is_q(i);
            const int v = piece_v(i);
            if (is_store) {
                if (is_q) {
                    if constexpr (!QK && LQ::NV == 8) lq[SET].store_packed(q_buf(nxt), v, packed);
                    else lq[SET].commit_piece(q_buf(nxt), v);
                } else {
                    if constexpr (!PK && LP::NV == 8) lp[SET].store_packed(p_buf(nxt), v, packed);
                    else lp[SET].commit_piece(p_buf(nxt), v);
                }
            } else {
                if (is_q) lq[SET].fetch_piece(qnext, v);
                else lp[SET].fetch_piece(pnext, v);
            }
        };
        // what follows MFMA number `slot` of the tile (KK == 4)
        auto after_mfma = [&](int slot, int next_buf, int from, int next_kk) {
            if constexpr (MID) {
                read_one(next_buf, from, next_kk, RORDER[slot % NMFMA]);
                if (slot < NLOAD) piece_op(slot, true);
                else piece_op(slot - NLOAD, false);
            } else if (slot % 2 == 0) {
                read_one(next_buf, from, next_kk, RORDER[(slot % NMFMA) / 2]);
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    if (SCH.st[i] == slot / 2) piece_pack(i);
            } else {
                const int o = slot / 2;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    if (SCH.st[i] == o) piece_op(i, true);
                    if (SCH.ld[i] == o) piece_op(i, false);
                }
            }
        };
#pragma unroll
        for (int kk = 0; kk < KK - 1; ++kk) {
#pragma unroll
            for (int m = 0; m < NMFMA; ++m) {
                mfma_one(kk & 1, m);
                if constexpr (KK > 2) {
                    after_mfma(kk * NMFMA + m, (kk + 1) & 1, cur, kk + 1);
                } else {
                    // two k-steps of 4 MFMAs per tile: reads and stores under the first, then all loads
                    if (m < NREAD) read_one((kk + 1) & 1, cur, kk + 1, m);
                    if (m < NLOAD) piece_op(m, true);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (KK == 2 && kk == 0) {
                fetch_all(SET, pnext, qnext);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // every store of this tile's loop is above this line
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < NMFMA; ++m) {
            mfma_one((KK - 1) & 1, m);
            if constexpr (KK > 2) after_mfma((KK - 1) * NMFMA + m, 0, nxt, 0);
            else if (m < NREAD) read_one(0, nxt, 0, m);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
#pragma unroll
    for (int r = 0; r < NREAD; ++r) read_one(0, 0, 0, KK > 2 ? RORDER[r % 8] : r);
    static_assert(!MID || NLOAD == 8, "MID: 8 stores, then 8 loads, in the 16 slots of a tile");
    // Two tiles per trip so that the LDS buffer of every access is a compile-time constant.
    constexpr std::integral_constant<int, 0> EVEN{};
    constexpr std::integral_constant<int, 1> ODD{};
    uint32_t ks = 0;
    for (; ks + 2 <= ksteps; ks += 2) {
        step(ks, EVEN);
        step(ks + 1, ODD);
    }
    if (ks < ksteps) step(ks, EVEN);
    if constexpr (RAGGED) {
        const uint32_t ktail = klen % TK;
        if (ktail != 0) {  // workgroup-uniform
            __syncthreads();  // every wave is done with the LDS buffers
            lp[0].fetch_tail(ptile + ksteps * pstep, ktail);
            lq[0].fetch_tail(qtile + ksteps * qstep, ktail);
            lp[0].commit(p_buf(0));
            lq[0].commit(q_buf(0));
            __syncthreads();
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
                for (int r = 0; r < NREAD; ++r) read_one(0, 0, kk, r);
#pragma unroll
                for (int m = 0; m < NMFMA; ++m) mfma_one(0, m);
            }
        }
    }

    // 32x32 accumulator tile: lane holds slot-column l32 and slot-rows 8*(e/4) + 4*lk + e%4.
    if (p.split_k > 1) {
        // f32 partials [split][batch][M][N]; gemm_splitk_reduce sums them and applies alpha, beta
        float *part = reinterpret_cast<float *>(p.partial) + ((size_t)split * p.batch + bat) * p.M * (size_t)p.N;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t i = i0 + LP::row_of_slot(LP::reader_slot(wm, tm, 8 * (e / 4) + 4 * lk + (e % 4)));
                if (RAGGED && i >= p.M) continue;
                float *row = part + (size_t)i * p.N + j0;
                if constexpr (LQ::PERMUTED) {
                    // the lane's TN tiles are TN adjacent columns (all inside N or all outside: N % 8 == 0)
                    const uint32_t jl = LQ::row_of_slot(LQ::reader_slot(wn, 0, l32));
                    if (RAGGED && j0 + jl >= p.N) continue;
                    float *dst = row + jl;
                    if constexpr (TN == 4) *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[tm][0][e], acc[tm][1][e], acc[tm][2][e], acc[tm][3][e]};
                    else {
#pragma unroll
                        for (int tn = 0; tn < TN; ++tn) dst[tn] = acc[tm][tn][e];
                    }
                } else {
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn) {
                        const uint32_t jl = LQ::row_of_slot(LQ::reader_slot(wn, tn, l32));
                        if (!RAGGED || j0 + jl < p.N) row[jl] = acc[tm][tn][e];
                    }
                }
            }
        return;
    }
    elem *db = reinterpret_cast<elem *>(p.d) + (int64_t)bat * p.d_sb;
    if (LQ::PERMUTED && p.d_sj == 1) {
        // the lane's TN tiles are TN adjacent columns of D: one 4*TN/2-byte store per row
        const uint32_t j = j0 + LQ::row_of_slot(LQ::reader_slot(wn, 0, l32));
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t i = i0 + LP::row_of_slot(LP::reader_slot(wm, tm, 8 * (e / 4) + 4 * lk + (e % 4)));
                if (RAGGED && (i >= p.M || j >= p.N)) continue;  // j .. j + TN - 1 are inside N together: N % 8 == 0
                elem *dst = db + (int64_t)i * p.d_si + j;
                union { elem h[TN]; uint32_t u[TN / 2]; } o, c;
                if (p.read_dst) {
#pragma unroll
                    for (int w = 0; w < TN / 2; ++w) c.u[w] = reinterpret_cast<const uint32_t *>(dst)[w];
                }
#pragma unroll
                for (int tn = 0; tn < TN; ++tn) {
                    float v = p.alpha * acc[tm][tn][e];
                    if (p.read_dst) v = p.beta * e2f(c.h[tn]) + v;
                    o.h[tn] = f2e(v);
                }
#pragma unroll
                for (int w = 0; w < TN / 2; ++w) reinterpret_cast<uint32_t *>(dst)[w] = o.u[w];
            }
    } else if (!LP::PERMUTED && p.d_si == 1) {
        // four consecutive accumulator rows are four adjacent rows of D: 8-byte stores (the group that
        // straddles a ragged M goes element by element)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const uint32_t j = j0 + LQ::row_of_slot(LQ::reader_slot(wn, tn, l32));
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t i = i0 + wm * WM + tm * 32 + 8 * q + 4 * lk;
                    if (RAGGED && (i >= p.M || j >= p.N)) continue;
                    elem *dst = db + i + (int64_t)j * p.d_sj;
                    if (RAGGED && i + 4 > p.M) {
#pragma unroll
                        for (int r = 0; r < 3; ++r) {
                            if (i + r >= p.M) break;
                            float v = p.alpha * acc[tm][tn][4 * q + r];
                            if (p.read_dst) v = p.beta * e2f(dst[r]) + v;
                            dst[r] = f2e(v);
                        }
                        continue;
                    }
                    union { elem h[4]; u32x2 u; } o, c;
                    if (p.read_dst) c.u = *reinterpret_cast<const u32x2 *>(dst);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float v = p.alpha * acc[tm][tn][4 * q + r];
                        if (p.read_dst) v = p.beta * e2f(c.h[r]) + v;
                        o.h[r] = f2e(v);
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
                    if (RAGGED && (i >= p.M || j >= p.N)) continue;
                    elem *dst = db + (int64_t)i * p.d_si + (int64_t)j * p.d_sj;
                    float v = p.alpha * acc[tm][tn][e];
                    if (p.read_dst) v = p.beta * e2f(*dst) + v;
                    *dst = f2e(v);
                }
            }
    }
}

// Every tile in two builds: for M and N in whole tiles (no clamps, no store guards), and `r` for the rest.
// (One build with the guards switched by a kernel argument runs the whole-tile shapes 3 - 4 % slower:
// the guards change the register allocation of the main loop.)
#define GEMM_TILE(NAME, BM, BN, PK, QK, TK, DEPTH)                                                    \
    extern "C" __global__ void __launch_bounds__(256) GEMM_KERNEL(gemm_tile_##NAME##_p##PK##_q##QK)(GemmParams p) {    \
        gemm_tile<BM, BN, PK, QK, TK, DEPTH, false>(p);                                               \
    }                                                                                                 \
    extern "C" __global__ void __launch_bounds__(256) GEMM_KERNEL(gemm_tile_##NAME##r_p##PK##_q##QK)(GemmParams p) {   \
        gemm_tile<BM, BN, PK, QK, TK, DEPTH, true>(p);                                                \
    }

GEMM_TILE(256x256, 256, 256, 1, 1, 64, 1)
GEMM_TILE(256x256, 256, 256, 1, 0, 64, 1)
GEMM_TILE(256x256, 256, 256, 0, 1, 64, 1)
GEMM_TILE(256x256, 256, 256, 0, 0, 64, 1)
GEMM_TILE(128x128, 128, 128, 1, 1, 64, 2)
GEMM_TILE(128x128, 128, 128, 1, 0, 64, 2)
GEMM_TILE(128x128, 128, 128, 0, 1, 64, 2)
GEMM_TILE(128x128, 128, 128, 0, 0, 64, 2)
GEMM_TILE(128x128k32, 128, 128, 1, 1, 32, 1)
GEMM_TILE(128x128k32, 128, 128, 1, 0, 32, 1)
GEMM_TILE(128x128k32, 128, 128, 0, 1, 32, 1)
GEMM_TILE(128x128k32, 128, 128, 0, 0, 32, 1)
