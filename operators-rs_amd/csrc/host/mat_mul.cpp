// mat_mul on the HIP backend.  Layout normalisation is Args::layout
// (mat_mul/args.rs:64-192); scalars follow the CPU backend
// (mat_mul/common_cpu/mod.rs:60-105): for f16 data alpha and beta are rounded
// to f16 first and C is read only when the f32 beta is non-zero.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "../kernels/params.h"
#include "handle.hpp"
#include "static_scratch.hpp"

using namespace ophip;

namespace {

struct Matrix {  // mat_mul/args.rs:124-192, strides in elements
    size_t batch;
    ptrdiff_t stride;
    size_t r, c;
    ptrdiff_t rs, cs;

    static Matrix from(const ophip_tensor_layout &t) {
        expect_arrays(t);
        for (size_t i = 0; i < t.ndim; ++i)
            if (is_dyn(t.shape[i]) || is_dyn(t.strides[i])) throw dyn_not_support("");
        if (t.ndim < 2) throw rank_not_support("Matrix must have rank 2 or more");
        if (t.ndim > 3) throw shape_not_support("Higher-rank tensors not supported");
        const ptrdiff_t unit = (ptrdiff_t)ophip_dtype_nbytes(t.dt);
        if (unit == 0) throw type_not_support("unknown data type");
        Matrix m;
        if (t.ndim == 2 || t.shape[0] == 1) {
            m.batch = 1;
            m.stride = 0;
        } else {
            m.batch = t.shape[0];
            m.stride = t.strides[0] / unit;
        }
        m.r = t.shape[t.ndim - 2];
        m.c = t.shape[t.ndim - 1];
        m.rs = t.strides[t.ndim - 2] / unit;
        m.cs = t.strides[t.ndim - 1] / unit;
        return m;
    }
    bool match_batch(size_t b) const { return batch == 1 || batch == b; }
    void transpose() {
        std::swap(r, c);
        std::swap(rs, cs);
    }
    void ld_trans(ptrdiff_t &ld, int32_t &trans) const {
        if (rs == 1) {
            ld = cs;
            trans = 0;
        } else if (cs == 1) {
            ld = rs;
            trans = 1;
        } else {
            throw strides_not_support("Matrix is not contiguous");
        }
    }
};

ophip_mat_mul_layout mat_mul_layout(const ophip_mat_mul_args &args) {
    Matrix c = Matrix::from(args.c_layout), a = Matrix::from(args.a_layout), b = Matrix::from(args.b_layout);
    if (c.r != a.r || c.c != b.c || a.c != b.r) throw shape_mismatch("Inconsistent matrix shapes");
    const size_t batch = c.batch;
    if (!a.match_batch(batch) || !b.match_batch(batch)) throw shape_mismatch("Inconsistent batch sizes");
    ophip_mat_mul_layout L{};
    if (c.rs == 1 && c.cs != 1) {
        L.ab_swap = 0;
    } else if (c.cs == 1) {  // C is row-major: C^T = B^T A^T
        c.transpose();
        a.transpose();
        b.transpose();
        std::swap(a, b);
        L.ab_swap = 1;
    } else {
        throw strides_not_support("Matrix is not contiguous");
    }
    a.ld_trans(L.a_ld, L.a_trans);
    b.ld_trans(L.b_ld, L.b_trans);
    L.dt = type_distinct({args.c_layout.dt, args.a_layout.dt, args.b_layout.dt});
    L.batch = batch;
    L.m = c.r;
    L.n = c.c;
    L.k = a.c;
    L.c_stride = c.stride;
    L.c_ld = c.cs;
    L.a_stride = a.stride;
    L.b_stride = b.stride;
    return L;
}

// The canonical problem handed to the kernels plus the kernel choice.
struct GemmPlan {
    GemmParams p{};
    enum Kind { Generic, Skinny, Tile } kind = Generic;
    // Skinny: 16-row blocks, weight layout mode (3: mode 0 with K-steps dealt in pairs; 4: gemm_stream, the build of
    // mode 0 for up to 16 rows and K in whole steps)
    int mt = 1, qmode = 0;
    int tile = 256, tk = 64, pk = 1, qk = 1;  // Tile: block size, K-step, and whether P / Q are K-contiguous
    bool ragged = false;                      // Tile: M or N not in whole tiles, or K not in whole K-steps
    size_t workspace = 0;
};

bool mult8(int64_t v) { return (v & 7) == 0; }

// Test and sweep knobs, read from the environment once, when an operator is created
// (OPHIP_GEMM_SPLITK, OPHIP_GEMM_TILE_SPLITK, OPHIP_GEMM_TILE); 0 = not set.
struct GemmKnobs {
    int skinny_split = 0, tile_split = 0, tile = 0;
    bool stream = true;   // OPHIP_GEMM_STREAM=0: keep gemm_skinny where gemm_stream would run
    int slow_split = -1;  // OPHIP_GEMM_SLOW_SPLIT: K ranges for strips on the slow granule classes (0: cut all strips alike)
    static GemmKnobs from_env() {
        GemmKnobs k;
        auto num = [](const char *name) {
            const char *e = std::getenv(name);
            const int v = e ? std::atoi(e) : 0;
            return v > 0 ? v : 0;
        };
        k.skinny_split = num("OPHIP_GEMM_SPLITK");
        k.tile_split = num("OPHIP_GEMM_TILE_SPLITK");
        k.tile = num("OPHIP_GEMM_TILE");
        if (const char *e = std::getenv("OPHIP_GEMM_STREAM")) k.stream = std::atoi(e) != 0;
        if (const char *e = std::getenv("OPHIP_GEMM_SLOW_SPLIT")) k.slow_split = std::max(0, std::atoi(e));
        return k;
    }
};

// f16, f32, f64: the CPU backend's types (mat_mul/common_cpu/mod.rs:99-103).  bf16: neither backend of the reference
// multiplies it (its CUDA backend checks for F16, mat_mul/cuda/mod.rs:73); taken here because the matrix cores do.
bool mat_mul_takes(uint64_t dt) { return dt == OPHIP_DT_F16 || dt == OPHIP_DT_BF16 || dt == OPHIP_DT_F32 || dt == OPHIP_DT_F64; }

// gemm_stream's uneven cut.  A workgroup that walks down one 128-column strip of an N-contiguous weight reads one
// 256-byte granule per row.  When the rows are a multiple of 1 KiB apart and start on a granule boundary, all
// granules of a strip have the same class (address bits 8..10) or alternate between c and c + 4, and HBM serves
// classes 1 and 5 about a quarter slower under this access pattern than the rest (4096 x 22016, cold weights, one
// workgroup per strip: the strips of those two classes take 32 us, the others 25; a plain sequential read of the same
// matrix shows no such difference, since there every request spans all classes).  The launch ends with its slowest
// strip, so those strips get more K ranges: as many as still leave at most one workgroup per CU.
// Returns the ranges for the slow strips and sets p.slow_mask / p.split_slow; 0 (and mask 0): all strips alike.
size_t plan_slow_strips(GemmParams &p, size_t ntiles, size_t cus, const GemmKnobs &knobs) {
    p.slow_mask = 0;
    p.split_slow = 0;
    if (knobs.slow_split == 0) return 0;
    const int64_t rowb = p.q_sl * 2, batb = p.q_sb * 2;
    const uintptr_t base = reinterpret_cast<uintptr_t>(p.q);
    if (base % 256 != 0 || rowb % 1024 != 0 || (p.batch > 1 && batb % 2048 != 0)) return 0;
    const uint32_t mask = 0x22;  // classes 1 and 5
    size_t slow = 0;
    for (size_t t = 0; t < ntiles; ++t) slow += (mask >> (((base >> 8) + t) & 7)) & 1;
    if (slow == 0) return 0;
    const size_t steps = p.K / 32, s0 = p.split_k;
    // Measured so far only for strips that are otherwise whole (4096 x 22016: 35.6 -> 31.3 us with the slow strips in two
    // ranges); with two ranges everywhere and four on the slow strips 4096 x 12288 stayed where it was (21.0 against
    // 21.2 us), so such products keep the even cut.
    if (s0 != 1 && knobs.slow_split < 0) return 0;
    auto whole = [&](size_t s) {  // a cut into s ranges of ceil(steps / s) steps leaves none of them empty
        const size_t sps = (steps + s - 1) / s;
        return (steps + sps - 1) / sps == s;
    };
    size_t best = s0;
    if (knobs.slow_split > 0) {
        best = std::min<size_t>((size_t)knobs.slow_split, steps);
        while (!whole(best)) --best;
    } else {
        // a slow strip costs 1.28 fast ones per byte: the smallest cut that brings its ranges under a fast strip's
        double best_cost = 1.28 / (double)s0;
        for (size_t s1 = s0 + 1; s1 <= 2 * s0 + 1 && s1 <= steps / 4; ++s1) {
            if (!whole(s1)) continue;
            if (((ntiles - slow) * s0 + slow * s1) * p.batch > cus) break;
            const double cost = std::max(1.0 / (double)s0, 1.28 / (double)s1);
            if (cost < best_cost - 1e-9) best = s1, best_cost = cost;
        }
    }
    if (best == s0) return 0;
    p.slow_mask = mask;
    p.split_slow = (uint32_t)best;
    return best;
}

GemmPlan make_plan(const ophip_mat_mul_args &args, const ophip_mat_mul_layout &L, unsigned cus, const GemmKnobs &knobs) {
    const void *a = L.ab_swap ? args.b_base : args.a_base;
    const void *b = L.ab_swap ? args.a_base : args.b_base;
    const int64_t a_si = L.a_trans ? L.a_ld : 1, a_sl = L.a_trans ? 1 : L.a_ld;
    const int64_t b_sl = L.b_trans ? L.b_ld : 1, b_sj = L.b_trans ? 1 : L.b_ld;

    GemmPlan g;
    GemmParams &p = g.p;
    p.batch = (uint32_t)L.batch;
    p.K = (uint32_t)L.k;
    p.d = args.c_base;
    p.d_sb = L.c_stride;
    // f16 and bf16 take the same MFMA kernels (two builds of one source); alpha and beta are rounded to the data's type
    // first, as the reference does for f16 (mat_mul/common_cpu/mod.rs:60-105)
    const bool f16 = L.dt == OPHIP_DT_F16 || L.dt == OPHIP_DT_BF16;
    auto rounded = [&](float v) { return L.dt == OPHIP_DT_F16 ? round_to_f16(v) : L.dt == OPHIP_DT_BF16 ? round_to_bf16(v) : v; };
    p.alpha = rounded(args.alpha);
    p.beta = rounded(args.beta);
    p.read_dst = args.beta != 0.f;
    p.split_k = 1;
    p.k_per_split = (uint32_t)((L.k + 31) / 32 * 32);

    auto orient = [&](bool transposed) {
        if (!transposed) {  // D = C, P = A, Q = B
            p.M = (uint32_t)L.m;
            p.N = (uint32_t)L.n;
            p.d_si = 1;
            p.d_sj = L.c_ld;
            p.p = a;
            p.p_si = a_si;
            p.p_sl = a_sl;
            p.p_sb = L.a_stride;
            p.q = b;
            p.q_sl = b_sl;
            p.q_sj = b_sj;
            p.q_sb = L.b_stride;
        } else {  // D = C^T, P = B^T, Q = A^T
            p.M = (uint32_t)L.n;
            p.N = (uint32_t)L.m;
            p.d_si = L.c_ld;
            p.d_sj = 1;
            p.p = b;
            p.p_si = b_sj;
            p.p_sl = b_sl;
            p.p_sb = L.b_stride;
            p.q = a;
            p.q_sl = a_sl;
            p.q_sj = a_si;
            p.q_sb = L.a_stride;
        }
    };
    auto skinny_ok = [&]() {
        if (!f16 || p.M == 0 || p.M > 64 || p.K == 0) return false;
        if (p.p_sl != 1 || !mult8(p.p_si) || !mult8(p.p_sb) || !aligned16(p.p)) return false;
        if (p.N % 8 != 0) return false;
        if (!aligned16(p.q) || !mult8(p.q_sb)) return false;
        if (p.q_sj == 1) {  // any K: the last K-step masks P element by element and Q by rows
            if (!mult8(p.q_sl)) return false;
        } else if (p.q_sl == 1) {
            if (p.K % 8 != 0 || !mult8(p.q_sj)) return false;
        } else {
            return false;
        }
        if (p.d_sj == 1 && (!aligned16(p.d) || !mult8(p.d_si) || !mult8(p.d_sb))) return false;
        return true;
    };

    // prefer the orientation whose row count is the small dimension
    const bool first_transposed = L.n <= L.m;
    auto plan_skinny = [&]() {
        for (int attempt = 0; attempt < 2; ++attempt) {
            orient(attempt == 0 ? first_transposed : !first_transposed);
            if (skinny_ok()) {
                g.kind = GemmPlan::Skinny;
                g.mt = p.M <= 16 ? 1 : p.M <= 32 ? 2 : 4;
                g.qmode = p.q_sj == 1 ? 0 : 1;
                // The kernel is latency-bound per CU, so a CU that holds two workgroups takes
                // twice as long as one that holds one: split K only as far as one workgroup
                // per CU (rounding down), keeping at least 16 K-steps per workgroup (the in-kernel
                // reduction of a split costs a few microseconds of tail).
                const size_t ntiles = (p.N + 127) / 128, slabs = (p.K + 31) / 32;
                const size_t base = ntiles * p.batch;
                size_t split = std::max<size_t>(1, (size_t)cus / base);
                split = std::min(split, std::max<size_t>(1, slabs / 16));
                // Slightly more workgroups than CUs is the worst case (the CUs that hold two finish last, at twice
                // the time): halving the workgroups evens the load out a little (measured on 16 x 4096 x 36864 and
                // 40960: 71 -> 65 and 72 -> 68 us; from 1.5 workgroups per CU on, a split only costs).
                if (base > (size_t)cus && base * 4 <= (size_t)cus * 5 && slabs >= 32) split = 2;
                if (knobs.skinny_split) split = (size_t)knobs.skinny_split;
                size_t sps = (slabs + split - 1) / split;  // K-steps per split
                split = (slabs + sps - 1) / sps;
                p.k_per_split = (uint32_t)(sps * 32);
                p.split_k = (uint32_t)split;
                // A long l-contiguous Q (a weight stored [N, K]): the mode that reads 256 contiguous bytes per
                // column, in K-chunks of 128 dealt to the four waves; needs whole chunks and at least one per wave.
                if (g.qmode == 1 && p.N % 128 == 0 && p.K % 128 == 0) {
                    // (cold-weight sweeps: at least 8 chunks per split, i.e. two per wave, or the split costs more than it hides)
                    const size_t chunks = p.K / 128;
                    if (!knobs.skinny_split) split = std::min(split, std::max<size_t>(1, chunks / 8));
                    const size_t cps = (chunks + split - 1) / split;  // chunks per split
                    if (cps >= 4) {
                        g.qmode = 2;
                        split = (chunks + cps - 1) / cps;
                        p.k_per_split = (uint32_t)(cps * 128);
                        p.split_k = (uint32_t)split;
                    }
                }
                // N-contiguous weight, long K range in whole groups of 8 steps: the build that deals the steps to the
                // waves in pairs and requests both halves of P's cache lines together (same box, cold weights,
                // 16 / 32 rows: 4096 x 22016 37.0 -> 35.9 / 42.2 -> 39.1 us, 4096 x 12288 split 2 23.4 -> 22.6 / 27.5 -> 26.3;
                // K = 4096 split 8 and 11008 split 8 lose 2 - 4 %, so they keep the plain dealing)
                // Up to 16 rows, N-contiguous weight, K in whole steps: gemm_stream (same wave tile, two register buffers
                // instead of three, no tail code; cold weights, 16 rows: 4096 x 22016 35.7 -> 35.5 us, 4096 x 12288 split 2
                // 21.9 -> 21.1, 4096 x 4096 split 8 11.5 -> 10.9, 11008 x 4096 split 8 20.1 -> 19.5).  Its lane offsets are 32 bits.
                size_t split_slow = 0;
                if (knobs.stream && g.mt == 1 && g.qmode == 0 && p.K % 32 == 0 && p.q_sl > 0 && p.q_sl < ((int64_t)1 << 24) && p.p_si >= 0 &&
                    p.p_si < ((int64_t)1 << 26)) {  // (unsigned lane offsets: rows of either operand ascend in memory)
                    g.qmode = 4;
                    split_slow = plan_slow_strips(p, ntiles, (size_t)cus, knobs);
                }
                if (g.qmode == 0 && p.k_per_split % 256 == 0 && p.k_per_split >= 1024 && p.K % p.k_per_split == 0) g.qmode = 3;
                const size_t ranges = std::max<size_t>(p.split_k, split_slow);
                g.workspace = ranges > 1 ? ranges * p.batch * (size_t)p.M * p.N * sizeof(float) : 0;
                return true;
            }
        }
        return false;
    };
    // Compute-bound shapes: the LDS-tiled MFMA kernel.  Of the two orientations take
    // the one whose epilogue can store several adjacent outputs per lane.
    // K-step of the tile kernels: 64, or 32 for a K in whole steps of 32 only; any other K from 64 on runs
    // the 64 step with a partial last one; 0: K too short.
    const size_t tile_tk = L.k % 64 == 0 ? 64 : L.k % 32 == 0 ? 32 : L.k >= 64 ? 64 : 0;
    // M and N need not be whole tiles: the last tiles load clamped rows and store what exists; 16-byte
    // loads along a contiguous i or j need that dimension in whole groups of 8.
    auto tile_ok = [&](uint32_t b) {
        if (!f16 || p.K == 0 || tile_tk == 0 || (b == 256 && tile_tk != 64)) return false;
        if ((p.p_sl != 1 && p.M % 8 != 0) || (p.q_sl != 1 && p.N % 8 != 0)) return false;
        if (!aligned16(p.p) || !aligned16(p.q) || !aligned16(p.d)) return false;
        if (!mult8(p.p_sb) || !mult8(p.q_sb) || !mult8(p.d_sb)) return false;
        if (!(p.p_sl == 1 ? mult8(p.p_si) : mult8(p.p_sl))) return false;
        if (!(p.q_sl == 1 ? mult8(p.q_sj) : mult8(p.q_sl))) return false;
        if (!(p.d_sj == 1 ? mult8(p.d_si) : mult8(p.d_sj))) return false;
        // the kernel addresses inside an operand tile with 32-bit byte offsets
        const int64_t lim = (int64_t)1 << 22;
        for (int64_t st : {p.p_si, p.p_sl, p.q_sj, p.q_sl})
            if (st <= 0 || st >= lim) return false;
        return true;
    };
    auto plan_tile = [&]() {
        for (uint32_t b : {256u, 128u}) {
            int best = -1;
            bool best_splits = false;
            // Tiles for less than half the CUs (a CU holds one 256 tile or two 128 tiles): split K,
            // keeping at least 8 K-steps per workgroup; the f32 partials are summed by
            // gemm_splitk_reduce, which wants the orientation whose D is j-contiguous.
            size_t split = 1;
            {
                const size_t wgs = ((L.m + b - 1) / b) * ((L.n + b - 1) / b) * L.batch, target = b == 256 ? cus : 2 * (size_t)cus;
                const size_t ksteps = tile_tk ? L.k / tile_tk : 1;
                if (wgs > 0 && wgs * 2 <= cus)
                    split = std::min<size_t>({target / wgs, (size_t)8, std::max<size_t>(1, ksteps / 8)});
                if (knobs.tile_split) split = (size_t)knobs.tile_split;
                split = std::max<size_t>(1, std::min(split, ksteps));
            }
            for (int attempt = 0; attempt < 2; ++attempt) {
                orient(attempt == 1);
                if (!tile_ok(b)) continue;
                // 256-tiles for less than 60 % of the CUs: the 128 pass is faster (measured on 512 .. 2048 row
                // shapes: at half the CUs the large tile loses by 10 - 50 %, at two thirds it wins by 10 %)
                // (OPHIP_GEMM_TILE=256 / 128 keeps one tile size, for tests and sweeps)
                const bool force = knobs.tile != 0;
                if (force && (uint32_t)knobs.tile != b) continue;
                // and when the part of the last tiles that lies outside the matrix costs more than the large tile's
                // advantage (about 1.4 x per multiply at these sizes)
                if (b == 256 && !force) {
                    const size_t t256 = (size_t)((p.M + 255) / 256) * ((p.N + 255) / 256) * p.batch;
                    const size_t t128 = (size_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
                    // A last round of a few tiles costs a whole round.  The 128 tiles (two to a CU) after full rounds:
                    const size_t tail128 = t128 % (2 * (size_t)cus), tail256 = t256 % (size_t)cus;
                    const bool bad128 = t128 > 2 * (size_t)cus && tail128 != 0 && tail128 * 4 <= (size_t)cus;
                    // and the 256 tiles: 640 x 22016 x 4096 is 258 of them, 198 us against 135 on 128 tiles (768 rows: 187 / 167;
                    // 1024 rows, 344 tiles: 189 / 202)
                    if (t256 > (size_t)cus && t256 < 3 * (size_t)cus && tail256 != 0 && tail256 * 4 < (size_t)cus) continue;
                    // too few 256 tiles for the CUs, unless the 128 tiles end on such a round (768 x 12288 x 4096: 144 tiles
                    // 81 us, 576 tiles of 128 97 us)
                    if (t256 * 5 < (size_t)cus * 3 && !bad128) continue;
                    // the part of the last tiles outside the matrix: at a third more area (384 rows) the 128 tiles win by a
                    // tenth (384 x 32000 x 4096: 128 / 117 us) unless they end on a short round (384 x 22016: 94 / 97)
                    if (t256 * 4 * 10 >= t128 * 13 && !bad128) continue;
                    if (t256 * 4 * 5 > t128 * 7) continue;
                }
                // (gemm_splitk_reduce works on groups of 8 columns: an orientation whose N is no multiple of 8 cannot split)
                const bool can_split = split > 1 && p.N % 8 == 0;
                const bool wide = split > 1 ? can_split && p.d_sj == 1
                                            : (p.q_sl != 1 && p.d_sj == 1) || (p.p_sl == 1 && p.d_si == 1);
                if (best < 0 || wide || (can_split && !best_splits)) {
                    best = attempt;
                    best_splits = can_split;
                }
                if (wide) break;
            }
            if (best >= 0) {
                orient(best == 1);
                if (!best_splits) split = 1;
                g.kind = GemmPlan::Tile;
                g.tile = (int)b;
                g.pk = p.p_sl == 1;
                g.qk = p.q_sl == 1;
                const size_t tk = tile_tk, ksteps = p.K / tk;
                g.tk = (int)tk;
                g.ragged = p.M % b != 0 || p.N % b != 0 || p.K % tk != 0;
                if (split > 1) {
                    const size_t sps = (ksteps + split - 1) / split;
                    split = (ksteps + sps - 1) / sps;
                    p.k_per_split = (uint32_t)(sps * tk);
                    p.split_k = (uint32_t)split;
                    g.workspace = split > 1 ? split * p.batch * (size_t)p.M * p.N * sizeof(float) : 0;
                }
                return true;
            }
        }
        return false;
    };
    // The streaming kernel slows down with its row count (every wave re-reads the rows of P for its K-steps
    // and multiplies 16 of them at a time); cold-weight sweeps over the decode GEMMs of a 7B layer put the
    // crossover to the 128 tile at 48 rows, at 32 for a weight of less than 64 MB (16 .. 64 rows against the
    // tile kernel at 65: 4096 x 22016 37 / 43 / 46 / 49 against 45 us; 4096 x 4096 13 / 18 / 22 / 26 against 18 us).
    const size_t rows = std::min(L.m, L.n), weight_bytes = (size_t)L.k * std::max(L.m, L.n) * 2;
    const bool tile_first = L.batch == 1 && rows > (weight_bytes < ((size_t)64 << 20) ? 32u : 48u);
    if (tile_first ? plan_tile() || plan_skinny() : plan_skinny() || plan_tile()) return g;
    orient(false);  // neither planner touches the split fields unless it succeeds
    g.kind = GemmPlan::Generic;
    return g;
}

}  // namespace

// u32 split-K arrival counters per (batch, column tile) of one launch
constexpr size_t SPLITK_COUNTERS = 1 << 16;

struct ophip_mat_mul {
    ophip_device *dev;
    GemmKnobs knobs = GemmKnobs::from_env();
    // the MFMA kernels exist twice, [0] on f16 and [1] on bf16 elements
    hipFunction_t skinny[2][3][4];  // [mt index 1,2,4][qmode; 3 = mode 0 with paired K-steps]
    hipFunction_t stream[2];        // gemm_stream_m1
    hipFunction_t reduce[2], fill, generic_f16, generic_bf16, generic_f32, generic_f64;
    // [256 x 64 / 128 x 64 / 128 x 32 (K-step)][M or N not in whole tiles][P K-contiguous][Q K-contiguous]
    hipFunction_t tile[2][3][2][2][2];
    // Arrival counters live in a buffer owned by the operator, one per stream:
    // launches on one stream run in order and every kernel leaves its counters at
    // zero, so a buffer is zeroed once.  The first stream gets the buffer made (and cleared) with the operator,
    // which costs no device work at launch time: that launch may be recorded into a graph.  A further stream
    // gets a new buffer, cleared by a kernel on that stream; allocating is not possible while a stream records,
    // so an operator's first split-K product on a second stream has to be an ordinary launch.
    // A stream that is destroyed (ophip_stream_destroy synchronises it first) gives its buffer back: all zero, ready
    // for the next stream.
    mutable std::mutex mu;
    mutable std::unordered_map<hipStream_t, void *> counters;
    mutable std::vector<void *> idle;
    mutable void *spare = nullptr;

    void *counters_for(hipStream_t stream) const {
        std::lock_guard<std::mutex> lock(mu);
        auto it = counters.find(stream);
        if (it != counters.end()) return it->second;
        if (spare || !idle.empty()) {
            void *buf = spare;
            if (spare) {
                spare = nullptr;
            } else {
                buf = idle.back();
                idle.pop_back();
            }
            counters[stream] = buf;
            return buf;
        }
        void *buf = nullptr;
        check_hip(hipMalloc(&buf, SPLITK_COUNTERS * sizeof(uint32_t)), "hipMalloc");
        FillU32Params f{buf, (uint32_t)SPLITK_COUNTERS, 0u};
        launch(fill, Dim3{(unsigned)(SPLITK_COUNTERS / 256)}, Dim3{256}, 0, stream, f);
        counters[stream] = buf;
        return buf;
    }
    explicit ophip_mat_mul(ophip_device *d) : dev(d) {
        ophip_device_retain(d);
        static const int mts[3] = {1, 2, 4};
        for (int e = 0; e < 2; ++e) {
            const char *gemm = e ? "gemm_bf16" : "gemm", *gemm_tile = e ? "gemm_tile_bf16" : "gemm_tile", *tag = e ? "_bf16" : "";
            for (int i = 0; i < 3; ++i)
                for (int q = 0; q < 4; ++q)
                    skinny[e][i][q] = d->kernel(
                        gemm, ("gemm_skinny_m" + std::to_string(mts[i]) + "_q" + (q == 3 ? "0p" : std::to_string(q)) + tag).c_str());
            for (int b = 0; b < 3; ++b)
                for (int r = 0; r < 2; ++r)
                    for (int pk = 0; pk < 2; ++pk)
                        for (int qk = 0; qk < 2; ++qk) {
                            const std::string sz = b == 0 ? "256x256" : b == 1 ? "128x128" : "128x128k32";
                            tile[e][b][r][pk][qk] = d->kernel(gemm_tile, ("gemm_tile_" + sz + (r ? "r" : "") + "_p" + std::to_string(pk) +
                                                                          "_q" + std::to_string(qk) + tag).c_str());
                        }
            stream[e] = d->kernel(gemm, (std::string("gemm_stream_m1") + tag).c_str());
            reduce[e] = d->kernel(gemm, (std::string("gemm_splitk_reduce") + tag).c_str());
        }
        fill = d->kernel("gemm", "gemm_fill_u32");
        d->make_current();
        check_hip(hipMalloc(&spare, SPLITK_COUNTERS * sizeof(uint32_t)), "hipMalloc");
        const hipError_t e = hipMemset(spare, 0, SPLITK_COUNTERS * sizeof(uint32_t));
        const hipError_t e2 = e == hipSuccess ? hipStreamSynchronize(nullptr) : e;
        if (e2 != hipSuccess) {
            (void)hipFree(spare);
            ophip_device_release(d);
            check_hip(e2, "hipMemset");
        }
        generic_f16 = d->kernel("gemm", "gemm_generic_f16");
        generic_bf16 = d->kernel("gemm_bf16", "gemm_generic_bf16");
        generic_f32 = d->kernel("gemm", "gemm_generic_f32");
        generic_f64 = d->kernel("gemm", "gemm_generic_f64");
        std::lock_guard<std::mutex> lock(d->hooks_mu);
        d->stream_gone[this] = [this](hipStream_t s) {
            std::lock_guard<std::mutex> l(mu);
            auto it = counters.find(s);
            if (it == counters.end()) return;
            idle.push_back(it->second);
            counters.erase(it);
        };
    }
    ~ophip_mat_mul() {
        {
            std::lock_guard<std::mutex> lock(dev->hooks_mu);
            dev->stream_gone.erase(this);
        }
        for (void *b : idle) (void)hipFree(b);
        for (auto &c : counters) (void)hipFree(c.second);
        if (spare) (void)hipFree(spare);
        ophip_device_release(dev);
    }
};

// One launch.  `fixed_counters` null: the ordinary entry point (workspace from the caller or the queue allocator,
// arrival counters owned by the operator).  Otherwise the caller of this function brings every byte of scratch:
// `workspace` holds the f32 partials, `fixed_counters` the arrival counters (all zero between launches: zero when the
// caller made them, and every kernel leaves the ones it used at zero), and nothing is allocated.
constexpr size_t GRID_Z_MAX = 65535;

static void mat_mul_launch_impl(const ophip_mat_mul *op, const ophip_mat_mul_args *args, void *workspace,
                                size_t workspace_len, const ophip_queue_alloc *qa, void *fixed_counters,
                                size_t fixed_counter_count, hipStream_t stream) {
    if (!op || !args) throw args_not_support("null argument");
    const ophip_mat_mul_layout L = mat_mul_layout(*args);
    if (!mat_mul_takes(L.dt)) throw type_not_support("mat_mul supports f16, bf16, f32 and f64");
    if (is_dyn(args->alpha) || is_dyn(args->beta)) throw dyn_not_support("");
    if (L.m == 0 || L.n == 0 || L.batch == 0) return;
    if (L.m > 0x7fffffffu || L.n > 0x7fffffffu || L.k > 0x7fffffffu) throw shape_not_support("mat_mul dimension too large");
    if (L.batch > GRID_Z_MAX) {
        // The batch rides on the grid's z extent, which ends at 65535 (cuBLAS, which the reference calls, takes any
        // count): the same product in as many launches as that needs, each on its share of the batches.
        for (size_t b0 = 0; b0 < L.batch; b0 += GRID_Z_MAX) {
            const size_t nb = std::min<size_t>(GRID_Z_MAX, L.batch - b0);
            ophip_mat_mul_args sub = *args;
            size_t shapes[3][3];
            auto cut = [&](ophip_tensor_layout &lay, size_t (&shape)[3]) -> ptrdiff_t {
                if (lay.ndim != 3 || lay.shape[0] == 1) return 0;  // one matrix shared by every batch
                std::copy(lay.shape, lay.shape + 3, shape);
                shape[0] = nb;
                lay.shape = shape;
                return (ptrdiff_t)b0 * lay.strides[0];
            };
            sub.c_base = static_cast<char *>(args->c_base) + cut(sub.c_layout, shapes[0]);
            sub.a_base = static_cast<const char *>(args->a_base) + cut(sub.a_layout, shapes[1]);
            sub.b_base = static_cast<const char *>(args->b_base) + cut(sub.b_layout, shapes[2]);
            mat_mul_launch_impl(op, &sub, workspace, workspace_len, qa, fixed_counters, fixed_counter_count, stream);
        }
        return;
    }
    GemmPlan g = make_plan(*args, L, (unsigned)op->dev->props.multiProcessorCount, op->knobs);
    const GemmParams &p = g.p;
    const bool fixed = fixed_counters != nullptr;
    const int e = L.dt == OPHIP_DT_BF16 ? 1 : 0;
    if (fixed && g.workspace > workspace_len)
        throw args_not_support("this product needs " + std::to_string(g.workspace) +
                               " bytes of split-K scratch, the library's static buffer holds " +
                               std::to_string(workspace_len));
    if (!args->c_base || !args->a_base || !args->b_base) throw args_not_support("null base address");
    op->dev->make_current();
    if (g.kind == GemmPlan::Skinny) {
        Workspace ws(fixed ? nullptr : qa, workspace, workspace_len, g.workspace);
        g.p.partial = ws.ptr();
        const size_t tiles = (size_t)((p.N + 127) / 128) * p.batch;
        if (fixed) {
            g.p.counters = ((p.split_k > 1 || p.slow_mask) && tiles <= fixed_counter_count && g.workspace < ((size_t)1 << 32)) ? fixed_counters : nullptr;
            // (the static array is zero when its module is loaded and every kernel hands its counters back at zero: the
            //  invariant the operator's own counter buffers rely on as well, so nothing is cleared here)
        } else {
            // (the in-kernel reduction addresses the partials with 32-bit offsets)
            g.p.counters = ((p.split_k > 1 || p.slow_mask) && tiles <= SPLITK_COUNTERS && g.workspace < ((size_t)1 << 32)) ? op->counters_for(stream) : nullptr;
        }
        const int mi = g.mt == 1 ? 0 : g.mt == 2 ? 1 : 2;
        if (g.qmode == 4) {
            const bool ranges = p.split_k > 1 || p.slow_mask;
            if (ranges && !g.p.counters) {  // too many strips for the counters: cut every strip alike and sum in a second launch
                g.p.slow_mask = 0;
                g.p.split_slow = 0;
            }
            launch(op->stream[e], Dim3{gemm_stream_units(&g.p, reinterpret_cast<uint64_t>(g.p.q)), 1, p.batch}, Dim3{256}, 0, stream, g.p);
        } else {
            launch(op->skinny[e][mi][g.qmode], Dim3{(p.N + 127) / 128, p.split_k, p.batch}, Dim3{256}, 0, stream, g.p);
        }
        if (p.split_k > 1 && !g.p.counters) {
            const size_t total = (size_t)p.batch * p.M * (p.N / 8);
            launch(op->reduce[e], Dim3{(unsigned)((total + 255) / 256)}, Dim3{256}, 0, stream, g.p);
        }
        return;
    }
    if (g.kind == GemmPlan::Tile) {
        Workspace ws(fixed ? nullptr : qa, workspace, workspace_len, g.workspace);
        g.p.partial = ws.ptr();
        const unsigned tiles = ((p.M + g.tile - 1) / g.tile) * ((p.N + g.tile - 1) / g.tile);
        launch(op->tile[e][g.tile == 256 ? 0 : g.tk == 64 ? 1 : 2][g.ragged][g.pk][g.qk], Dim3{tiles, p.split_k, p.batch}, Dim3{256}, 0,
               stream, g.p);
        if (p.split_k > 1) {
            const size_t total = (size_t)p.batch * p.M * (p.N / 8);
            launch(op->reduce[e], Dim3{(unsigned)((total + 255) / 256)}, Dim3{256}, 0, stream, g.p);
        }
        return;
    }
    const unsigned gx = (p.N + 63) / 64, gy = (p.M + 63) / 64;
    if (gy > 65535) throw shape_not_support("mat_mul dimension too large for the generic kernel");
    launch(L.dt == OPHIP_DT_F16 ? op->generic_f16 : L.dt == OPHIP_DT_BF16 ? op->generic_bf16 : L.dt == OPHIP_DT_F32 ? op->generic_f32 : op->generic_f64,
           Dim3{gx, gy, p.batch}, Dim3{256}, 0, stream, g.p);
}

namespace ophip {
void mat_mul_launch_fixed_scratch(const ophip_mat_mul *op, const ophip_mat_mul_args *args, void *partials,
                                  size_t partial_bytes, void *counters, size_t counter_count, hipStream_t stream) {
    mat_mul_launch_impl(op, args, partials, partial_bytes, nullptr, counters, counter_count, stream);
}
const ophip_device *mat_mul_device(const ophip_mat_mul *op) { return op->dev; }
}  // namespace ophip

extern "C" {

int ophip_mat_mul_plan(const ophip_mat_mul_args *args, ophip_mat_mul_layout *out) {
    return guard([&] {
        if (!args || !out) throw args_not_support("null argument");
        *out = mat_mul_layout(*args);
    });
}

int ophip_mat_mul_create(ophip_device *dev, ophip_mat_mul **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_mat_mul(dev);
    });
}
void ophip_mat_mul_destroy(ophip_mat_mul *op) { delete op; }

// The reference's scheme() prepares nothing and never fails (mat_mul/cuda/mod.rs:30-37): the
// composites rely on that and hand it layouts that are not even a valid product
// (attention/operator.rs:104-128 passes q and the untransposed k).  Here it additionally
// reports the split-K workspace when the arguments already describe a launchable product;
// anything else is left for launch() to judge.
int ophip_mat_mul_scheme(ophip_mat_mul *op, const ophip_mat_mul_args *args, size_t max_ws, size_t *ws) {
    return guard([&] {
        if (ws) *ws = 0;
        if (!op || !args) return;
        try {
            const ophip_mat_mul_layout L = mat_mul_layout(*args);
            if (!mat_mul_takes(L.dt)) return;
            if (L.m == 0 || L.n == 0 || L.batch == 0) return;  // nothing to compute, nothing to plan (launch returns at once)
            const GemmPlan g = make_plan(*args, L, (unsigned)op->dev->props.multiProcessorCount, op->knobs);
            if (ws && g.workspace <= max_ws) *ws = g.workspace;
        } catch (const Error &) {
        }
    });
}

int ophip_mat_mul_describe(const ophip_mat_mul *op, const ophip_mat_mul_args *args, char *out, size_t len) {
    return guard([&] {
        if (!args || !out || len == 0) throw args_not_support("null argument");
        const ophip_mat_mul_layout L = mat_mul_layout(*args);
        if (!mat_mul_takes(L.dt)) throw type_not_support("mat_mul supports f16, bf16, f32 and f64");
        if (L.m == 0 || L.n == 0 || L.batch == 0) {
            std::snprintf(out, len, "empty");
            return;
        }
        const GemmPlan g = op ? make_plan(*args, L, (unsigned)op->dev->props.multiProcessorCount, op->knobs)
                              : make_plan(*args, L, 256u, GemmKnobs::from_env());
        if (g.kind == GemmPlan::Skinny)
            if (g.qmode == 4 && g.p.slow_mask)
                std::snprintf(out, len, "stream rows<=16 qN split_k=%u (%u on granule classes 0x%02x)", g.p.split_k, g.p.split_slow,
                              g.p.slow_mask);
            else if (g.qmode == 4)
                std::snprintf(out, len, "stream rows<=16 qN split_k=%u", g.p.split_k);
            else
                std::snprintf(out, len, "skinny rows<=%d q%s split_k=%u", 16 * g.mt,
                              g.qmode == 0 ? "N" : g.qmode == 1 ? "K" : g.qmode == 2 ? "K256" : "N paired", g.p.split_k);
        else if (g.kind == GemmPlan::Tile)
            std::snprintf(out, len, "tile%dx%d%s p%s q%s split_k=%u", g.tile, g.tk,
                          g.ragged ? " ragged" : "", g.pk ? "K" : "M", g.qk ? "K" : "N", g.p.split_k);
        else
            std::snprintf(out, len, "generic");
    });
}

int ophip_mat_mul_launch(const ophip_mat_mul *op, const ophip_mat_mul_args *args, void *workspace,
                         size_t workspace_len, const ophip_queue_alloc *qa) {
    return guard([&] { mat_mul_launch_impl(op, args, workspace, workspace_len, qa, nullptr, 0, stream_of(qa)); });
}

}  // extern "C"
