// random_sample for gfx950: argmax, and temperature / top-k / top-p sampling that
// returns the index the reference's sort-and-scan would return.
//
// One 1024-thread workgroup owns one row of logits (rows are independent; a
// grid of R workgroups serves R rows).  The whole row (64 KB at vocab 32000)
// stays in L2 between the sweeps of one workgroup.
//
// argmax: the reference keeps the LATER of two equal maxima and lets a NaN
// restart the scan.  A first sweep finds the last maximum among non-NaN values
// together with the index of the last NaN; only if a NaN exists does a second
// sweep redo the search on the suffix after it.
//
// sampling, top_k <= 8192 (`sample_topk`, `sample_topk_k64` for top_k <= 64): the reference's answer always lies
// in the first min(top_k, n) entries of the order (value descending, index
// ascending), so no full sort is needed:
//   1. radix-select the k-th largest key (8-bit digits through an LDS histogram),
//      and, if the k-th value is tied, radix-select on the index among the ties;
//   2. gather exactly k candidates, bitonic-sort them in LDS by (value desc, idx asc);
//   3. the f32 running sum over those k entries is done by ONE lane in sorted
//      order, each term being libm's expf restated bit for bit, so cum[0..k) is the
//      reference's; the sum over all n entries (needed for top_p) is known as an
//      interval around a parallel sum, and only a row whose draw falls between two
//      entries inside that interval pays for the sequential total (sample_settle).
// the same for rows that do not fit the registers (`sample_topk_list`): after the first digit the
// elements that can still matter (the chosen bucket and everything above it) are copied to a short list in
// LDS, in the same sweep that sums the exponentials of the whole row; the rest runs on the list.
// sampling, any top_k (`sample_full`): full bitonic sort in a global workspace, then the same sequential scan
// over all n entries (by wave 0, 64 terms at a time).  The host puts the top-k kernels in front of it with 64,
// 1024 and 8192 candidates standing in for the larger top_k: a try whose candidates already hold top_p of
// the probability gives the same answer and settles the row (a word per row in the workspace says so), and
// the kernels behind it leave that row alone.  On the peaked distributions of a language model the first
// try does; the full sort is for flat ones.
#include "device_util.h"

struct KvPair {
    uint32_t idx, val;
};

template <typename T>
struct Logit;
template <>
struct Logit<f16> {
    static constexpr int KEY_BITS = 16;
    __device__ static __forceinline__ uint32_t bits(const void *row, uint32_t i) {
        return reinterpret_cast<const uint16_t *>(row)[i];
    }
    __device__ static __forceinline__ float value(uint32_t b) {
        union { uint16_t u; f16 h; } c;
        c.u = (uint16_t)b;
        return h2f(c.h);
    }
    // order-preserving key; -0 and +0 share a key because the reference compares values
    __device__ static __forceinline__ uint32_t key(uint32_t b) {
        if (b == 0x8000u) b = 0;
        return (b & 0x8000u) ? (~b & 0xffffu) : (b | 0x8000u);
    }
    __device__ static __forceinline__ uint32_t unkey(uint32_t k) {
        return (k & 0x8000u) ? (k & 0x7fffu) : (~k & 0xffffu);
    }
    __device__ static __forceinline__ uint32_t from_f32(float f) {
        union { uint16_t u; f16 h; } c;
        c.h = f2h(f);
        return c.u;
    }
};
template <>
struct Logit<float> {
    static constexpr int KEY_BITS = 32;
    __device__ static __forceinline__ uint32_t bits(const void *row, uint32_t i) {
        return reinterpret_cast<const uint32_t *>(row)[i];
    }
    __device__ static __forceinline__ float value(uint32_t b) { return __uint_as_float(b); }
    __device__ static __forceinline__ uint32_t key(uint32_t b) {
        if (b == 0x80000000u) b = 0;
        return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    }
    __device__ static __forceinline__ uint32_t unkey(uint32_t k) {
        return (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    }
    __device__ static __forceinline__ uint32_t from_f32(float f) { return __float_as_uint(f); }
};

constexpr int SB = 1024;  // workgroup size of every kernel in this file
// the full-sort workspace of the row this workgroup serves (npow2 u64 sort keys, then n f32 running sums)
__device__ __forceinline__ char *sample_row_workspace(const SampleParams &p) {
    const size_t ws_row = (size_t)p.npow2 * 8 + (((size_t)p.n * 4 + 15) & ~(size_t)15);
    return reinterpret_cast<char *>(p.workspace) + blockIdx.x * ws_row;
}

// An earlier kernel in line has finished this row (all threads call; workgroup-uniform).
__device__ __forceinline__ bool sample_row_done(const SampleParams &p) {
    if (!(p.verify_cover & 2)) return false;
    const uint32_t todo = *reinterpret_cast<const uint32_t *>(sample_row_workspace(p));
    __syncthreads();  // everybody has read the word before anybody writes it again
    return todo == 0;
}

constexpr uint32_t KCAP = 8192;  // largest top_k the single-workgroup kernels sort in LDS (the host's TOPK_FAST_MAX)

// Calls f(index, raw bits) for every element of the row, 16 bytes per load when the
// row is 16-byte aligned (8 f16 or 4 f32 per thread and step), else element-wise.
template <typename T, typename F>
__device__ __forceinline__ void for_each_logit(const char *row, uint32_t n, F &&f) {
    constexpr uint32_t PER = 16 / sizeof(T);
    if ((reinterpret_cast<uintptr_t>(row) & 15u) == 0) {
        const uint32_t nvec = n / PER;
        for (uint32_t v = threadIdx.x; v < nvec; v += SB) {
            const u32x4 raw = ld128(row + (size_t)v * 16);
#pragma unroll
            for (uint32_t e = 0; e < PER; ++e) {
                uint32_t b;
                if constexpr (sizeof(T) == 2) b = (raw[e / 2] >> (16 * (e & 1))) & 0xffffu;
                else b = raw[e];
                f(v * PER + e, b);
            }
        }
        for (uint32_t i = nvec * PER + threadIdx.x; i < n; i += SB) f(i, Logit<T>::bits(row, i));
    } else {
        for (uint32_t i = threadIdx.x; i < n; i += SB) f(i, Logit<T>::bits(row, i));
    }
}

// A row that fits (n <= 32768) is pulled into registers once, with every load in
// flight at the same time, and all later sweeps of the workgroup run from there;
// longer or misaligned rows are swept from memory (L2) each time.
template <typename T>
struct RowCache {
    static constexpr uint32_t PER = 16 / sizeof(T);
    static constexpr int NV = 32768 / (SB * PER);  // vectors per thread: 4 for f16, 8 for f32
    u32x4 v[NV];
    bool cached;

    __device__ __forceinline__ void load(const char *row, uint32_t n) {
        cached = (reinterpret_cast<uintptr_t>(row) & 15u) == 0 && n <= (uint32_t)NV * SB * PER;
        if (!cached) return;
        const uint32_t nvec = n / PER;
#pragma unroll
        for (int c = 0; c < NV; ++c) {
            const uint32_t idx = threadIdx.x + c * SB;
            v[c] = u32x4{0, 0, 0, 0};
            if (idx < nvec) v[c] = ld128(row + (size_t)idx * 16);
        }
    }

    template <typename F>
    __device__ __forceinline__ void for_each(const char *row, uint32_t n, F &&f) const {
        if (!cached) {
            for_each_logit<T>(row, n, f);
            return;
        }
        const uint32_t nvec = n / PER;
#pragma unroll
        for (int c = 0; c < NV; ++c) {
            const uint32_t idx = threadIdx.x + c * SB;
            if (idx < nvec) {
#pragma unroll
                for (uint32_t e = 0; e < PER; ++e) {
                    uint32_t b;
                    if constexpr (sizeof(T) == 2) b = (v[c][e / 2] >> (16 * (e & 1))) & 0xffffu;
                    else b = v[c][e];
                    f(idx * PER + e, b);
                }
            }
        }
        for (uint32_t i = nvec * PER + threadIdx.x; i < n; i += SB) f(i, Logit<T>::bits(row, i));
    }
};

// ---------------------------------------------------------------- argmax ----

struct Best {
    float v;
    int idx;
};
// a beats b when it is larger, or equal and later
__device__ __forceinline__ Best best_of(Best a, Best b) {
    return (a.v > b.v || (a.v == b.v && a.idx > b.idx)) ? a : b;
}
__device__ __forceinline__ Best block_best(Best b, Best *smem) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
        Best t;
        t.v = __shfl_xor(b.v, o, WAVE);
        t.idx = __shfl_xor(b.idx, o, WAVE);
        b = best_of(b, t);
    }
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) smem[threadIdx.x / WAVE] = b;
    __syncthreads();
    Best r = smem[0];
#pragma unroll
    for (int i = 1; i < SB / WAVE; ++i) r = best_of(r, smem[i]);
    return r;
}
__device__ __forceinline__ int block_max_int(int v, int *smem) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, WAVE));
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) smem[threadIdx.x / WAVE] = v;
    __syncthreads();
    int r = smem[0];
#pragma unroll
    for (int i = 1; i < SB / WAVE; ++i) r = max(r, smem[i]);
    return r;
}

template <typename T>
__device__ __forceinline__ void argmax_impl(const SampleParams &p) {
    __shared__ Best sbest[SB / WAVE];
    __shared__ int sint[SB / WAVE];
    const char *row = reinterpret_cast<const char *>(p.logits) + (int64_t)blockIdx.x * p.row_stride;
    const int n = (int)p.n;

    Best b{-INFINITY, -1};
    int last_nan = -1;
    // within a thread indices ascend, so "replace unless strictly greater" keeps the last maximum
    for_each_logit<T>(row, (uint32_t)n, [&](uint32_t i, uint32_t bits) {
        const float v = Logit<T>::value(bits);
        if (v != v) last_nan = (int)i;
        else if (!(b.v > v)) b = Best{v, (int)i};
    });
    last_nan = block_max_int(last_nan, sint);
    b = block_best(b, sbest);
    if (last_nan >= 0) {  // uniform branch
        if (last_nan == n - 1) {
            b.idx = n - 1;
        } else {
            b = Best{-INFINITY, -1};
            for (int i = last_nan + 1 + threadIdx.x; i < n; i += SB) {
                const float v = Logit<T>::value(Logit<T>::bits(row, i));
                if (!(b.v > v)) b = Best{v, i};
            }
            b = block_best(b, sbest);
        }
    }
    if (threadIdx.x == 0) {
        KvPair *out = reinterpret_cast<KvPair *>(p.kv) + blockIdx.x;
        out->idx = (uint32_t)b.idx;
        out->val = Logit<T>::bits(row, b.idx);
    }
}

extern "C" __global__ void __launch_bounds__(SB) argmax_f16(SampleParams p) { argmax_impl<f16>(p); }
extern "C" __global__ void __launch_bounds__(SB) argmax_f32(SampleParams p) { argmax_impl<float>(p); }

// -------------------------------------------------------------- sampling ----

__device__ __forceinline__ uint64_t composite(uint32_t key, uint32_t idx) {
    return ((uint64_t)key << 32) | (uint64_t)(0xffffffffu - idx);
}
__device__ __forceinline__ uint32_t comp_key(uint64_t c) { return (uint32_t)(c >> 32); }
__device__ __forceinline__ uint32_t comp_idx(uint64_t c) { return 0xffffffffu - (uint32_t)c; }

__device__ __forceinline__ float row_seed(const SampleParams &p) { return p.seeds ? p.seeds[blockIdx.x] : p.seed; }

// expf() as the host's C library computes it, bit for bit: the reference's f32::exp is libm's expf, which is
// not correctly rounded (it differs from the rounded exact value on about 1 input in 11 500).  This is the
// published algorithm of glibc's expf (sysdeps/ieee754/flt-32/e_expf.c, from ARM's optimized routines): x * 32 / ln 2 =
// k + r, a 32-entry table of 2^(i/32) and a cubic in r, all in f64; as built for x86-64 the remainder r is one fused
// multiply-add.  Equal to the host's expf on every f32 in [-103, -0] (1 120 796 673 inputs, checked on the CPU).
static __device__ const uint64_t EXPF_TAB[32] = {
    0x3ff0000000000000, 0x3fefd9b0d3158574, 0x3fefb5586cf9890f, 0x3fef9301d0125b51, 0x3fef72b83c7d517b,
    0x3fef54873168b9aa, 0x3fef387a6e756238, 0x3fef1e9df51fdee1, 0x3fef06fe0a31b715, 0x3feef1a7373aa9cb,
    0x3feedea64c123422, 0x3feece086061892d, 0x3feebfdad5362a27, 0x3feeb42b569d4f82, 0x3feeab07dd485429,
    0x3feea47eb03a5585, 0x3feea09e667f3bcd, 0x3fee9f75e8ec5f74, 0x3feea11473eb0187, 0x3feea589994cce13,
    0x3feeace5422aa0db, 0x3feeb737b0cdc5e5, 0x3feec49182a3f090, 0x3feed503b23e255d, 0x3feee89f995ad3ad,
    0x3feeff76f2fb5e47, 0x3fef199bdd85529c, 0x3fef3720dcef9069, 0x3fef5818dcfba487, 0x3fef7c97337b9b5f,
    0x3fefa4afa2a490da, 0x3fefd0765b6e4540,
};
__device__ __forceinline__ float expf_libm(float x) {
#pragma clang fp contract(off)
    if (x < -0x1.9fe368p6f) return 0.f;  // below log(2^-150): libm's underflow result
    if (x > 0x1.62e42ep6f) return INFINITY;
    constexpr double INV_LN2_N = 0x1.71547652b82fep+0 * 32, SHIFT = 0x1.8p+52;
    constexpr double C0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32, C1 = 0x1.ebfce50fac4f3p-3 / 32 / 32,
                     C2 = 0x1.62e42ff0c52d6p-1 / 32;
    const double xd = (double)x;
    const double z = INV_LN2_N * xd;
    double kd = z + SHIFT;  // round to nearest integer: the low bits of kd's encoding hold it
    const uint64_t ki = (uint64_t)__double_as_longlong(kd);
    kd -= SHIFT;
    const double r = __builtin_fma(INV_LN2_N, xd, -kd);
    const double sc = __longlong_as_double((long long)(EXPF_TAB[ki & 31u] + (ki << 47)));
    const double q = __builtin_fma(C0, r, C1);
    const double r2 = r * r;
    double y = __builtin_fma(C2, r, 1.0);
    y = __builtin_fma(q, r2, y);
    y = y * sc;
    return (float)y;
}

__device__ __forceinline__ float block_sum_f32(float v, float *smem) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) smem[threadIdx.x / WAVE] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < SB / WAVE; ++i) s += smem[i];
    return s;
}

// Descending bitonic network over `cnt` (power of two) u64 values in LDS, all
// (k2, j) stages with k2 from k2_first and j <= j_first for the first k2.
template <typename K>
__device__ __forceinline__ void bitonic_lds(K *a, uint32_t cnt, uint32_t k2_first,
                                            uint32_t k2_last, uint32_t j_cap, uint32_t base) {
    for (uint32_t k2 = k2_first; k2 <= k2_last; k2 <<= 1) {
        uint32_t j = k2 >> 1;
        if (j > j_cap) j = j_cap;
        for (; j > 0; j >>= 1) {
            for (uint32_t t = threadIdx.x; t < cnt / 2; t += SB) {
                const uint32_t i = 2 * t - (t & (j - 1));
                const uint32_t l = i + j;
                const bool desc = (((base + i) & k2) == 0);
                const K x = a[i], y = a[l];
                if ((x < y) == desc) {
                    a[i] = y;
                    a[l] = x;
                }
            }
            __syncthreads();
        }
    }
}

// Finds, among 256 histogram bins scanned from the top (descending) or from the
// bottom, the bin in which the running count reaches `want`; writes the bin and the
// count still wanted inside it to out[0..1].  All threads call; out is valid after return.
__device__ __forceinline__ void pick_bucket(const uint32_t *hist, uint32_t want, bool descending, uint32_t *wave_tot,
                                            uint32_t *out) {
    const uint32_t lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    uint32_t bin = 0, c = 0, incl = 0;
    if (threadIdx.x < 256) {
        bin = descending ? 255u - threadIdx.x : threadIdx.x;
        c = hist[bin];
        incl = c;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
            const uint32_t t = __shfl_up(incl, o, WAVE);
            if (lane >= (uint32_t)o) incl += t;
        }
        if (lane == WAVE - 1) wave_tot[wave] = incl;
    }
    __syncthreads();
    if (threadIdx.x < 256) {
        for (uint32_t w = 0; w < wave; ++w) incl += wave_tot[w];
        const uint32_t excl = incl - c;
        if (excl < want && want <= incl) {
            out[0] = bin;
            out[1] = want - excl;
        }
    }
    __syncthreads();
}

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int m) {
    const uint32_t lo = __shfl_xor((uint32_t)v, m, WAVE), hi = __shfl_xor((uint32_t)(v >> 32), m, WAVE);
    return ((uint64_t)hi << 32) | lo;
}

// Among the elements whose key is `kstar` (there are eq_count of them), the index of the krem-th smallest
// (krem >= 1), written to *out.  each(f) calls f(index, key) for every element in play.  The tied indices
// are collected in `scratch` (LDS, room for SB of them) in one sweep and ranked by counting: ties at the k-th
// value are common with f16 logits and larger k, and are nearly always a handful.  Returns false, with nothing
// done, when there are more than SB of them: the caller then selects digit by digit.
template <typename Each>
__device__ __forceinline__ bool kth_tied_index(Each &&each, uint32_t kstar, uint32_t krem, uint32_t eq_count,
                                               uint32_t *scratch, uint32_t *counter, uint32_t *out) {
    if (eq_count > SB) return false;  // workgroup-uniform
    if (threadIdx.x == 0) *counter = 0;
    __syncthreads();
    each([&](uint32_t i, uint32_t key) {
        if (key == kstar) scratch[atomicAdd(counter, 1u)] = i;
    });
    __syncthreads();
    if (threadIdx.x < eq_count) {
        const uint32_t mine = scratch[threadIdx.x];
        uint32_t smaller = 0;
        for (uint32_t u = 0; u < eq_count; ++u) smaller += scratch[u] < mine ? 1u : 0u;
        if (smaller == krem - 1) *out = mine;
    }
    __syncthreads();
    return true;
}

// Descending sort of `cnt` <= 256 (a power of two, >= 64) u64 values in LDS by wave 0 alone: four values per
// lane in registers, exchanges inside a lane or by shuffle, no barrier per stage (the LDS network above
// spends most of its time in its 36 barriers at this size).  All threads call; the result is in `a` after return.
__device__ __forceinline__ void sort_desc_256(uint64_t *a, uint32_t cnt) {
    if (threadIdx.x < WAVE) {
        const uint32_t lane = threadIdx.x;
        uint64_t x[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) x[r] = lane * 4 + r < cnt ? a[lane * 4 + r] : 0;  // zeros sort to the end
#pragma unroll
        for (int k2 = 2; k2 <= 256; k2 <<= 1)
#pragma unroll
            for (int j = k2 >> 1; j > 0; j >>= 1) {
                if (j >= 4) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const uint32_t i = lane * 4 + r;
                        const uint64_t y = shfl_xor_u64(x[r], j / 4);
                        const bool desc = (i & k2) == 0, lower = (i & j) == 0;
                        x[r] = (lower == desc) ? (x[r] > y ? x[r] : y) : (x[r] < y ? x[r] : y);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if ((r & j) != 0) continue;  // r is the lower of the pair (r, r + j)
                        const uint32_t i = lane * 4 + r;
                        const bool desc = (i & k2) == 0;
                        const uint64_t lo = x[r] < x[r + j] ? x[r] : x[r + j], hi = x[r] < x[r + j] ? x[r + j] : x[r];
                        x[r] = desc ? hi : lo;
                        x[r + j] = desc ? lo : hi;
                    }
                }
            }
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (lane * 4 + r < cnt) a[lane * 4 + r] = x[r];
    }
    __syncthreads();
}

__device__ __forceinline__ uint32_t shfl_xor_key(uint32_t v, int m) { return __shfl_xor(v, m, WAVE); }
__device__ __forceinline__ uint64_t shfl_xor_key(uint64_t v, int m) { return shfl_xor_u64(v, m); }

// Descending sort of P (a power of two, 64 <= P <= SB * PER) keys in LDS by the whole workgroup: PER consecutive
// keys per thread in registers; exchanges at a distance below PER stay inside the thread, below 64 * PER they are
// shuffles inside the wave, and only the few stages with longer distances go through LDS with barriers (for
// 4096 keys: 10 of 78 stages; the all-LDS network above takes 36 us for them, this one 4).
// All threads call; `a` holds the result after return.
template <typename K, int PER>
__device__ __forceinline__ void block_sort_desc(K *a, uint32_t P) {
    const uint32_t first = threadIdx.x * PER;
    K x[PER];
#pragma unroll
    for (int r = 0; r < PER; ++r) x[r] = first + r < P ? a[first + r] : (K)0;
    auto settle = [&](K &mine, K other, uint32_t i, uint32_t k2, uint32_t j) {
        const bool desc = (i & k2) == 0, lower = (i & j) == 0;
        mine = (lower == desc) ? (mine > other ? mine : other) : (mine < other ? mine : other);
    };
    for (uint32_t k2 = 2; k2 <= P; k2 <<= 1)
        for (uint32_t j = k2 >> 1; j > 0; j >>= 1) {
            if (j >= (uint32_t)PER * WAVE) {
                __syncthreads();
#pragma unroll
                for (int r = 0; r < PER; ++r)
                    if (first + r < P) a[first + r] = x[r];
                __syncthreads();
#pragma unroll
                for (int r = 0; r < PER; ++r)
                    if (first + r < P) settle(x[r], a[(first + r) ^ j], first + r, k2, j);
            } else if (j >= (uint32_t)PER) {
                K y[PER];  // all the exchanges are requested before the first is used
#pragma unroll
                for (int r = 0; r < PER; ++r) y[r] = shfl_xor_key(x[r], (int)(j / PER));
#pragma unroll
                for (int r = 0; r < PER; ++r) settle(x[r], y[r], first + r, k2, j);
            } else {
#pragma unroll
                for (int jj = PER / 2; jj >= 1; jj >>= 1)
                    if (j == (uint32_t)jj) {
#pragma unroll
                        for (int r = 0; r < PER; ++r)
                            if ((r & jj) == 0) {
                                const bool desc = ((first + r) & k2) == 0;
                                const K lo = x[r] < x[r + jj] ? x[r] : x[r + jj], hi = x[r] < x[r + jj] ? x[r + jj] : x[r];
                                x[r] = desc ? hi : lo;
                                x[r + jj] = desc ? lo : hi;
                            }
                    }
            }
        }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < PER; ++r)
        if (first + r < P) a[first + r] = x[r];
    __syncthreads();
}

// ---- the total over all n entries, as the reference's sequential sum gives it -----------------------------------
//
// The reference's top_p bound is top_p * cum[n-1], the last of its sequential f32 running sums over the sorted
// row.  The kernels sum the row in parallel instead, so they only know an interval [T_lo, T_hi] that holds
// cum[n-1]; the sampled entry is a monotone function of that total, so when both ends of the interval give the same
// entry the row is settled.  Three stages, each run only by the rows the stage before could not settle:
//   0. hardware-exp2 parallel f32 sum F; cum[n-1] lies within n * 2^-24 (sequential rounding) + 6e-5 (the fast
//      exponentials and the parallel sum) of it, relatively;
//   1. the exact terms e_i (libm's expf) summed in f64, S, and E = sum of min(e_i, 2^-24 * T_hi): one sequential
//      addition errs by at most half an ulp of the running sum, and by the term itself when that is smaller, so
//      |cum[n-1] - S| <= E;
//   2. the sequential sum itself, continued from cum[k-1] over the entries behind the k candidates in sorted
//      order (sample_exact_total below).
struct TotalBounds {
    float lo, hi;
};
__device__ __forceinline__ float f32_not_above(double x) {
    float f = (float)x;
    if ((double)f > x) f = __uint_as_float(__float_as_uint(f) - 1u);  // x >= 1 here: positive, normal
    return f;
}
__device__ __forceinline__ float f32_not_below(double x) {
    float f = (float)x;
    if ((double)f < x) f = __uint_as_float(__float_as_uint(f) + 1u);
    return f;
}
__device__ __forceinline__ TotalBounds bounds_from_fast_sum(float F, uint32_t n) {
    const double seq = (double)n * 0x1p-24 * 1.001, par = 6e-5;
    TotalBounds b;
    b.lo = seq < 0.5 ? fmaxf(1.0f, f32_not_above((double)F / (1.0 + par) * (1.0 - seq))) : 1.0f;
    b.hi = seq < 0.5 ? f32_not_below((double)F / (1.0 - par) * (1.0 + seq)) : INFINITY;
    if (!(F == F)) b.lo = 1.0f, b.hi = INFINITY;
    return b;
}

__device__ __forceinline__ double block_sum_f64(double v, double *smem) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) smem[threadIdx.x / WAVE] = v;
    __syncthreads();
    double r = 0.0;
#pragma unroll
    for (int i = 0; i < SB / WAVE; ++i) r += smem[i];
    return r;
}

constexpr uint32_t XCH = 4096;  // entries sample_exact_total sorts per round
// LDS the later stages work in (the caller's histogram arrays serve again).  The members are LDS pointers by type:
// handed to a function that is not inlined as plain pointers they would make every access a flat one.
#define LDS_PTR(T) __attribute__((address_space(3))) T *
struct TotalScratchLds {
    LDS_PTR(uint32_t) hist;    // [256]
    LDS_PTR(uint32_t) hist_w;  // [SB / WAVE][256]
    LDS_PTR(uint32_t) wtot;    // [4]
    LDS_PTR(uint32_t) sel;     // [2]
    LDS_PTR(uint32_t) cnt;     // [1]
    LDS_PTR(uint32_t) keys;    // [XCH]
    LDS_PTR(double) red;       // [SB / WAVE]
    LDS_PTR(float) fl;         // [2]
};
// the same as plain pointers, made from the above inside a function (the compiler keeps track of where they point)
struct TotalScratch {
    uint32_t *hist;
    uint32_t (*hist_w)[256];
    uint32_t *wtot, *sel, *cnt, *keys;
    double *red;
    float *fl;
    __device__ __forceinline__ explicit TotalScratch(const TotalScratchLds &l)
        : hist((uint32_t *)l.hist), hist_w((uint32_t(*)[256])l.hist_w), wtot((uint32_t *)l.wtot), sel((uint32_t *)l.sel),
          cnt((uint32_t *)l.cnt), keys((uint32_t *)l.keys), red((double *)l.red), fl((float *)l.fl) {
    }
};

// Stage 1: the exact terms summed in f64 and the bound on what the sequential f32 sum can lose or gain against that
// (`t_hi`: the stage-0 upper bound of the total).  All threads call; every thread gets the interval.
// (Like sample_exact_total a function of its own that reads the row from memory: the callers' common path
// carries neither its code nor its registers.)
template <typename T>
__device__ __noinline__ TotalBounds sample_total_bounds(const char *row, uint32_t n, float mx, float t, float t_hi,
                                                        TotalScratchLds lds) {
    typedef Logit<T> L;
    const TotalScratch s(lds);
    const double h = (double)t_hi * 0x1p-24 * (1.0 + 1e-6);
    double sum = 0.0, err = 0.0;
    for_each_logit<T>(row, n, [&](uint32_t, uint32_t bits) {
        const double e = (double)expf_libm((L::value(bits) - mx) / t);
        sum += e;
        err += e < h ? e : h;
    });
    sum = block_sum_f64(sum, s.red);
    err = block_sum_f64(err, s.red);
    TotalBounds b;
    b.lo = fmaxf(1.0f, f32_not_above((sum - err) * (1.0 - 1e-9)));
    b.hi = f32_not_below((sum + err) * (1.0 + 1e-9));
    if (!(sum == sum) || !(err == err)) b.lo = 1.0f, b.hi = INFINITY;
    return b;
}

// The reference's sequential sum continued: `c` is cum[k-1]; behind the k candidates come `leftover` more entries
// with the k-th key and then every entry whose key is below it, in descending order.  They are taken in rounds of up
// to XCH keys: gathered into LDS, sorted, and added in order (add_sorted below).  The rounds' key ranges come from one
// histogram of the keys' top 12 bits (a range of whole bins that holds at most XCH keys); a row with more than XCH keys
// in one bin (heavy ties) is cut by radix-selecting the XCH-th largest key still to come instead, the entries
// with that key itself (any number of them) being one term added that many times.  The sum stops early once a term
// no longer changes it: every later term is smaller and the sum only grows.  All threads call; every thread gets
// the total.
template <typename T>
__device__ __noinline__ float sample_exact_total(const char *row, uint32_t n, float c, uint32_t kstar, uint32_t leftover,
                                                 float mx, float t, TotalScratchLds lds) {
    typedef Logit<T> L;
    const TotalScratch s(lds);
    // (the row is read from memory here even when the caller holds it in registers: this is a function of its
    // own so that its code and its registers stay out of the callers' common path)
    auto each_key = [&](auto &&f) { for_each_logit<T>(row, n, [&](uint32_t, uint32_t bits) { f(L::key(bits)); }); };
    auto term = [&](uint32_t key) { return expf_libm((L::value(L::unkey(key)) - mx) / t); };
    // `count` times the same term, by every lane of wave 0 alike; false once the sum no longer moves
    auto add_run = [&](float e, uint32_t count) {
        for (uint32_t i = 0; i < count; ++i) {
            const float nc = c + e;
            if (nc == c) return false;
            c = nc;
        }
        return true;
    };
    const bool wave0 = threadIdx.x < WAVE;
    const uint32_t lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    bool moving = true;  // between rounds wave 0 holds the sum and this flag; keep_going() tells everybody
    auto keep_going = [&]() {
        if (wave0 && lane == 0) s.fl[0] = moving ? 1.f : 0.f;
        __syncthreads();
        const bool go = s.fl[0] != 0.f;
        __syncthreads();
        return go;
    };

    // The `cnt` keys in s.keys, sorted descending, are added in parallel, yet with the sequential sum's roundings.
    // While the sum stays in one binade [2^b, 2^(b+1)), it is an integer M of 24 bits times u = 2^(b-23), and adding a
    // term e adds an integer number of u: d = e / u rounded to nearest, a fixed number except on an exact tie
    // (e / u = q + 1/2), where round-to-even makes it depend on M's parity: q + (q & 1) for even M, q + ((q + 1) & 1)
    // for odd M.  So every term is a pair (d for even M, d for odd M); pairs compose, in order, to pairs, and an
    // ordered scan gives M in front of every term.  The first term that carries M to 2^24 leaves the binade: it is
    // added in floating point, and the scan starts again behind it with the next binade's u.
    auto add_sorted = [&](uint32_t cnt) {
        for (uint32_t pos = 0; pos < cnt;) {  // (workgroup-uniform)
            if (wave0 && lane == 0) {
                const float e0 = term(s.keys[pos]);
                s.fl[0] = (c + e0 == c) ? 0.f : 1.f;  // the largest term left no longer moves the sum
                s.fl[1] = c;
                s.sel[0] = cnt;  // index of the first term that leaves the binade
            }
            __syncthreads();
            if (s.fl[0] == 0.f) {
                moving = false;
                break;
            }
            const float c_now = s.fl[1];
            const uint32_t cbits = __float_as_uint(c_now);
            const uint32_t bexp = cbits >> 23;  // biased exponent of the sum (it is >= 1.0)
            const uint32_t M = (cbits & 0x7fffffu) | 0x800000u;
            const double scale = __longlong_as_double((long long)(1023 + 23 + 127 - (int)bexp) << 52);  // 1 / u
            constexpr uint32_t PER = XCH / SB;
            uint32_t f0[PER], f1[PER];
            uint32_t t0 = 0, t1 = 0;  // this thread's terms composed
#pragma unroll
            for (uint32_t j = 0; j < PER; ++j) {
                const uint32_t i = pos + threadIdx.x * PER + j;
                f0[j] = f1[j] = 0;
                if (i < cnt) {
                    const double es = (double)term(s.keys[i]) * scale;
                    const double fl = floor(es);
                    const uint32_t q = (uint32_t)fl;
                    const double frac = es - fl;
                    if (frac == 0.5) f0[j] = q + (q & 1u), f1[j] = q + ((q + 1u) & 1u);
                    else f0[j] = f1[j] = q + (frac > 0.5 ? 1u : 0u);
                }
                const uint32_t n0 = t0 + ((t0 & 1u) ? f1[j] : f0[j]);
                const uint32_t n1 = t1 + (((t1 + 1u) & 1u) ? f1[j] : f0[j]);
                t0 = n0, t1 = n1;
            }
            // ordered inclusive scan over the threads: (l0, l1) from the left is applied first
            uint32_t i0 = t0, i1 = t1;
#pragma unroll
            for (int o = 1; o < WAVE; o <<= 1) {
                const uint32_t l0 = __shfl_up(i0, o, WAVE), l1 = __shfl_up(i1, o, WAVE);
                if (lane >= (uint32_t)o) {
                    const uint32_t n0 = l0 + ((l0 & 1u) ? i1 : i0);
                    const uint32_t n1 = l1 + (((l1 + 1u) & 1u) ? i1 : i0);
                    i0 = n0, i1 = n1;
                }
            }
            if (lane == WAVE - 1) s.hist[2 * wave] = i0, s.hist[2 * wave + 1] = i1;
            __syncthreads();
            uint32_t w0 = 0, w1 = 0;  // the waves to the left composed
            for (uint32_t w = 0; w < wave; ++w) {
                const uint32_t g0 = s.hist[2 * w], g1 = s.hist[2 * w + 1];
                const uint32_t n0 = w0 + ((w0 & 1u) ? g1 : g0);
                const uint32_t n1 = w1 + (((w1 + 1u) & 1u) ? g1 : g0);
                w0 = n0, w1 = n1;
            }
            // exclusive prefix of this thread: waves to the left, then lanes to the left
            uint32_t x0 = __shfl_up(i0, 1, WAVE), x1 = __shfl_up(i1, 1, WAVE);
            if (lane == 0) x0 = x1 = 0;
            const uint32_t Mw = M + ((M & 1u) ? w1 : w0);
            const uint32_t Mt = Mw + ((Mw & 1u) ? x1 : x0);  // M in front of this thread's first term
            uint32_t Mi = Mt;
#pragma unroll
            for (uint32_t j = 0; j < PER; ++j) {
                const uint32_t i = pos + threadIdx.x * PER + j;
                if (i < cnt) {
                    const uint32_t d = (Mi & 1u) ? f1[j] : f0[j];
                    if (Mi + d >= 0x1000000u || Mi >= 0x1000000u) {
                        atomicMin(&s.sel[0], i);
                        break;
                    }
                    Mi += d;
                }
            }
            __syncthreads();
            const uint32_t cross = s.sel[0];
            __syncthreads();
            if (cross >= cnt) {  // the whole piece stays in the binade: the last thread's M is the sum
                if (threadIdx.x == SB - 1) s.fl[1] = __uint_as_float((bexp << 23) | (Mi & 0x7fffffu));
                __syncthreads();
                c = s.fl[1];
                __syncthreads();
                break;
            }
            // the thread that owns term `cross` has M in front of it: that one term is added in floating point
            if (threadIdx.x == (cross - pos) / PER) {
                uint32_t Mc = Mt;
#pragma unroll
                for (uint32_t j = 0; j < PER; ++j)
                    if (j < (cross - pos) % PER) Mc += (Mc & 1u) ? f1[j] : f0[j];
                s.fl[1] = __uint_as_float((bexp << 23) | (Mc & 0x7fffffu)) + term(s.keys[cross]);
            }
            __syncthreads();
            c = s.fl[1];
            pos = cross + 1;
            __syncthreads();
        }
    };
    // keys picked by `take` into s.keys (up to XCH of them), sorted descending; returns how many
    auto gather_sorted = [&](uint32_t expect, auto &&take) {
        uint32_t P = 64;
        while (P < expect) P <<= 1;
        if (threadIdx.x == 0) *s.cnt = 0;
        for (uint32_t i = threadIdx.x; i < P; i += SB) s.keys[i] = 0;
        __syncthreads();
        each_key([&](uint32_t key) {
            if (take(key)) {
                const uint32_t slot = atomicAdd(s.cnt, 1u);
                if (slot < XCH) s.keys[slot] = key;
            }
        });
        __syncthreads();
        const uint32_t cnt = min(*s.cnt, XCH);
        block_sort_desc<uint32_t, XCH / SB>(s.keys, P);
        return cnt;
    };

    if (wave0 && leftover) moving = add_run(term(kstar), leftover);

    // histogram of the keys below kstar by their top 12 bits, then in place: tail[b] = keys in bins >= b
    constexpr int BSH = L::KEY_BITS - 12;
    constexpr uint32_t NBIN = 4096, BPT = NBIN / SB;
    uint32_t *tail = &s.hist_w[0][0];
    for (uint32_t i = threadIdx.x; i < NBIN; i += SB) tail[i] = 0;
    if (threadIdx.x == 0) s.sel[1] = 0;
    __syncthreads();
    each_key([&](uint32_t key) {
        if (key < kstar) atomicAdd(&tail[key >> BSH], 1u);
    });
    __syncthreads();
    {
        uint32_t mine[BPT], sum = 0, big = 0;
#pragma unroll
        for (uint32_t j = 0; j < BPT; ++j) {  // this thread's bins, highest first
            mine[j] = tail[NBIN - 1 - (threadIdx.x * BPT + j)];
            big = max(big, mine[j]);
            sum += mine[j];
            mine[j] = sum;
        }
        uint32_t incl = sum;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
            const uint32_t l = __shfl_up(incl, o, WAVE);
            if (lane >= (uint32_t)o) incl += l;
        }
        if (lane == WAVE - 1) s.hist[wave] = incl;
        atomicMax(&s.sel[1], big);
        __syncthreads();
        uint32_t base = incl - sum;
        for (uint32_t w = 0; w < wave; ++w) base += s.hist[w];
#pragma unroll
        for (uint32_t j = 0; j < BPT; ++j) tail[NBIN - 1 - (threadIdx.x * BPT + j)] = base + mine[j];
        __syncthreads();
    }
    const bool heavy = s.sel[1] > XCH;  // a bin alone overflows a round
    __syncthreads();

    if (!heavy) {
        uint32_t done = 0, bin_hi = NBIN;  // keys taken so far; bins below bin_hi are still to come
        while (keep_going() && bin_hi > 0 && tail[0] > done) {
            // the lowest bin down to which everything still to come fits one round
            uint32_t lo_b = 0, hi_b = bin_hi - 1;
            while (lo_b < hi_b) {
                const uint32_t mid = (lo_b + hi_b) / 2;
                if (tail[mid] - done <= XCH) hi_b = mid;
                else lo_b = mid + 1;
            }
            const uint32_t bin_lo = lo_b, expect = tail[bin_lo] - done;
            __syncthreads();
            if (expect) {
                const uint32_t cnt = gather_sorted(expect, [&](uint32_t key) {
                    const uint32_t bin = key >> BSH;
                    return key < kstar && bin >= bin_lo && bin < bin_hi;
                });
                add_sorted(cnt);
            }
            done += expect;
            bin_hi = bin_lo;
        }
    } else {
        uint32_t hi = kstar;  // keys below `hi` are still to come
        while (keep_going() && hi > 0) {
            // the XCH-th largest key below hi, digit by digit; the first digit's histogram also counts what is left
            uint32_t prefix = 0, krem = XCH, eq_count = 0, left = 0;
            bool all = false;  // XCH or fewer left: this round takes them all
            for (int shift = L::KEY_BITS - 8; shift >= 0 && !all; shift -= 8) {
                for (uint32_t i = threadIdx.x; i < (SB / WAVE) * 256; i += SB) (&s.hist_w[0][0])[i] = 0;
                __syncthreads();
                const bool first = shift == L::KEY_BITS - 8;
                const uint32_t hi_mask = first ? 0u : (0xffffffffu << (shift + 8));
                uint32_t *my_hist = s.hist_w[wave];
                each_key([&](uint32_t key) {
                    if (key < hi && ((key ^ prefix) & hi_mask) == 0) atomicAdd(&my_hist[(key >> shift) & 255u], 1u);
                });
                __syncthreads();
                if (threadIdx.x < 256) {
                    uint32_t cnt = 0;
#pragma unroll
                    for (int w = 0; w < SB / WAVE; ++w) cnt += s.hist_w[w][threadIdx.x];
                    s.hist[threadIdx.x] = cnt;
                }
                __syncthreads();
                if (first) {
                    for (uint32_t i = 0; i < 256; ++i) left += s.hist[i];
                    if (left <= XCH) {
                        all = true;
                        break;
                    }
                }
                pick_bucket(s.hist, krem, true, s.wtot, s.sel);
                prefix |= s.sel[0] << shift;
                krem = s.sel[1];
                eq_count = s.hist[s.sel[0]];
                __syncthreads();
            }
            if (left == 0) break;
            const uint32_t lo = all ? 0u : prefix;  // gather lo < key < hi (all: every key below hi)
            const uint32_t cnt = gather_sorted(all ? left : XCH - krem, [&](uint32_t key) { return key < hi && (all || key > lo); });
            add_sorted(cnt);
            if (all) break;
            if (wave0 && moving) moving = add_run(term(lo), eq_count);  // the entries with the selected key itself
            hi = lo;
        }
    }
    __syncthreads();
    if (wave0 && lane == 0) s.fl[1] = c;
    __syncthreads();
    return s.fl[1];
}

// Stages 0 to 2 for one row whose k candidates are sorted and summed.  Wave 0 holds the running sums: find(plimit)
// returns the first candidate whose running sum reaches plimit (k - 1 if none), emit(i) writes candidate i as the
// row's result; both are called by all lanes of wave 0 only.  `pk` is cum[k-1] (valid in wave 0), `fast_total`
// the stage-0 sum.  All threads call.
template <typename T, typename Find, typename Emit>
__device__ __forceinline__ void sample_settle(const SampleParams &p, const char *row, float fast_total, float mx, float pk,
                                              uint32_t k, uint32_t kstar, uint32_t leftover, Find &&find, Emit &&emit,
                                              const TotalScratchLds &s, uint32_t *s_state) {
    typedef Logit<T> L;
    const bool wave0 = threadIdx.x < WAVE;
    const uint32_t lane = threadIdx.x % WAVE;
    const float seed = row_seed(p), top_p = p.top_p, t = p.temperature;
    // wave 0: 1 = the row is settled (result written, or left to the next kernel in line), 0 = the interval is too wide
    auto judge = [&](float t_lo, float t_hi) -> uint32_t {
        const float pp_lo = t_lo * top_p, pp_hi = t_hi * top_p;
        if (p.verify_cover & 1) {  // k stands in for a larger top_k: do these candidates hold top_p of the mass?
            if (pk < pp_lo) {
                if (lane == 0) *reinterpret_cast<uint32_t *>(sample_row_workspace(p)) = 1u;  // no: the next kernel does the row
                return 1u;
            }
            if (!(pk >= pp_hi)) return 0u;
        }
        const float pl_lo = seed * fminf(pk, pp_lo), pl_hi = seed * fminf(pk, pp_hi);
        const uint32_t a_lo = find(pl_lo);
        const uint32_t a_hi = pl_hi == pl_lo ? a_lo : find(pl_hi);
        if (a_lo != a_hi) return 0u;
        if ((p.verify_cover & 1) && lane == 0) *reinterpret_cast<uint32_t *>(sample_row_workspace(p)) = 0u;
        emit(a_lo);
        return 1u;
    };
    const TotalBounds b0 = bounds_from_fast_sum(fast_total, p.n);
    if (wave0) {
        const uint32_t done = judge(b0.lo, b0.hi);
        if (lane == 0) *s_state = done;
    }
    __syncthreads();
    if (__builtin_expect(*s_state != 0, 1)) return;
    __syncthreads();

    // stage 1
    const TotalBounds b1 = sample_total_bounds<T>(row, p.n, mx, t, b0.hi, s);
    if (wave0) {
        const uint32_t done = judge(b1.lo, b1.hi);
        if (lane == 0) *s_state = done;
    }
    __syncthreads();
    if (__builtin_expect(*s_state != 0, 1)) return;
    __syncthreads();

    // stage 2
    const float pk_all = __shfl(pk, 0, WAVE);  // (wave 0's; the other waves' copy is not used)
    if (wave0 && lane == 0) s.fl[1] = pk_all;
    __syncthreads();
    const float total = sample_exact_total<T>(row, p.n, s.fl[1], kstar, leftover, mx, t, s);
    if (wave0) (void)judge(total, total);
}

// SMALLK: top_k <= 64, the common case (sort, prefix and search in the registers of wave 0) as a kernel of its own:
// it is short, and the code of the general case beside it cost it 3 % even unexecuted.
template <typename T, bool SMALLK>
__device__ __forceinline__ void sample_topk_impl(const SampleParams &p) {
    typedef Logit<T> L;
    __shared__ uint32_t hist[256];
    __shared__ uint32_t hist_w[SB / WAVE][256];  // one histogram per wave: 16x less contention on hot bins
    __shared__ uint32_t s_wtot[4];
    __shared__ uint32_t s_sel[2];
    __shared__ uint32_t s_cnt;
    constexpr uint32_t KC = SMALLK ? SB : KCAP;  // candidates the kernel has room for
    __shared__ uint64_t cand[KC];
    __shared__ float s_cum[KC];
    __shared__ float s_red[SB / WAVE];
    __shared__ float s_mx;
    __shared__ uint32_t s_xkeys[XCH];
    __shared__ double s_xred[SB / WAVE];
    __shared__ float s_xfl[2];
    __shared__ uint32_t s_state;

    if constexpr (!SMALLK)
        if (sample_row_done(p)) return;
    const char *row = reinterpret_cast<const char *>(p.logits) + (int64_t)blockIdx.x * p.row_stride;
    const uint32_t n = p.n, k = p.k_eff;
    RowCache<T> rc;
    rc.load(row, n);

    // 1a. k-th largest key, one 8-bit digit per sweep
    uint32_t prefix = 0, krem = k, eq_count = 0;
    for (int shift = L::KEY_BITS - 8; shift >= 0; shift -= 8) {
        for (uint32_t i = threadIdx.x; i < (SB / WAVE) * 256; i += SB) (&hist_w[0][0])[i] = 0;
        __syncthreads();
        const bool first = shift == L::KEY_BITS - 8;
        const uint32_t hi_mask = first ? 0u : (0xffffffffu << (shift + 8));
        uint32_t *my_hist = hist_w[threadIdx.x / WAVE];
        rc.for_each(row, n, [&](uint32_t, uint32_t bits) {
            const uint32_t key = L::key(bits);
            if (((key ^ prefix) & hi_mask) == 0) atomicAdd(&my_hist[(key >> shift) & 255u], 1u);
        });
        __syncthreads();
        if (threadIdx.x < 256) {
            uint32_t c = 0;
#pragma unroll
            for (int w = 0; w < SB / WAVE; ++w) c += hist_w[w][threadIdx.x];
            hist[threadIdx.x] = c;
        }
        __syncthreads();
        pick_bucket(hist, krem, true, s_wtot, s_sel);
        prefix |= s_sel[0] << shift;
        krem = s_sel[1];
        eq_count = hist[s_sel[0]];
        __syncthreads();
    }
    const uint32_t kstar = prefix;  // k-th largest key; `krem` of the `eq_count` ties are wanted

    // 1b. among the ties, the krem-th smallest index
    uint32_t istar = 0xffffffffu;
    bool ranked = false;
    if constexpr (!SMALLK) {
        if (eq_count > krem) {
            ranked = kth_tied_index([&](auto &&f) { rc.for_each(row, n, [&](uint32_t i, uint32_t bits) { f(i, L::key(bits)); }); },
                                    kstar, krem, eq_count, reinterpret_cast<uint32_t *>(cand), &s_cnt, &s_sel[0]);
            if (ranked) istar = s_sel[0];
            __syncthreads();
        }
    }
    if (eq_count > krem && !ranked) {  // uniform branch
        uint32_t ipre = 0, irem = krem;
        for (int shift = 24; shift >= 0; shift -= 8) {
            if (threadIdx.x < 256) hist[threadIdx.x] = 0;
            __syncthreads();
            const uint32_t hi_mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
            rc.for_each(row, n, [&](uint32_t i, uint32_t bits) {
                if (L::key(bits) == kstar && ((i ^ ipre) & hi_mask) == 0) atomicAdd(&hist[(i >> shift) & 255u], 1u);
            });
            __syncthreads();
            pick_bucket(hist, irem, false, s_wtot, s_sel);
            ipre |= s_sel[0] << shift;
            irem = s_sel[1];
            __syncthreads();
        }
        istar = ipre;
    }

    // 2. gather exactly k candidates, pad to a power of two
    uint32_t P = 64;
    if constexpr (!SMALLK)
        while (P < k) P <<= 1;
    if (threadIdx.x == 0) s_cnt = 0;
    for (uint32_t i = threadIdx.x; i < P; i += SB) cand[i] = 0;
    __syncthreads();
    rc.for_each(row, n, [&](uint32_t i, uint32_t bits) {
        const uint32_t key = L::key(bits);
        if (key > kstar || (key == kstar && i <= istar)) {
            const uint32_t slot = atomicAdd(&s_cnt, 1u);
            if (slot < KC) cand[slot] = composite(key, i);
        }
    });
    __syncthreads();

    const float t = p.temperature;
    const uint32_t leftover = eq_count - krem;  // entries with the k-th key that are not among the candidates
    TotalScratchLds scratch;
    scratch.hist = (LDS_PTR(uint32_t))hist, scratch.hist_w = (LDS_PTR(uint32_t)) & hist_w[0][0];
    scratch.wtot = (LDS_PTR(uint32_t))s_wtot, scratch.sel = (LDS_PTR(uint32_t))s_sel, scratch.cnt = (LDS_PTR(uint32_t)) & s_cnt;
    scratch.keys = (LDS_PTR(uint32_t))s_xkeys, scratch.red = (LDS_PTR(double))s_xred, scratch.fl = (LDS_PTR(float))s_xfl;
    if (SMALLK || P == 64) {
        // k <= 64: sort, prefix and search live in the registers of wave 0
        const uint32_t lane = threadIdx.x % WAVE;
        uint64_t x = 0;
        if (threadIdx.x < WAVE) {
            x = cand[lane];
#pragma unroll
            for (int k2 = 2; k2 <= WAVE; k2 <<= 1)
#pragma unroll
                for (int j = k2 >> 1; j > 0; j >>= 1) {
                    const uint64_t y = shfl_xor_u64(x, j);
                    const bool desc = (lane & k2) == 0, lower = (lane & j) == 0;
                    x = (lower == desc) ? (x > y ? x : y) : (x < y ? x : y);
                }
            if (lane == 0) s_mx = L::value(L::unkey(comp_key(x)));
        }
        __syncthreads();
        const float mx = s_mx;
        float part = 0.f;
        // stage 0 of the total (see sample_settle): hardware exp2 and a reciprocal keep this sweep cheap
        const float inv_t = 1.0f / t;
        rc.for_each(row, n, [&](uint32_t, uint32_t bits) { part += fast_exp((L::value(bits) - mx) * inv_t); });
        const float total = block_sum_f32(part, s_red);
        float mine = 1.0f, pk = 1.0f;
        if (threadIdx.x < WAVE) {
            float e = 0.f;
            if (lane > 0 && lane < k) e = expf_libm((L::value(L::unkey(comp_key(x))) - mx) / t);
            // cum[i] = cum[i-1] + e[i], strictly in order, every lane replaying the same chain
            float c = 1.0f;
#pragma unroll
            for (int i = 1; i < WAVE; ++i) {
                c = c + __shfl(e, i, WAVE);
                if (lane == (uint32_t)i) mine = c;
            }
            pk = c;  // terms past k are zero, so the chain ends at cum[k-1]
        }
        sample_settle<T>(
            p, row, total, mx, pk, k, kstar, leftover,
            [&](float plimit) {
                const uint64_t hit = __ballot(lane < k && mine >= plimit);
                return hit ? (uint32_t)__ffsll((long long)hit) - 1 : k - 1;
            },
            [&](uint32_t ans) {
                if (lane == ans) {
                    KvPair *out = reinterpret_cast<KvPair *>(p.kv) + blockIdx.x;
                    out->idx = comp_idx(x);
                    out->val = L::from_f32(mine);
                }
            },
            scratch, &s_state);
        return;
    }

    if constexpr (!SMALLK) {
        if (P <= 256) sort_desc_256(cand, P);
        else bitonic_lds(cand, P, 2, P, P, 0);
        // 3. running sums
        const float mx = L::value(L::unkey(comp_key(cand[0])));
        float part = 0.f;
        const float inv_t = 1.0f / t;
        rc.for_each(row, n, [&](uint32_t, uint32_t bits) { part += fast_exp((L::value(bits) - mx) * inv_t); });
        const float total = block_sum_f32(part, s_red);
        for (uint32_t i = threadIdx.x; i < P; i += SB)
            s_cum[i] = i == 0 ? 1.0f : i < k ? expf_libm((L::value(L::unkey(comp_key(cand[i]))) - mx) / t) : 0.f;
        __syncthreads();
        const uint32_t lane = threadIdx.x % WAVE;
        float pk = 1.0f;
        if (threadIdx.x < WAVE) {
            // wave 0 replays the sequential sum 64 entries at a time, carrying the running value
            float c = 0.f;
            for (uint32_t base = 0; base < P; base += WAVE) {
                const float e = s_cum[base + lane];
                float mine = 0.f;
    #pragma unroll
                for (int i = 0; i < WAVE; ++i) {
                    c = c + __shfl(e, i, WAVE);
                    if (lane == (uint32_t)i) mine = c;
                }
                s_cum[base + lane] = mine;
            }
            pk = c;  // entries past k add zero
        }
        sample_settle<T>(
            p, row, total, mx, pk, k, kstar, leftover,
            [&](float plimit) {
                for (uint32_t base = 0; base < P; base += WAVE) {
                    const uint64_t hit = __ballot(base + lane < k && s_cum[base + lane] >= plimit);
                    if (hit) return base + (uint32_t)__ffsll((long long)hit) - 1;
                }
                return k - 1;
            },
            [&](uint32_t ans) {
                if (lane == 0) {
                    KvPair *out = reinterpret_cast<KvPair *>(p.kv) + blockIdx.x;
                    out->idx = comp_idx(cand[ans]);
                    out->val = L::from_f32(s_cum[ans]);
                }
            },
            scratch, &s_state);
    }
}

extern "C" __global__ void __launch_bounds__(SB) sample_topk_k64_f16(SampleParams p) { sample_topk_impl<f16, true>(p); }
extern "C" __global__ void __launch_bounds__(SB) sample_topk_k64_f32(SampleParams p) { sample_topk_impl<float, true>(p); }
extern "C" __global__ void __launch_bounds__(SB) sample_topk_f16(SampleParams p) { sample_topk_impl<f16, false>(p); }
extern "C" __global__ void __launch_bounds__(SB) sample_topk_f32(SampleParams p) { sample_topk_impl<float, false>(p); }

constexpr uint32_t LIST_CAP = 2048;  // entries of the short list a row is cut down to after the first digit

// sample_topk for a row that does not fit the registers (more than 32768 logits, or not 16-byte aligned): every
// sweep reads it from memory at one CU's pace, so the row is cut down to a short list in LDS as early as possible.
// (For a row held in registers building the list costs more than the sweeps it saves: that case keeps
// sample_topk_impl above.)
template <typename T>
__device__ __forceinline__ void sample_topk_list_impl(const SampleParams &p) {
    typedef Logit<T> L;
    if (sample_row_done(p)) return;
    const char *row = reinterpret_cast<const char *>(p.logits) + (int64_t)blockIdx.x * p.row_stride;
    const uint32_t n = p.n;
    auto sweep_row = [&](auto &&f) { for_each_logit<T>(row, n, f); };  // f(index, raw bits) for every element
    __shared__ uint32_t hist[256];
    __shared__ uint32_t hist_w[SB / WAVE][256];  // one histogram per wave: 16x less contention on hot bins
    __shared__ uint32_t s_wtot[4];
    __shared__ uint32_t s_sel[2];
    __shared__ uint32_t s_cnt;
    constexpr uint32_t KC = KCAP;
    __shared__ uint64_t cand[KC];
    __shared__ uint64_t list[LIST_CAP];
    __shared__ float s_cum[KC];
    __shared__ float s_red[SB / WAVE];
    __shared__ uint32_t s_kmax[SB / WAVE];
    __shared__ uint32_t s_xkeys[XCH];
    __shared__ double s_xred[SB / WAVE];
    __shared__ float s_xfl[2];
    __shared__ uint32_t s_state;
    const uint32_t k = p.k_eff;
    const float t = p.temperature, inv_t = 1.0f / t;

    // 1a. k-th largest key, one 8-bit digit per sweep.  The first sweep also finds the largest key (the
    // maximum every exponent is taken against).  If few enough elements share the first digit of the
    // k-th key or lie above it, a second sweep copies them to a short list in LDS, summing the
    // exponentials of the whole row on the way, and every later sweep runs over that list: two passes
    // over the row instead of five or more, which is what a row too long for registers pays for.
    uint32_t prefix = 0, krem = k, eq_count = 0, nlist = 0;
    bool use_list = false;  // workgroup-uniform
    float total = 0.f, mx = 0.f;
    // f(index, key) for every element still in play
    auto each = [&](auto &&f) {
        if (use_list) {
            for (uint32_t e = threadIdx.x; e < nlist; e += SB) {
                const uint64_t c = list[e];
                f(comp_idx(c), comp_key(c));
            }
        } else {
            sweep_row([&](uint32_t i, uint32_t bits) { f(i, L::key(bits)); });
        }
    };
    for (int shift = L::KEY_BITS - 8; shift >= 0; shift -= 8) {
        for (uint32_t i = threadIdx.x; i < (SB / WAVE) * 256; i += SB) (&hist_w[0][0])[i] = 0;
        __syncthreads();
        const bool first = shift == L::KEY_BITS - 8;
        const uint32_t hi_mask = first ? 0u : (0xffffffffu << (shift + 8));
        uint32_t *my_hist = hist_w[threadIdx.x / WAVE];
        uint32_t kmax = 0;
        each([&](uint32_t, uint32_t key) {
            if (first) kmax = max(kmax, key);
            if (((key ^ prefix) & hi_mask) == 0) atomicAdd(&my_hist[(key >> shift) & 255u], 1u);
        });
        if (first) {
#pragma unroll
            for (int o = WAVE / 2; o > 0; o >>= 1) kmax = max(kmax, (uint32_t)__shfl_xor((int)kmax, o, WAVE));
            if (threadIdx.x % WAVE == 0) s_kmax[threadIdx.x / WAVE] = kmax;
        }
        __syncthreads();
        if (threadIdx.x < 256) {
            uint32_t c = 0;
#pragma unroll
            for (int w = 0; w < SB / WAVE; ++w) c += hist_w[w][threadIdx.x];
            hist[threadIdx.x] = c;
        }
        __syncthreads();
        pick_bucket(hist, krem, true, s_wtot, s_sel);
        const uint32_t above = krem - s_sel[1];  // elements in the buckets above the chosen one
        prefix |= s_sel[0] << shift;
        krem = s_sel[1];
        eq_count = hist[s_sel[0]];
        if (first) {
            uint32_t km = 0;
#pragma unroll
            for (int w = 0; w < SB / WAVE; ++w) km = max(km, s_kmax[w]);
            mx = L::value(L::unkey(km));
            // the chosen bucket and everything above it: `above + eq_count` elements
            if (above + eq_count <= LIST_CAP) {
                if (threadIdx.x == 0) s_cnt = 0;
                __syncthreads();
                const uint32_t floor_digit = s_sel[0];
                float part = 0.f;
                // (the total only feeds the top_p bound: hardware exp2 and a reciprocal keep this sweep cheap)
                sweep_row([&](uint32_t i, uint32_t bits) {
                    part += fast_exp((L::value(bits) - mx) * inv_t);
                    const uint32_t key = L::key(bits);
                    if ((key >> shift) >= floor_digit) list[atomicAdd(&s_cnt, 1u)] = composite(key, i);
                });
                total = block_sum_f32(part, s_red);
                __syncthreads();
                nlist = s_cnt;
                use_list = true;  // (the elements above the chosen bucket are in the list for the gather step)
            }
        }
        __syncthreads();
    }
    const uint32_t kstar = prefix;  // k-th largest key; `krem` of the `eq_count` ties are wanted

    // 1b. among the ties, the krem-th smallest index
    uint32_t istar = 0xffffffffu;
    bool ranked = false;
    if (eq_count > krem) {
        ranked = kth_tied_index(each, kstar, krem, eq_count, reinterpret_cast<uint32_t *>(cand), &s_cnt, &s_sel[0]);
        if (ranked) istar = s_sel[0];
        __syncthreads();
    }
    if (eq_count > krem && !ranked) {  // uniform branch
        uint32_t ipre = 0, irem = krem;
        for (int shift = 24; shift >= 0; shift -= 8) {
            if (threadIdx.x < 256) hist[threadIdx.x] = 0;
            __syncthreads();
            const uint32_t hi_mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
            each([&](uint32_t i, uint32_t key) {
                if (key == kstar && ((i ^ ipre) & hi_mask) == 0) atomicAdd(&hist[(i >> shift) & 255u], 1u);
            });
            __syncthreads();
            pick_bucket(hist, irem, false, s_wtot, s_sel);
            ipre |= s_sel[0] << shift;
            irem = s_sel[1];
            __syncthreads();
        }
        istar = ipre;
    }

    // 2. gather exactly k candidates, pad to a power of two
    uint32_t P = 64;
    while (P < k) P <<= 1;
    if (threadIdx.x == 0) s_cnt = 0;
    for (uint32_t i = threadIdx.x; i < P; i += SB) cand[i] = 0;
    __syncthreads();
    each([&](uint32_t i, uint32_t key) {
        if (key > kstar || (key == kstar && i <= istar)) {
            const uint32_t slot = atomicAdd(&s_cnt, 1u);
            if (slot < KC) cand[slot] = composite(key, i);
        }
    });
    __syncthreads();
    if (!use_list) {  // the sweep the short-list path has already made
        float part = 0.f;
        sweep_row([&](uint32_t, uint32_t bits) { part += fast_exp((L::value(bits) - mx) * inv_t); });
        total = block_sum_f32(part, s_red);
    }

    const uint32_t leftover = eq_count - krem;  // entries with the k-th key that are not among the candidates
    TotalScratchLds scratch;
    scratch.hist = (LDS_PTR(uint32_t))hist, scratch.hist_w = (LDS_PTR(uint32_t)) & hist_w[0][0];
    scratch.wtot = (LDS_PTR(uint32_t))s_wtot, scratch.sel = (LDS_PTR(uint32_t))s_sel, scratch.cnt = (LDS_PTR(uint32_t)) & s_cnt;
    scratch.keys = (LDS_PTR(uint32_t))s_xkeys, scratch.red = (LDS_PTR(double))s_xred, scratch.fl = (LDS_PTR(float))s_xfl;
    const uint32_t lane = threadIdx.x % WAVE;
    if (P == 64) {
        // k <= 64: sort, prefix and search live in the registers of wave 0
        uint64_t x = 0;
        float mine = 1.0f, pk = 1.0f;
        if (threadIdx.x < WAVE) {
            x = cand[lane];
#pragma unroll
            for (int k2 = 2; k2 <= WAVE; k2 <<= 1)
#pragma unroll
                for (int j = k2 >> 1; j > 0; j >>= 1) {
                    const uint64_t y = shfl_xor_u64(x, j);
                    const bool desc = (lane & k2) == 0, lower = (lane & j) == 0;
                    x = (lower == desc) ? (x > y ? x : y) : (x < y ? x : y);
                }
            float e = 0.f;
            if (lane > 0 && lane < k) e = expf_libm((L::value(L::unkey(comp_key(x))) - mx) / t);
            // cum[i] = cum[i-1] + e[i], strictly in order, every lane replaying the same chain
            float c = 1.0f;
#pragma unroll
            for (int i = 1; i < WAVE; ++i) {
                c = c + __shfl(e, i, WAVE);
                if (lane == (uint32_t)i) mine = c;
            }
            pk = c;  // terms past k are zero, so the chain ends at cum[k-1]
        }
        sample_settle<T>(
            p, row, total, mx, pk, k, kstar, leftover,
            [&](float plimit) {
                const uint64_t hit = __ballot(lane < k && mine >= plimit);
                return hit ? (uint32_t)__ffsll((long long)hit) - 1 : k - 1;
            },
            [&](uint32_t ans) {
                if (lane == ans) {
                    KvPair *out = reinterpret_cast<KvPair *>(p.kv) + blockIdx.x;
                    out->idx = comp_idx(x);
                    out->val = L::from_f32(mine);
                }
            },
            scratch, &s_state);
        return;
    }

    if (P <= 256) sort_desc_256(cand, P);
    else bitonic_lds(cand, P, 2, P, P, 0);
    // 3. running sums
    for (uint32_t i = threadIdx.x; i < P; i += SB)
        s_cum[i] = i == 0 ? 1.0f : i < k ? expf_libm((L::value(L::unkey(comp_key(cand[i]))) - mx) / t) : 0.f;
    __syncthreads();
    float pk = 1.0f;
    if (threadIdx.x < WAVE) {
        // wave 0 replays the sequential sum 64 entries at a time, carrying the running value
        float c = 0.f;
        for (uint32_t base = 0; base < P; base += WAVE) {
            const float e = s_cum[base + lane];
            float mine = 0.f;
#pragma unroll
            for (int i = 0; i < WAVE; ++i) {
                c = c + __shfl(e, i, WAVE);
                if (lane == (uint32_t)i) mine = c;
            }
            s_cum[base + lane] = mine;
        }
        pk = c;  // entries past k add zero
    }
    sample_settle<T>(
        p, row, total, mx, pk, k, kstar, leftover,
        [&](float plimit) {
            for (uint32_t base = 0; base < P; base += WAVE) {
                const uint64_t hit = __ballot(base + lane < k && s_cum[base + lane] >= plimit);
                if (hit) return base + (uint32_t)__ffsll((long long)hit) - 1;
            }
            return k - 1;
        },
        [&](uint32_t ans) {
            if (lane == 0) {
                KvPair *out = reinterpret_cast<KvPair *>(p.kv) + blockIdx.x;
                out->idx = comp_idx(cand[ans]);
                out->val = L::from_f32(s_cum[ans]);
            }
        },
        scratch, &s_state);
}

extern "C" __global__ void __launch_bounds__(SB) sample_topk_list_f16(SampleParams p) { sample_topk_list_impl<f16>(p); }
extern "C" __global__ void __launch_bounds__(SB) sample_topk_list_f32(SampleParams p) { sample_topk_list_impl<float>(p); }

// Full sort.  Workspace per row: npow2 u64 sort keys, then n f32 running sums.
constexpr uint32_t TILE = 2048;  // u64 entries sorted per LDS tile (16 KB)

template <typename T>
__device__ __forceinline__ void sample_full_impl(const SampleParams &p) {
    typedef Logit<T> L;
    __shared__ uint64_t tile[TILE];
    __shared__ float s_red[SB / WAVE];
    __shared__ uint32_t s_ans;

    const uint32_t n = p.n, np2 = p.npow2;
    const char *row = reinterpret_cast<const char *>(p.logits) + (int64_t)blockIdx.x * p.row_stride;
    uint64_t *keys = reinterpret_cast<uint64_t *>(sample_row_workspace(p));
    float *cum = reinterpret_cast<float *>(keys + np2);
    if (sample_row_done(p)) return;  // a top-k kernel ran first and finished the row

    for (uint32_t i = threadIdx.x; i < np2; i += SB)
        keys[i] = i < n ? composite(L::key(L::bits(row, i)), i) : 0;
    __syncthreads();

    const uint32_t tile_n = np2 < TILE ? np2 : TILE;
    // all stages with k2 <= tile_n are local to a tile
    for (uint32_t base = 0; base < np2; base += tile_n) {
        for (uint32_t i = threadIdx.x; i < tile_n; i += SB) tile[i] = keys[base + i];
        __syncthreads();
        bitonic_lds(tile, tile_n, 2, tile_n, tile_n, base);
        for (uint32_t i = threadIdx.x; i < tile_n; i += SB) keys[base + i] = tile[i];
        __syncthreads();
    }
    for (uint32_t k2 = tile_n << 1; k2 <= np2; k2 <<= 1) {
        for (uint32_t j = k2 >> 1; j >= tile_n; j >>= 1) {  // strides that leave a tile: in global memory
            for (uint32_t t = threadIdx.x; t < np2 / 2; t += SB) {
                const uint32_t i = 2 * t - (t & (j - 1));
                const uint32_t l = i + j;
                const bool desc = ((i & k2) == 0);
                const uint64_t x = keys[i], y = keys[l];
                if ((x < y) == desc) {
                    keys[i] = y;
                    keys[l] = x;
                }
            }
            __syncthreads();
        }
        for (uint32_t base = 0; base < np2; base += tile_n) {  // the remaining strides per tile
            for (uint32_t i = threadIdx.x; i < tile_n; i += SB) tile[i] = keys[base + i];
            __syncthreads();
            bitonic_lds(tile, tile_n, k2, k2, tile_n >> 1, base);
            for (uint32_t i = threadIdx.x; i < tile_n; i += SB) keys[base + i] = tile[i];
            __syncthreads();
        }
    }

    const float mx = L::value(L::unkey(comp_key(keys[0])));
    const float t = p.temperature;
    for (uint32_t i = threadIdx.x; i < n; i += SB)
        cum[i] = i == 0 ? 1.0f : expf_libm((L::value(L::unkey(comp_key(keys[i]))) - mx) / t);
    __syncthreads();
    if (threadIdx.x < WAVE) {
        // the sequential f32 running sum, by wave 0: 64 terms at a time are loaded together (the next 64 already
        // on their way), then every lane replays the same chain of 64 additions and keeps its own prefix
        // (0 + cum[0] is exactly the 1.0 the sum starts from; lanes past n add zeros)
        const uint32_t lane = threadIdx.x;
        float c = 0.f;
        float e = lane < n ? cum[lane] : 0.f;
        for (uint32_t base = 0; base < n; base += WAVE) {
            const uint32_t nxt = base + WAVE + lane;
            const float e_next = nxt < n ? cum[nxt] : 0.f;
            float mine = 0.f;
#pragma unroll
            for (int i = 0; i < WAVE; ++i) {
                c = c + __shfl(e, i, WAVE);
                if (lane == (uint32_t)i) mine = c;
            }
            if (base + lane < n) cum[base + lane] = mine;
            e = e_next;
        }
        if (lane == 0) s_ans = n - 1;
    }
    __syncthreads();
    const float pk = cum[p.k_eff - 1];
    const float pp = cum[n - 1] * p.top_p;
    const float plimit = row_seed(p) * fminf(pk, pp);
    uint32_t mine = 0xffffffffu;
    for (uint32_t i = threadIdx.x; i < n; i += SB)
        if (cum[i] >= plimit) {
            mine = i;
            break;
        }
    if (mine != 0xffffffffu) atomicMin(&s_ans, mine);
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t ans = s_ans;
        KvPair *out = reinterpret_cast<KvPair *>(p.kv) + blockIdx.x;
        out->idx = comp_idx(keys[ans]);
        out->val = L::from_f32(cum[ans]);
    }
    (void)s_red;
}

extern "C" __global__ void __launch_bounds__(SB) sample_full_f16(SampleParams p) { sample_full_impl<f16>(p); }
extern "C" __global__ void __launch_bounds__(SB) sample_full_f32(SampleParams p) { sample_full_impl<float>(p); }
