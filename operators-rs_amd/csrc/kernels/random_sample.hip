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
// sampling, top_k <= 1024 (`sample_topk`): the reference's answer always lies
// in the first min(top_k, n) entries of the order (value descending, index
// ascending), so no full sort is needed:
//   1. radix-select the k-th largest key (8-bit digits through an LDS histogram),
//      and, if the k-th value is tied, radix-select on the index among the ties;
//   2. gather exactly k candidates, bitonic-sort them in LDS by (value desc, idx asc);
//   3. the f32 running sum over those k entries is done by ONE lane in sorted
//      order, each term being exp() evaluated in f64 and rounded once to f32, so
//      cum[0..k) follows the sequential definition; the sum over all n entries
//      (needed for top_p) is a parallel f32 reduction in a fixed order.
// sampling, any top_k (`sample_full`): full bitonic sort in a global workspace,
// then the same sequential scan over all n entries.
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
    for (int i = threadIdx.x; i < n; i += SB) {
        const float v = Logit<T>::value(Logit<T>::bits(row, i));
        if (v != v) last_nan = i;
        else if (!(b.v > v)) b = Best{v, i};
    }
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

// exp() the way a correctly rounded expf would return it
__device__ __forceinline__ float exp_cr(float x) { return (float)exp((double)x); }

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
__device__ __forceinline__ void bitonic_lds(uint64_t *a, uint32_t cnt, uint32_t k2_first,
                                            uint32_t k2_last, uint32_t j_cap, uint32_t base) {
    for (uint32_t k2 = k2_first; k2 <= k2_last; k2 <<= 1) {
        uint32_t j = k2 >> 1;
        if (j > j_cap) j = j_cap;
        for (; j > 0; j >>= 1) {
            for (uint32_t t = threadIdx.x; t < cnt / 2; t += SB) {
                const uint32_t i = 2 * t - (t & (j - 1));
                const uint32_t l = i + j;
                const bool desc = (((base + i) & k2) == 0);
                const uint64_t x = a[i], y = a[l];
                if ((x < y) == desc) {
                    a[i] = y;
                    a[l] = x;
                }
            }
            __syncthreads();
        }
    }
}

template <typename T>
__device__ __forceinline__ void sample_topk_impl(const SampleParams &p) {
    typedef Logit<T> L;
    __shared__ uint32_t hist[256];
    __shared__ uint32_t s_sel[2];
    __shared__ uint32_t s_cnt;
    __shared__ uint64_t cand[SB];
    __shared__ float s_cum[SB];
    __shared__ float s_red[SB / WAVE];

    const char *row = reinterpret_cast<const char *>(p.logits) + (int64_t)blockIdx.x * p.row_stride;
    const uint32_t n = p.n, k = p.k_eff;

    // 1a. k-th largest key
    uint32_t prefix = 0, krem = k, eq_count = 0;
    for (int shift = L::KEY_BITS - 8; shift >= 0; shift -= 8) {
        if (threadIdx.x < 256) hist[threadIdx.x] = 0;
        __syncthreads();
        const bool first = shift == L::KEY_BITS - 8;
        for (uint32_t i = threadIdx.x; i < n; i += SB) {
            const uint32_t key = L::key(L::bits(row, i));
            if (first || (key >> (shift + 8)) == (prefix >> (shift + 8)))
                atomicAdd(&hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t acc = 0;
            int b = 255;
            for (; b > 0; --b) {
                const uint32_t c = hist[b];
                if (acc + c >= krem) break;
                acc += c;
            }
            s_sel[0] = prefix | ((uint32_t)b << shift);
            s_sel[1] = krem - acc;
        }
        __syncthreads();
        prefix = s_sel[0];
        krem = s_sel[1];
        eq_count = hist[(prefix >> shift) & 255u];
        __syncthreads();
    }
    const uint32_t kstar = prefix;  // k-th largest key; `krem` of the `eq_count` ties are wanted

    // 1b. among the ties, the krem-th smallest index
    uint32_t istar = 0xffffffffu;
    if (eq_count > krem) {  // uniform branch
        uint32_t ipre = 0, irem = krem;
        for (int shift = 24; shift >= 0; shift -= 8) {
            if (threadIdx.x < 256) hist[threadIdx.x] = 0;
            __syncthreads();
            for (uint32_t i = threadIdx.x; i < n; i += SB) {
                if (L::key(L::bits(row, i)) != kstar) continue;
                if (shift == 24 || (i >> (shift + 8)) == (ipre >> (shift + 8)))
                    atomicAdd(&hist[(i >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (threadIdx.x == 0) {
                uint32_t acc = 0;
                int b = 0;
                for (; b < 255; ++b) {
                    const uint32_t c = hist[b];
                    if (acc + c >= irem) break;
                    acc += c;
                }
                s_sel[0] = ipre | ((uint32_t)b << shift);
                s_sel[1] = irem - acc;
            }
            __syncthreads();
            ipre = s_sel[0];
            irem = s_sel[1];
            __syncthreads();
        }
        istar = ipre;
    }

    // 2. gather exactly k candidates, pad to a power of two, sort
    uint32_t P = 64;
    while (P < k) P <<= 1;
    if (threadIdx.x == 0) s_cnt = 0;
    for (uint32_t i = threadIdx.x; i < P; i += SB) cand[i] = 0;
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < n; i += SB) {
        const uint32_t key = L::key(L::bits(row, i));
        if (key > kstar || (key == kstar && i <= istar)) {
            const uint32_t slot = atomicAdd(&s_cnt, 1u);
            if (slot < SB) cand[slot] = composite(key, i);
        }
    }
    __syncthreads();
    bitonic_lds(cand, P, 2, P, P, 0);

    // 3. running sums
    const float mx = L::value(L::unkey(comp_key(cand[0])));
    const float t = p.temperature;
    float part = 0.f;
    for (uint32_t i = threadIdx.x; i < n; i += SB)
        part += expf((L::value(L::bits(row, i)) - mx) / t);
    const float total = block_sum_f32(part, s_red);
    if (threadIdx.x < k)
        s_cum[threadIdx.x] = threadIdx.x == 0
                                 ? 1.0f
                                 : exp_cr((L::value(L::unkey(comp_key(cand[threadIdx.x]))) - mx) / t);
    __syncthreads();
    if (threadIdx.x == 0) {
        float cum = 1.0f;
        for (uint32_t i = 1; i < k; ++i) {
            cum = cum + s_cum[i];
            s_cum[i] = cum;
        }
        const float pk = cum;
        const float pp = total * p.top_p;
        const float plimit = p.seed * fminf(pk, pp);
        uint32_t ans = k - 1;
        for (uint32_t i = 0; i < k; ++i)
            if (s_cum[i] >= plimit) {
                ans = i;
                break;
            }
        KvPair *out = reinterpret_cast<KvPair *>(p.kv) + blockIdx.x;
        out->idx = comp_idx(cand[ans]);
        out->val = L::from_f32(s_cum[ans]);
    }
}

extern "C" __global__ void __launch_bounds__(SB) sample_topk_f16(SampleParams p) { sample_topk_impl<f16>(p); }
extern "C" __global__ void __launch_bounds__(SB) sample_topk_f32(SampleParams p) { sample_topk_impl<float>(p); }

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
    const size_t ws_row = (size_t)np2 * 8 + (((size_t)n * 4 + 15) & ~(size_t)15);
    uint64_t *keys = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(p.workspace) + blockIdx.x * ws_row);
    float *cum = reinterpret_cast<float *>(keys + np2);

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
        cum[i] = i == 0 ? 1.0f : exp_cr((L::value(L::unkey(comp_key(keys[i]))) - mx) / t);
    __syncthreads();
    if (threadIdx.x == 0) {
        float c = 1.0f;
        for (uint32_t i = 1; i < n; ++i) {
            c = c + cum[i];
            cum[i] = c;
        }
        s_ans = n - 1;
    }
    __syncthreads();
    const float pk = cum[p.k_eff - 1];
    const float pp = cum[n - 1] * p.top_p;
    const float plimit = p.seed * fminf(pk, pp);
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
