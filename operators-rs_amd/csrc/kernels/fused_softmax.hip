// Fused (causal) softmax over the last dim of att[nh, seq, att_len] for gfx950.
//
// Row (h, r) keeps the first  kept = att_len - seq + r + 1  columns (all of them
// without a mask); the rest become +0.  A row is owned by a group of G threads
// (one wave up to 2048 columns, a workgroup beyond) that holds its share of the
// row in registers, so HBM sees one read and one write per element; columns
// past `kept` are never loaded.  Rows too long for registers fall back to a
// three-sweep streaming kernel whose LDS use does not grow with att_len.
//
// Arithmetic mirrors the reference's f16 path: max-subtract, e = exp(x - max),
// the f32 sum runs over the un-rounded e while the value that is later scaled
// is the f16-rounded e:  y = f16( f32(f16(e)) * (1 / sum) ).
#include "device_util.h"

__device__ __forceinline__ uint32_t kept_columns(const SoftmaxParams &p, uint32_t r) {
    return p.causal ? p.att_len - p.seq + r + 1 : p.att_len;
}

// VEC = 8: 16-byte accesses (16-byte aligned rows; the last, partial group of an att_len that is no
// multiple of 8 goes element by element, so nothing past att_len is read or written); VEC = 1: element-wise.
// PT = register slots per thread (vectors or elements).
// T: f16, or bf16 (which neither backend of the reference has for this operator: the same arithmetic, the stored
// exponential rounded to bf16 where the f16 path rounds it to f16).
template <typename T, int VEC, int PT, int G>
__device__ __forceinline__ void softmax_reg(const SoftmaxParams &p) {
    constexpr int BLOCK = G < 256 ? 256 : G;
    constexpr int RPB = BLOCK / G;
    __shared__ float smem[BLOCK / WAVE];

    const uint32_t rows = p.nh * p.seq;
    const uint32_t lane = threadIdx.x % G;
    uint32_t flat = blockIdx.x * RPB + threadIdx.x / G;
    const bool live = flat < rows;
    if (!live) flat = rows - 1;
    const uint32_t h = flat / p.seq, r = flat % p.seq;
    const uint32_t kept = kept_columns(p, r);
    T *row = reinterpret_cast<T *>(reinterpret_cast<char *>(p.att) + (int64_t)h * p.sh + (int64_t)r * p.ss);

    float x[PT][VEC];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const uint32_t col0 = (lane + i * G) * VEC;
        if constexpr (VEC == 8) {
            PackOf<T> v;
            v.u = u32x4{0, 0, 0, 0};
            if (col0 + 8 <= p.att_len) {
                if (col0 < kept) v.u = ld128_nt(row + col0);
            } else {
#pragma unroll
                for (int e = 0; e < 7; ++e)
                    if (col0 + e < kept) v.e[e] = row[col0 + e];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[i][e] = col0 + e < kept ? (float)v.e[e] : -INFINITY;
                mx = fmaxf(mx, x[i][e]);
            }
        } else {
            x[i][0] = col0 < kept ? (float)row[col0] : -INFINITY;
            mx = fmaxf(mx, x[i][0]);
        }
    }
    mx = group_max<G>(mx, smem);

    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < PT; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const uint32_t col = (lane + i * G) * VEC + e;
            if (col < kept) {
                const float ex = fast_exp(x[i][e] - mx);
                sum += ex;
                x[i][e] = (float)(T)ex;  // the reference stores f16(e) and re-reads it
            } else {
                x[i][e] = 0.f;
            }
        }
    sum = group_sum<G>(sum, smem);
    const float inv = 1.0f / sum;

#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const uint32_t col0 = (lane + i * G) * VEC;
        if (col0 < p.att_len && live) {
            if constexpr (VEC == 8) {
                PackOf<T> o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o.e[e] = col0 + e < kept ? (T)(x[i][e] * inv) : (T)0.f;
                if (col0 + 8 <= p.att_len) {
                    st128(row + col0, o.u);
                } else {
#pragma unroll
                    for (int e = 0; e < 7; ++e)
                        if (col0 + e < p.att_len) row[col0 + e] = o.e[e];
                }
            } else {
                row[col0] = col0 < kept ? (T)(x[i][0] * inv) : (T)0.f;
            }
        }
    }
}

// Many short rows (a prefill's [nh, seq, att <= 1024] scores): a wave that serves one row of 512 columns lives for
// one load, two reductions and one store, and 16384 such waves cost more in start-up than in traffic.  Here a wave
// takes four rows at once, all their loads in flight together; under a causal mask the four are two pairs
// (r, seq - 1 - r), so every wave moves the same number of bytes whatever its place in the triangle.
// 16-byte aligned rows of a multiple of 8 columns only; PT 16-byte vectors per lane and row (att_len <= 512 * PT).
template <int PT>
__device__ __forceinline__ void softmax_rows4(const SoftmaxParams &p) {
    constexpr int ROWS = 4;
    // keep[n]: the 16 bytes that keep the first n of a vector's 8 columns.  What a row masks becomes -inf with one
    // bit-field insert per register, before anything is converted; from then on masked columns take care of
    // themselves: they never win the maximum, their exponential is 0, they add nothing to the sum, and 0 / sum is
    // the +0 the mask asks for.
    __shared__ u32x4 keep[9];
    if (threadIdx.x < 9) {
        const uint32_t n = threadIdx.x;
        u32x4 m;
#pragma unroll
        for (uint32_t w = 0; w < 4; ++w) m[w] = n >= 2 * w + 2 ? 0xffffffffu : n == 2 * w + 1 ? 0x0000ffffu : 0u;
        keep[n] = m;
    }
    __syncthreads();
    const uint32_t lane = threadIdx.x % WAVE;
    const uint32_t per_head = (p.seq + ROWS - 1) / ROWS;  // waves per head
    const uint32_t w = blockIdx.x * (WG_THREADS / WAVE) + threadIdx.x / WAVE;
    if (w >= p.nh * per_head) return;  // (no barrier below this line)
    const uint32_t h = w / per_head, j = w - h * per_head;
    const bool paired = p.seq % ROWS == 0;

    f16 *row[ROWS];
    int kept[ROWS];
    bool live[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        uint32_t r = paired ? (i % 2 == 0 ? 2 * j + i / 2 : p.seq - 1 - (2 * j + i / 2)) : ROWS * j + i;
        live[i] = r < p.seq;
        if (!live[i]) r = p.seq - 1;
        kept[i] = (int)kept_columns(p, r);
        row[i] = reinterpret_cast<f16 *>(reinterpret_cast<char *>(p.att) + (int64_t)h * p.sh + (int64_t)r * p.ss);
    }
    // att_len is a multiple of 8 (the host sends other lengths to the general kernel): a lane's vector is inside the
    // row or outside it, and what a row keeps of it is the first n of its 8 columns, n = kept - col0.
    Pack8 v[ROWS][PT];
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
#pragma unroll
        for (int q = 0; q < PT; ++q) {
            const int col0 = (int)(lane + q * WAVE) * 8;
            v[i][q].u = u32x4{0, 0, 0, 0};
            if (col0 < kept[i]) v[i][q].u = ld128_nt(row[i] + col0);
        }
    constexpr uint32_t NEG_INF2 = 0xfc00fc00u;  // two f16 -inf
    float mx[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        f16x2 m2 = __builtin_bit_cast(f16x2, NEG_INF2);
#pragma unroll
        for (int q = 0; q < PT; ++q) {
            const int n = min(max(kept[i] - (int)(lane + q * WAVE) * 8, 0), 8);
            const u32x4 m = keep[n];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                v[i][q].u[c] = (v[i][q].u[c] & m[c]) | (NEG_INF2 & ~m[c]);
                m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(f16x2, v[i][q].u[c]));  // exact: the maximum is one of them
            }
        }
        mx[i] = fmaxf(h2f(m2[0]), h2f(m2[1]));
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) mx[i] = wave_max_dpp(mx[i]);
    float x[ROWS][PT][8];
    float sum[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        sum[i] = 0.f;
        constexpr float LOG2E = 1.44269504088896340736f;
        const float shift = -mx[i] * LOG2E;  // exp(x - mx) = 2^(x * log2(e) - mx * log2(e)): one fused multiply-add per element
#pragma unroll
        for (int q = 0; q < PT; ++q)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float ex = __builtin_amdgcn_exp2f(__builtin_fmaf(h2f(v[i][q].e[e]), LOG2E, shift));
                sum[i] += ex;
                x[i][q][e] = h2f(f2h(ex));  // the reference stores f16(e) and re-reads it
            }
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) sum[i] = wave_sum_dpp(sum[i]);
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const float inv = 1.0f / sum[i];
#pragma unroll
        for (int q = 0; q < PT; ++q) {
            const uint32_t col0 = (lane + q * WAVE) * 8;
            if (col0 < p.att_len && live[i]) {
                Pack8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o.e[e] = f2h(x[i][q][e] * inv);
                st128(row[i] + col0, o.u);
            }
        }
    }
}
extern "C" __global__ void __launch_bounds__(256) softmax_f16_rows4_p1(SoftmaxParams p) { softmax_rows4<1>(p); }
extern "C" __global__ void __launch_bounds__(256) softmax_f16_rows4_p2(SoftmaxParams p) { softmax_rows4<2>(p); }

// Any att_len: one 1024-thread workgroup per row, three sweeps (max; exp + sum,
// storing f16(e); scale), O(1) LDS.
template <typename T>
__device__ __forceinline__ void softmax_stream(const SoftmaxParams &p) {  // T: f16 or bf16
    constexpr int G = 1024;
    __shared__ float smem[G / WAVE];
    const uint32_t flat = blockIdx.x;
    const uint32_t h = flat / p.seq, r = flat % p.seq;
    const uint32_t kept = kept_columns(p, r);
    T *row = reinterpret_cast<T *>(reinterpret_cast<char *>(p.att) + (int64_t)h * p.sh + (int64_t)r * p.ss);
    float mx = -INFINITY;
    for (uint32_t c = threadIdx.x; c < kept; c += G) mx = fmaxf(mx, (float)row[c]);
    mx = group_max<G>(mx, smem);
    float sum = 0.f;
    for (uint32_t c = threadIdx.x; c < kept; c += G) {
        const float ex = fast_exp((float)row[c] - mx);
        sum += ex;
        row[c] = (T)ex;
    }
    sum = group_sum<G>(sum, smem);
    const float inv = 1.0f / sum;
    for (uint32_t c = threadIdx.x; c < kept; c += G) row[c] = (T)((float)row[c] * inv);
    for (uint32_t c = kept + threadIdx.x; c < p.att_len; c += G) row[c] = (T)0.f;
}
extern "C" __global__ void __launch_bounds__(1024) softmax_f16_stream(SoftmaxParams p) { softmax_stream<f16>(p); }
extern "C" __global__ void __launch_bounds__(1024) softmax_bf16_stream(SoftmaxParams p) { softmax_stream<bf16>(p); }

// f32 and f64 rows (fuesd_softmax/common_cpu/mod.rs:147-193): the same three sweeps in the element's own arithmetic, the
// library's exp; one 1024-thread workgroup per row.  No register-resident variants: the hot path is f16.
template <typename T>
__device__ __forceinline__ void softmax_stream_wide(const SoftmaxParams &p) {
    constexpr int G = 1024;
    __shared__ T smem[G / WAVE];
    const uint32_t flat = blockIdx.x;
    const uint32_t h = flat / p.seq, r = flat % p.seq;
    const uint32_t kept = kept_columns(p, r);
    T *row = reinterpret_cast<T *>(reinterpret_cast<char *>(p.att) + (int64_t)h * p.sh + (int64_t)r * p.ss);
    const uint32_t wave = threadIdx.x / WAVE;
    auto across = [&](T v, auto op) {  // every thread ends with op over the whole workgroup, combined in a fixed order
#pragma unroll
        for (int o = WAVE / 2; o > 0; o >>= 1) v = op(v, __shfl_xor(v, o, WAVE));
        __syncthreads();
        if ((threadIdx.x & (WAVE - 1)) == 0) smem[wave] = v;
        __syncthreads();
        T s = smem[0];
#pragma unroll
        for (int i = 1; i < G / WAVE; ++i) s = op(s, smem[i]);
        return s;
    };
    T mx = -INFINITY;
    for (uint32_t c = threadIdx.x; c < kept; c += G) mx = row[c] > mx ? row[c] : mx;
    mx = across(mx, [](T a, T b) { return a > b ? a : b; });
    T sum = 0;
    for (uint32_t c = threadIdx.x; c < kept; c += G) {
        T ex;
        if constexpr (sizeof(T) == 8) ex = exp(row[c] - mx);
        else ex = expf(row[c] - mx);
        sum += ex;
        row[c] = ex;
    }
    sum = across(sum, [](T a, T b) { return a + b; });
    const T inv = (T)1 / sum;
    for (uint32_t c = threadIdx.x; c < kept; c += G) row[c] = row[c] * inv;
    for (uint32_t c = kept + threadIdx.x; c < p.att_len; c += G) row[c] = (T)0;
}
extern "C" __global__ void __launch_bounds__(1024) softmax_f32_stream(SoftmaxParams p) { softmax_stream_wide<float>(p); }
extern "C" __global__ void __launch_bounds__(1024) softmax_f64_stream(SoftmaxParams p) { softmax_stream_wide<double>(p); }

#define SOFTMAX_REG(VEC, PT, G)                                                                  \
    extern "C" __global__ void __launch_bounds__((G) < 256 ? 256 : (G))                          \
        softmax_f16_v##VEC##_p##PT##_g##G(SoftmaxParams p) {                                     \
        softmax_reg<f16, VEC, PT, G>(p);                                                         \
    }                                                                                            \
    extern "C" __global__ void __launch_bounds__((G) < 256 ? 256 : (G))                          \
        softmax_bf16_v##VEC##_p##PT##_g##G(SoftmaxParams p) {                                    \
        softmax_reg<bf16, VEC, PT, G>(p);                                                        \
    }

// vector variants: capacity = 8 * PT * G columns
SOFTMAX_REG(8, 1, 64)
SOFTMAX_REG(8, 2, 64)
SOFTMAX_REG(8, 4, 64)
SOFTMAX_REG(8, 1, 256)
SOFTMAX_REG(8, 2, 256)
SOFTMAX_REG(8, 4, 256)
SOFTMAX_REG(8, 8, 256)
SOFTMAX_REG(8, 4, 1024)
SOFTMAX_REG(8, 8, 1024)
// element-wise variants: capacity = PT * G columns
SOFTMAX_REG(1, 8, 64)
SOFTMAX_REG(1, 16, 64)
SOFTMAX_REG(1, 8, 256)
SOFTMAX_REG(1, 16, 256)
SOFTMAX_REG(1, 32, 256)
SOFTMAX_REG(1, 16, 1024)
