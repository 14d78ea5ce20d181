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
template <int VEC, int PT, int G>
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
    f16 *row = reinterpret_cast<f16 *>(reinterpret_cast<char *>(p.att) + (int64_t)h * p.sh + (int64_t)r * p.ss);

    float x[PT][VEC];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const uint32_t col0 = (lane + i * G) * VEC;
        if constexpr (VEC == 8) {
            Pack8 v;
            v.u = u32x4{0, 0, 0, 0};
            if (col0 + 8 <= p.att_len) {
                if (col0 < kept) v.u = ld128(row + col0);
            } else {
#pragma unroll
                for (int e = 0; e < 7; ++e)
                    if (col0 + e < kept) v.e[e] = row[col0 + e];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[i][e] = col0 + e < kept ? h2f(v.e[e]) : -INFINITY;
                mx = fmaxf(mx, x[i][e]);
            }
        } else {
            x[i][0] = col0 < kept ? h2f(row[col0]) : -INFINITY;
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
                x[i][e] = h2f(f2h(ex));  // the reference stores f16(e) and re-reads it
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
                Pack8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o.e[e] = col0 + e < kept ? f2h(x[i][e] * inv) : (f16)0.f;
                if (col0 + 8 <= p.att_len) {
                    st128(row + col0, o.u);
                } else {
#pragma unroll
                    for (int e = 0; e < 7; ++e)
                        if (col0 + e < p.att_len) row[col0 + e] = o.e[e];
                }
            } else {
                row[col0] = col0 < kept ? f2h(x[i][0] * inv) : (f16)0.f;
            }
        }
    }
}

// Any att_len: one 1024-thread workgroup per row, three sweeps (max; exp + sum,
// storing f16(e); scale), O(1) LDS.
extern "C" __global__ void __launch_bounds__(1024) softmax_f16_stream(SoftmaxParams p) {
    constexpr int G = 1024;
    __shared__ float smem[G / WAVE];
    const uint32_t flat = blockIdx.x;
    const uint32_t h = flat / p.seq, r = flat % p.seq;
    const uint32_t kept = kept_columns(p, r);
    f16 *row = reinterpret_cast<f16 *>(reinterpret_cast<char *>(p.att) + (int64_t)h * p.sh + (int64_t)r * p.ss);
    float mx = -INFINITY;
    for (uint32_t c = threadIdx.x; c < kept; c += G) mx = fmaxf(mx, h2f(row[c]));
    mx = group_max<G>(mx, smem);
    float sum = 0.f;
    for (uint32_t c = threadIdx.x; c < kept; c += G) {
        const float ex = fast_exp(h2f(row[c]) - mx);
        sum += ex;
        row[c] = f2h(ex);
    }
    sum = group_sum<G>(sum, smem);
    const float inv = 1.0f / sum;
    for (uint32_t c = threadIdx.x; c < kept; c += G) row[c] = f2h(h2f(row[c]) * inv);
    for (uint32_t c = kept + threadIdx.x; c < p.att_len; c += G) row[c] = (f16)0.f;
}

#define SOFTMAX_REG(VEC, PT, G)                                                                  \
    extern "C" __global__ void __launch_bounds__((G) < 256 ? 256 : (G))                          \
        softmax_f16_v##VEC##_p##PT##_g##G(SoftmaxParams p) {                                     \
        softmax_reg<VEC, PT, G>(p);                                                              \
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
