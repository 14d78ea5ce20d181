// layer_norm for gfx950:  y = (x - e) * (scale * k) + bias,  e = mean(x),
// k = 1 / (sqrt(mean(x^2) - e^2) + eps)  -- epsilon is added to the standard deviation,
// as the reference does (layer_norm/common_cpu/mod.rs:127-147).
//
// Same shape as rms_norm: a row is owned by a group of G threads (a wave, or a whole
// workgroup for few / long rows), up to 8 vectors per thread stay in registers so the row
// is read once, the two sums go through wave butterflies and one LDS slot per wave.  The
// output uses one fused multiply-add per element, like the reference's mul_add.
#include "device_util.h"

template <typename TA>
struct Vec {  // 16 bytes of TA
    static constexpr int N = 16 / sizeof(TA);
    PackOf<TA> v;
    __device__ __forceinline__ float get(int i) const { return (float)v.e[i]; }
    __device__ __forceinline__ void set(int i, float f) { v.e[i] = (TA)f; }
};

// N consecutive parameters starting at element j (j multiple of N, base 16-byte aligned)
template <typename TW, int N>
__device__ __forceinline__ void load_param_vec(const void *w, uint32_t j, float (&out)[N]) {
    constexpr int PER = 16 / sizeof(TW);
#pragma unroll
    for (int c = 0; c < N / PER; ++c) {
        PackOf<TW> p;
        p.u = ld128(reinterpret_cast<const TW *>(w) + j + PER * c);
#pragma unroll
        for (int i = 0; i < PER; ++i) out[PER * c + i] = (float)p.e[i];
    }
}

__device__ __forceinline__ void mean_and_scale(float sum, float sum2, uint32_t d, float eps, float &e, float &k) {
    const float n = (float)d;
    e = sum / n;
    const float e2 = sum2 / n;
    k = 1.0f / (sqrtf(e2 - e * e) + eps);
}

template <typename TA, typename TW, int G>
__device__ __forceinline__ void layer_norm_vec(const LayerNormParams &p) {
    constexpr int N = Vec<TA>::N;
    constexpr int CACHE = 8;
    constexpr int BLOCK = G < 256 ? 256 : G;
    constexpr int RPB = BLOCK / G;
    __shared__ float smem[BLOCK / WAVE];

    const uint32_t lane = threadIdx.x % G;
    uint32_t row = blockIdx.x * RPB + threadIdx.x / G;
    const bool live = row < p.n;
    if (!live) row = p.n - 1;  // keep every thread on the barriers; stores are suppressed

    const char *xr = reinterpret_cast<const char *>(p.x) + (int64_t)row * p.nsx;
    char *yr = reinterpret_cast<char *>(p.y) + (int64_t)row * p.nsy;
    const uint32_t nvec = p.d / N;

    Vec<TA> cache[CACHE];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int c = 0; c < CACHE; ++c) {
        const uint32_t v = lane + c * G;
        if (v < nvec) {
            cache[c].v.u = ld128_nt(xr + (size_t)v * 16);
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const float f = cache[c].get(i);
                s1 += f;
                s2 += f * f;
            }
        }
    }
    for (uint32_t v = lane + CACHE * G; v < nvec; v += G) {
        Vec<TA> t;
        t.v.u = ld128_nt(xr + (size_t)v * 16);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const float f = t.get(i);
            s1 += f;
            s2 += f * f;
        }
    }
    s1 = group_sum<G>(s1, smem);
    s2 = group_sum<G>(s2, smem);
    float e, k;
    mean_and_scale(s1, s2, p.d, p.epsilon, e, k);

    auto emit = [&](const Vec<TA> &x, uint32_t v) {
        float s[N], b[N];
        load_param_vec<TW, N>(p.scale, v * N, s);
        load_param_vec<TW, N>(p.bias, v * N, b);
        Vec<TA> o;
#pragma unroll
        for (int i = 0; i < N; ++i) o.set(i, __builtin_fmaf(x.get(i) - e, s[i] * k, b[i]));
        if (live) st128(yr + (size_t)v * 16, o.v.u);
    };
#pragma unroll
    for (int c = 0; c < CACHE; ++c) {
        const uint32_t v = lane + c * G;
        if (v < nvec) emit(cache[c], v);
    }
    for (uint32_t v = lane + CACHE * G; v < nvec; v += G) {
        Vec<TA> t;
        t.v.u = ld128_nt(xr + (size_t)v * 16);
        emit(t, v);
    }
}

// Element-wise variant for rows that are not 16-byte friendly (odd d, odd strides).
template <typename TA, typename TW>
__device__ __forceinline__ void layer_norm_scalar(const LayerNormParams &p) {
    constexpr int G = 256;
    __shared__ float smem[G / WAVE];
    const uint32_t row = blockIdx.x;
    const TA *xr = reinterpret_cast<const TA *>(reinterpret_cast<const char *>(p.x) + (int64_t)row * p.nsx);
    TA *yr = reinterpret_cast<TA *>(reinterpret_cast<char *>(p.y) + (int64_t)row * p.nsy);
    float s1 = 0.f, s2 = 0.f;
    for (uint32_t j = threadIdx.x; j < p.d; j += G) {
        const float f = (float)xr[j];
        s1 += f;
        s2 += f * f;
    }
    s1 = group_sum<G>(s1, smem);
    s2 = group_sum<G>(s2, smem);
    float e, k;
    mean_and_scale(s1, s2, p.d, p.epsilon, e, k);
    const TW *sc = reinterpret_cast<const TW *>(p.scale), *bi = reinterpret_cast<const TW *>(p.bias);
    for (uint32_t j = threadIdx.x; j < p.d; j += G)
        yr[j] = (TA)__builtin_fmaf((float)xr[j] - e, (float)sc[j] * k, (float)bi[j]);
}

// Many short rows of f16 or bf16 (d <= 4096): a persistent workgroup converts scale and bias to f32
// once into LDS, then each of its waves streams rows (dealt round-robin over all waves of the
// grid) with the next row's loads in flight while the current one is reduced and written.
// Per row the only global traffic left is x in and y out.
// CACHE: 16-byte vectors per lane and row: 8 (d <= 4096) or 16 (d <= 8192: 64 KiB of LDS for scale and bias, two
// workgroups per CU).
template <typename TA, typename TW, int CACHE = 8>
__device__ __forceinline__ void layer_norm_rows(const LayerNormParams &p) {
    constexpr int MAXD = CACHE * WAVE * 8;
    __shared__ float s_scale[MAXD], s_bias[MAXD];
    for (uint32_t j = threadIdx.x; j < p.d; j += WG_THREADS) {
        s_scale[j] = (float)reinterpret_cast<const TW *>(p.scale)[j];
        s_bias[j] = (float)reinterpret_cast<const TW *>(p.bias)[j];
    }
    __syncthreads();

    const uint32_t lane = threadIdx.x % WAVE;
    const uint32_t waves = gridDim.x * (WG_THREADS / WAVE);
    uint32_t row = blockIdx.x * (WG_THREADS / WAVE) + threadIdx.x / WAVE;
    const uint32_t nvec = p.d / 8;
    if (row >= p.n) return;

    PackOf<TA> cur[CACHE], nxt[CACHE];
    {
        const char *xr = reinterpret_cast<const char *>(p.x) + (int64_t)row * p.nsx;
#pragma unroll
        for (int c = 0; c < CACHE; ++c) {
            const uint32_t v = lane + c * WAVE;
            if (v < nvec) cur[c].u = ld128_nt(xr + (size_t)v * 16);
        }
    }
    for (; row < p.n; row += waves) {
        const uint32_t next = row + waves;
        if (next < p.n) {
            const char *xn = reinterpret_cast<const char *>(p.x) + (int64_t)next * p.nsx;
#pragma unroll
            for (int c = 0; c < CACHE; ++c) {
                const uint32_t v = lane + c * WAVE;
                if (v < nvec) nxt[c].u = ld128_nt(xn + (size_t)v * 16);
            }
        }
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int c = 0; c < CACHE; ++c) {
            const uint32_t v = lane + c * WAVE;
            if (v < nvec) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float f = (float)cur[c].e[i];
                    s1 += f;
                    s2 += f * f;
                }
            }
        }
        s1 = wave_sum_dpp(s1);
        s2 = wave_sum_dpp(s2);
        float e, k;
        mean_and_scale(s1, s2, p.d, p.epsilon, e, k);
        char *yr = reinterpret_cast<char *>(p.y) + (int64_t)row * p.nsy;
#pragma unroll
        for (int c = 0; c < CACHE; ++c) {
            const uint32_t v = lane + c * WAVE;
            if (v < nvec) {
                PackOf<TA> o;
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    o.e[i] = (TA)__builtin_fmaf((float)cur[c].e[i] - e, s_scale[v * 8 + i] * k, s_bias[v * 8 + i]);
                st128_nt(yr + (size_t)v * 16, o.u);
            }
        }
#pragma unroll
        for (int c = 0; c < CACHE; ++c) cur[c] = nxt[c];
    }
}

// The same for rows of up to 2048 elements.  S: vectors per lane one row takes (d <= 512 S elements); a wave takes
// CACHE / S consecutive rows per trip, all their loads in flight together ([524288, 512]: 39 % of 8 TB/s with one row
// per trip, 67 % with eight).  (A build of its own: the general form of the loop made the one-row-per-trip kernel above
// 14 points slower.)
template <typename TA, typename TW, int CACHE, int S>
__device__ __forceinline__ void layer_norm_rows_short(const LayerNormParams &p) {
    constexpr int MAXD = S * WAVE * 8, R = CACHE / S;
    __shared__ float s_scale[MAXD], s_bias[MAXD];
    for (uint32_t j = threadIdx.x; j < p.d; j += WG_THREADS) {
        s_scale[j] = (float)reinterpret_cast<const TW *>(p.scale)[j];
        s_bias[j] = (float)reinterpret_cast<const TW *>(p.bias)[j];
    }
    __syncthreads();

    const uint32_t lane = threadIdx.x % WAVE;
    const uint32_t waves = gridDim.x * (WG_THREADS / WAVE);
    uint32_t row = (blockIdx.x * (WG_THREADS / WAVE) + threadIdx.x / WAVE) * R;  // first row of the trip
    const uint32_t nvec = p.d / 8;
    if (row >= p.n) return;

    // slot c of the trip: row c / S of it, vector lane + (c % S) * 64 of that row
    PackOf<TA> cur[CACHE], nxt[CACHE];
    auto request = [&](PackOf<TA>(&buf)[CACHE], uint32_t first) {
#pragma unroll
        for (int c = 0; c < CACHE; ++c) {
            const uint32_t v = lane + (c % S) * WAVE, r = first + c / S;
            if (v < nvec && r < p.n) buf[c].u = ld128_nt(reinterpret_cast<const char *>(p.x) + (int64_t)r * p.nsx + (size_t)v * 16);
        }
    };
    request(cur, row);
    for (; row < p.n; row += waves * R) {
        if (row + waves * R < p.n) request(nxt, row + waves * R);
        float s1[R], s2[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            s1[rr] = 0.f, s2[rr] = 0.f;
#pragma unroll
            for (int c = rr * S; c < (rr + 1) * S; ++c) {
                if (lane + (c % S) * WAVE < nvec) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const float f = (float)cur[c].e[i];
                        s1[rr] += f;
                        s2[rr] += f * f;
                    }
                }
            }
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            s1[rr] = wave_sum_dpp(s1[rr]);
            s2[rr] = wave_sum_dpp(s2[rr]);
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            if (row + rr >= p.n) break;  // wave-uniform
            float e, k;
            mean_and_scale(s1[rr], s2[rr], p.d, p.epsilon, e, k);
            char *yr = reinterpret_cast<char *>(p.y) + (int64_t)(row + rr) * p.nsy;
#pragma unroll
            for (int c = rr * S; c < (rr + 1) * S; ++c) {
                const uint32_t v = lane + (c % S) * WAVE;
                if (v < nvec) {
                    PackOf<TA> o;
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        o.e[i] = (TA)__builtin_fmaf((float)cur[c].e[i] - e, s_scale[v * 8 + i] * k, s_bias[v * 8 + i]);
                    st128_nt(yr + (size_t)v * 16, o.u);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < CACHE; ++c) cur[c] = nxt[c];
    }
}

extern "C" __global__ void __launch_bounds__(256) layer_norm_f16_f16_rows(LayerNormParams p) { layer_norm_rows<f16, f16>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_f16_f32_rows(LayerNormParams p) { layer_norm_rows<f16, float>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_bf16_bf16_rows(LayerNormParams p) { layer_norm_rows<bf16, bf16>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_bf16_f32_rows(LayerNormParams p) { layer_norm_rows<bf16, float>(p); }
#define LAYER_NORM_ROWS_SHORT(NAME, TA, TW)                                                                                             \
    extern "C" __global__ void __launch_bounds__(256) layer_norm_##NAME##_rows_s1(LayerNormParams p) { layer_norm_rows_short<TA, TW, 8, 1>(p); } \
    extern "C" __global__ void __launch_bounds__(256) layer_norm_##NAME##_rows_s2(LayerNormParams p) { layer_norm_rows_short<TA, TW, 8, 2>(p); } \
    extern "C" __global__ void __launch_bounds__(256) layer_norm_##NAME##_rows_s4(LayerNormParams p) { layer_norm_rows_short<TA, TW, 8, 4>(p); }
LAYER_NORM_ROWS_SHORT(f16_f16, f16, f16)
LAYER_NORM_ROWS_SHORT(f16_f32, f16, float)
LAYER_NORM_ROWS_SHORT(bf16_bf16, bf16, bf16)
LAYER_NORM_ROWS_SHORT(bf16_f32, bf16, float)
extern "C" __global__ void __launch_bounds__(256) layer_norm_f16_f16_rows16(LayerNormParams p) { layer_norm_rows<f16, f16, 16>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_f16_f32_rows16(LayerNormParams p) { layer_norm_rows<f16, float, 16>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_bf16_bf16_rows16(LayerNormParams p) { layer_norm_rows<bf16, bf16, 16>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_bf16_f32_rows16(LayerNormParams p) { layer_norm_rows<bf16, float, 16>(p); }

#define LAYER_NORM(NAME, TA, TW)                                                                                  \
    extern "C" __global__ void __launch_bounds__(256) layer_norm_##NAME##_g64(LayerNormParams p) {                \
        layer_norm_vec<TA, TW, 64>(p);                                                                            \
    }                                                                                                             \
    extern "C" __global__ void __launch_bounds__(256) layer_norm_##NAME##_g256(LayerNormParams p) {               \
        layer_norm_vec<TA, TW, 256>(p);                                                                           \
    }                                                                                                             \
    extern "C" __global__ void __launch_bounds__(1024) layer_norm_##NAME##_g1024(LayerNormParams p) {             \
        layer_norm_vec<TA, TW, 1024>(p);                                                                          \
    }                                                                                                             \
    extern "C" __global__ void __launch_bounds__(256) layer_norm_##NAME##_scalar(LayerNormParams p) {             \
        layer_norm_scalar<TA, TW>(p);                                                                             \
    }
LAYER_NORM(f16_f16, f16, f16)
LAYER_NORM(f16_f32, f16, float)
LAYER_NORM(f32_f32, float, float)
// bf16 rows with bf16 or f32 scale and bias: pairs the reference's CUDA backend compiles a kernel for like for any
// other named types (layer_norm/cuda/mod.rs:158-159); its CPU backend has none.  f32 arithmetic, result rounded to bf16.
LAYER_NORM(bf16_bf16, bf16, bf16)
LAYER_NORM(bf16_f32, bf16, float)

// The remaining pairs of two- and four-byte floating types, which the reference's CUDA backend would compile a kernel
// for like for any pair of named types (layer_norm/cuda/mod.rs:158-159) and its CPU backend does not have: the
// element-wise kernel only, same arithmetic (f32 throughout, one rounding to the rows' type).
extern "C" __global__ void __launch_bounds__(256) layer_norm_f16_bf16_scalar(LayerNormParams p) { layer_norm_scalar<f16, bf16>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_bf16_f16_scalar(LayerNormParams p) { layer_norm_scalar<bf16, f16>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_f32_f16_scalar(LayerNormParams p) { layer_norm_scalar<float, f16>(p); }
extern "C" __global__ void __launch_bounds__(256) layer_norm_f32_bf16_scalar(LayerNormParams p) { layer_norm_scalar<float, bf16>(p); }

// f64 rows with f64 scale and bias (layer_norm/common_cpu/mod.rs:97 lists the pair): all arithmetic in f64, as the
// reference's, one workgroup per row.  No vector variant: the hot path is f16.
extern "C" __global__ void __launch_bounds__(256) layer_norm_f64_f64_scalar(LayerNormParams p) {
    constexpr int G = 256;
    __shared__ double smem[2][G / WAVE];
    const uint32_t row = blockIdx.x;
    const double *xr = reinterpret_cast<const double *>(reinterpret_cast<const char *>(p.x) + (int64_t)row * p.nsx);
    double *yr = reinterpret_cast<double *>(reinterpret_cast<char *>(p.y) + (int64_t)row * p.nsy);
    double s1 = 0.0, s2 = 0.0;
    for (uint32_t j = threadIdx.x; j < p.d; j += G) {
        const double f = xr[j];
        s1 += f;
        s2 += f * f;
    }
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
        s1 += __shfl_xor(s1, o, WAVE);
        s2 += __shfl_xor(s2, o, WAVE);
    }
    if ((threadIdx.x & (WAVE - 1)) == 0) {
        smem[0][threadIdx.x / WAVE] = s1;
        smem[1][threadIdx.x / WAVE] = s2;
    }
    __syncthreads();
    s1 = (smem[0][0] + smem[0][1]) + (smem[0][2] + smem[0][3]);
    s2 = (smem[1][0] + smem[1][1]) + (smem[1][2] + smem[1][3]);
    const double n = (double)p.d, e = s1 / n, e2 = s2 / n;
    const double k = 1.0 / (sqrt(e2 - e * e) + (double)p.epsilon);
    const double *sc = reinterpret_cast<const double *>(p.scale), *bi = reinterpret_cast<const double *>(p.bias);
    for (uint32_t j = threadIdx.x; j < p.d; j += G) yr[j] = fma(xr[j] - e, sc[j] * k, bi[j]);
}
