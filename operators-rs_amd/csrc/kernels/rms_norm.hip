// rms_norm for gfx950:  y = (k * w) * x,  k = 1 / sqrt(mean(x^2) + eps).
//
// A row of d elements is owned by a group of G threads (one wave, or a whole
// 256/1024-thread workgroup for few or long rows).  Each thread pulls 16-byte
// vectors of x, keeps up to CACHE of them in registers, and the row is read
// from HBM exactly once; w is shared by all rows and stays in L2.
// Sum of squares: per-thread f32 partials, wave butterfly, then one LDS slot per
// wave combined in fixed order.  The product keeps the reference's (k*w)*x
// order and 1/sqrt is the IEEE divide and square root.
#include "device_util.h"

template <typename TA>
struct Vec {
    static constexpr int N = 16 / sizeof(TA);
    PackOf<TA> v;
    __device__ __forceinline__ float get(int i) const { return (float)v.e[i]; }
    __device__ __forceinline__ void set(int i, float f) { v.e[i] = (TA)f; }
};

template <typename TW>
__device__ __forceinline__ float load_w(const void *w, uint32_t j) {
    return (float)reinterpret_cast<const TW *>(w)[j];
}

// The same in two steps, so that the load can be issued before the row's reduction and the conversion done
// after it: N consecutive weights are N * sizeof(TW) / 16 vectors of 16 bytes.
template <typename TW, int N>
struct RawW {
    static constexpr int NV = N * sizeof(TW) / 16;
    u32x4 v[NV];
    __device__ __forceinline__ void load(const void *w, uint32_t j) {
#pragma unroll
        for (int c = 0; c < NV; ++c) v[c] = ld128(reinterpret_cast<const TW *>(w) + j + c * (16 / sizeof(TW)));
    }
    __device__ __forceinline__ void get(float (&out)[N]) const {
        constexpr int PER = 16 / sizeof(TW);
#pragma unroll
        for (int c = 0; c < NV; ++c) {
            PackOf<TW> p;
            p.u = v[c];
#pragma unroll
            for (int i = 0; i < PER; ++i) out[PER * c + i] = (float)p.e[i];
        }
    }
};

// N consecutive weights starting at element j (j multiple of N, base 16-byte aligned)
template <typename TW, int N>
__device__ __forceinline__ void load_w_vec(const void *w, uint32_t j, float (&out)[N]) {
    RawW<TW, N> raw;
    raw.load(w, j);
    raw.get(out);
}

template <typename TA, typename TW, int G>
__device__ __forceinline__ void rms_norm_vec(const RmsNormParams &p) {
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
    // w for the cached vectors is requested together with x: asked for after the reduction (a barrier the
    // compiler will not move a load across) it would put a second memory latency into a kernel that, on a
    // few rows, is nothing but latency
    RawW<TW, N> wraw[CACHE];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CACHE; ++c) {
        const uint32_t v = lane + c * G;
        if (v < nvec) {
            cache[c].v.u = ld128(xr + (size_t)v * 16);
            wraw[c].load(p.w, v * N);
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const float f = cache[c].get(i);
                ss += f * f;
            }
        }
    }
    for (uint32_t v = lane + CACHE * G; v < nvec; v += G) {
        Vec<TA> t;
        t.v.u = ld128(xr + (size_t)v * 16);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const float f = t.get(i);
            ss += f * f;
        }
    }
    ss = group_sum<G>(ss, smem);
    const float k = 1.0f / sqrtf(ss / (float)p.d + p.epsilon);

#pragma unroll
    for (int c = 0; c < CACHE; ++c) {
        const uint32_t v = lane + c * G;
        if (v < nvec) {
            float w[N];
            wraw[c].get(w);
            Vec<TA> o;
#pragma unroll
            for (int i = 0; i < N; ++i) o.set(i, (k * w[i]) * cache[c].get(i));
            if (live) st128(yr + (size_t)v * 16, o.v.u);
        }
    }
    for (uint32_t v = lane + CACHE * G; v < nvec; v += G) {
        Vec<TA> t, o;
        t.v.u = ld128(xr + (size_t)v * 16);
        float w[N];
        load_w_vec<TW, N>(p.w, v * N, w);
#pragma unroll
        for (int i = 0; i < N; ++i) o.set(i, (k * w[i]) * t.get(i));
        if (live) st128(yr + (size_t)v * 16, o.v.u);
    }
}

// Element-wise variant for rows that are not 16-byte friendly (odd d, odd strides).
template <typename TA, typename TW>
__device__ __forceinline__ void rms_norm_scalar(const RmsNormParams &p) {
    constexpr int G = 256;
    __shared__ float smem[G / WAVE];
    const uint32_t row = blockIdx.x;
    const TA *xr = reinterpret_cast<const TA *>(reinterpret_cast<const char *>(p.x) + (int64_t)row * p.nsx);
    TA *yr = reinterpret_cast<TA *>(reinterpret_cast<char *>(p.y) + (int64_t)row * p.nsy);
    float ss = 0.f;
    for (uint32_t j = threadIdx.x; j < p.d; j += G) {
        const float f = (float)xr[j];
        ss += f * f;
    }
    ss = group_sum<G>(ss, smem);
    const float k = 1.0f / sqrtf(ss / (float)p.d + p.epsilon);
    for (uint32_t j = threadIdx.x; j < p.d; j += G)
        yr[j] = (TA)((k * load_w<TW>(p.w, j)) * (float)xr[j]);
}


// Many short rows (d <= 4096 elements of two bytes): one wave per row, rows dealt round-robin to a
// fixed number of waves.  w is converted once and stays in registers for all rows
// of the wave; the next row's x is already in flight while the current one is reduced
// and written, so each wave keeps reads and writes streaming.
// CACHE: 16-byte vectors per lane and row: 8 (rows of up to 4096 elements) or 16 (up to 8192: twice the registers, half
// the waves per CU; two-byte weights only).
// S: vectors per lane one row takes (d <= 512 S elements); a wave takes CACHE / S consecutive rows per trip, all their
// loads in flight together: a wave on one 1 KB row at a time leaves the memory system idle
// ([524288, 512]: 52 % of 8 TB/s with one row per trip).
template <typename TA, typename TW, int CACHE = 8, int S = CACHE>
__device__ __forceinline__ void rms_norm_rows(const RmsNormParams &p) {
    constexpr int R = CACHE / S;  // rows per trip
    const uint32_t lane = threadIdx.x % WAVE;
    const uint32_t waves = gridDim.x * (WG_THREADS / WAVE);
    uint32_t row = (blockIdx.x * (WG_THREADS / WAVE) + threadIdx.x / WAVE) * R;  // first row of the trip
    const uint32_t nvec = p.d / 8;
    if (row >= p.n) return;

    // w stays in its storage type (two-byte weights: 4 registers per vector) and is widened on use
    struct WVec {
        u32x4 raw[sizeof(TW) / 2];
        __device__ __forceinline__ float get(int i) const {
            if constexpr (sizeof(TW) == 2) {
                PackOf<TW> t;
                t.u = raw[0];
                return (float)t.e[i];
            } else {
                return __uint_as_float(raw[i / 4][i % 4]);
            }
        }
    } w[S];
#pragma unroll
    for (int c = 0; c < S; ++c) {
        const uint32_t v = lane + c * WAVE;
        if (v < nvec) {
#pragma unroll
            for (int q = 0; q < (int)(sizeof(TW) / 2); ++q)
                w[c].raw[q] = ld128(reinterpret_cast<const char *>(p.w) + ((size_t)v * 8 * sizeof(TW)) + 16 * q);
        }
    }
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
        float ss[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            ss[rr] = 0.f;
#pragma unroll
            for (int c = rr * S; c < (rr + 1) * S; ++c) {
                if (lane + (c % S) * WAVE < nvec) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const float f = (float)cur[c].e[i];
                        ss[rr] += f * f;
                    }
                }
            }
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) ss[rr] = wave_sum_dpp(ss[rr]);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            if (row + rr >= p.n) break;  // wave-uniform
            const float k = 1.0f / sqrtf(ss[rr] / (float)p.d + p.epsilon);
            char *yr = reinterpret_cast<char *>(p.y) + (int64_t)(row + rr) * p.nsy;
#pragma unroll
            for (int c = rr * S; c < (rr + 1) * S; ++c) {
                const uint32_t v = lane + (c % S) * WAVE;
                if (v < nvec) {
                    PackOf<TA> o;
#pragma unroll
                    for (int i = 0; i < 8; ++i) o.e[i] = (TA)((k * w[c % S].get(i)) * (float)cur[c].e[i]);
                    st128_nt(yr + (size_t)v * 16, o.u);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < CACHE; ++c) cur[c] = nxt[c];
    }
}

extern "C" __global__ void __launch_bounds__(256) rms_norm_f16_f16_rows(RmsNormParams p) { rms_norm_rows<f16, f16>(p); }
extern "C" __global__ void __launch_bounds__(256) rms_norm_f16_f32_rows(RmsNormParams p) { rms_norm_rows<f16, float>(p); }
extern "C" __global__ void __launch_bounds__(256) rms_norm_bf16_bf16_rows(RmsNormParams p) { rms_norm_rows<bf16, bf16>(p); }
extern "C" __global__ void __launch_bounds__(256) rms_norm_bf16_f32_rows(RmsNormParams p) { rms_norm_rows<bf16, float>(p); }
#define RMS_ROWS_SHORT(NAME, TA, TW)                                                                                          \
    extern "C" __global__ void __launch_bounds__(256) rms_norm_##NAME##_rows_s1(RmsNormParams p) { rms_norm_rows<TA, TW, 8, 1>(p); } \
    extern "C" __global__ void __launch_bounds__(256) rms_norm_##NAME##_rows_s2(RmsNormParams p) { rms_norm_rows<TA, TW, 8, 2>(p); } \
    extern "C" __global__ void __launch_bounds__(256) rms_norm_##NAME##_rows_s4(RmsNormParams p) { rms_norm_rows<TA, TW, 8, 4>(p); }
RMS_ROWS_SHORT(f16_f16, f16, f16)
RMS_ROWS_SHORT(f16_f32, f16, float)
RMS_ROWS_SHORT(bf16_bf16, bf16, bf16)
RMS_ROWS_SHORT(bf16_f32, bf16, float)
extern "C" __global__ void __launch_bounds__(256) rms_norm_f16_f16_rows16(RmsNormParams p) { rms_norm_rows<f16, f16, 16>(p); }
extern "C" __global__ void __launch_bounds__(256) rms_norm_bf16_bf16_rows16(RmsNormParams p) { rms_norm_rows<bf16, bf16, 16>(p); }

#define RMS_VEC(NAME, TA, TW, G)                                                        \
    extern "C" __global__ void __launch_bounds__((G) < 256 ? 256 : (G)) NAME(RmsNormParams p) { \
        rms_norm_vec<TA, TW, G>(p);                                                     \
    }
#define RMS_SCALAR(NAME, TA, TW) \
    extern "C" __global__ void __launch_bounds__(256) NAME(RmsNormParams p) { rms_norm_scalar<TA, TW>(p); }

RMS_VEC(rms_norm_f16_f16_g64, f16, f16, 64)
RMS_VEC(rms_norm_f16_f16_g256, f16, f16, 256)
RMS_VEC(rms_norm_f16_f16_g1024, f16, f16, 1024)
RMS_VEC(rms_norm_f16_f32_g64, f16, float, 64)
RMS_VEC(rms_norm_f16_f32_g256, f16, float, 256)
RMS_VEC(rms_norm_f16_f32_g1024, f16, float, 1024)
RMS_VEC(rms_norm_f32_f32_g64, float, float, 64)
RMS_VEC(rms_norm_f32_f32_g256, float, float, 256)
RMS_VEC(rms_norm_f32_f32_g1024, float, float, 1024)
// bf16 activations with bf16 or f32 weights: what the reference's CUDA backend also compiles a kernel for
// (rms_norm/cuda/mod.rs:146-147 through handle/cuda/mod.rs:204); its CPU backend has no such pair.  Same arithmetic:
// f32 throughout, the result rounded to bf16 (nearest even).
RMS_VEC(rms_norm_bf16_bf16_g64, bf16, bf16, 64)
RMS_VEC(rms_norm_bf16_bf16_g256, bf16, bf16, 256)
RMS_VEC(rms_norm_bf16_bf16_g1024, bf16, bf16, 1024)
RMS_VEC(rms_norm_bf16_f32_g64, bf16, float, 64)
RMS_VEC(rms_norm_bf16_f32_g256, bf16, float, 256)
RMS_VEC(rms_norm_bf16_f32_g1024, bf16, float, 1024)
RMS_SCALAR(rms_norm_bf16_bf16_scalar, bf16, bf16)
RMS_SCALAR(rms_norm_bf16_f32_scalar, bf16, float)
RMS_SCALAR(rms_norm_f16_f16_scalar, f16, f16)
RMS_SCALAR(rms_norm_f16_f32_scalar, f16, float)
RMS_SCALAR(rms_norm_f32_f32_scalar, float, float)
// The remaining pairs of two- and four-byte floating types, which the reference's CUDA backend would compile a kernel
// for like for any pair of named types (rms_norm/cuda/mod.rs:117-122) and its CPU backend does not have: the
// element-wise kernel only, same arithmetic (f32 throughout, one rounding to the activations' type).
RMS_SCALAR(rms_norm_f16_bf16_scalar, f16, bf16)
RMS_SCALAR(rms_norm_bf16_f16_scalar, bf16, f16)
RMS_SCALAR(rms_norm_f32_f16_scalar, float, f16)
RMS_SCALAR(rms_norm_f32_bf16_scalar, float, bf16)

// f64 rows with f64 weights (rms_norm/common_cpu/mod.rs:84-90 lists the pair): all arithmetic in f64, as the
// reference's, one workgroup per row.  No vector variant: the hot path is f16.
extern "C" __global__ void __launch_bounds__(256) rms_norm_f64_f64_scalar(RmsNormParams p) {
    constexpr int G = 256;
    __shared__ double smem[G / WAVE];
    const uint32_t row = blockIdx.x;
    const double *xr = reinterpret_cast<const double *>(reinterpret_cast<const char *>(p.x) + (int64_t)row * p.nsx);
    double *yr = reinterpret_cast<double *>(reinterpret_cast<char *>(p.y) + (int64_t)row * p.nsy);
    const double *w = reinterpret_cast<const double *>(p.w);
    double ss = 0.0;
    for (uint32_t j = threadIdx.x; j < p.d; j += G) ss += xr[j] * xr[j];
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, WAVE);
    if ((threadIdx.x & (WAVE - 1)) == 0) smem[threadIdx.x / WAVE] = ss;
    __syncthreads();
    ss = (smem[0] + smem[1]) + (smem[2] + smem[3]);
    const double k = 1.0 / sqrt(ss / (double)p.d + (double)p.epsilon);
    for (uint32_t j = threadIdx.x; j < p.d; j += G) yr[j] = (k * w[j]) * xr[j];
}
