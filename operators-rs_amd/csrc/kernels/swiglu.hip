// swiglu for gfx950:  gate <- (a * sigmoid(a)) * b,  a = gate, b = up, f32 inside.
//
// Pure streaming: every thread moves one 16-byte vector of gate and one of up
// per step; gate and up rows carry independent byte strides because they are
// normally the two halves of one [n, 2*di] GEMM output.
#include "device_util.h"

__device__ __forceinline__ float swiglu_f32(float a, float b) {
    // same evaluation order as the reference: a * (1 / (1 + exp(-a))) * b; hardware exp2 and
    // reciprocal (1 ulp each) keep the kernel memory-bound, the result is rounded to f16 anyway
    const float sig = __builtin_amdgcn_rcpf(1.0f + fast_exp(-a));
    return (a * sig) * b;
}

// NT: more data than the caches hold (the host decides): the result is stored with the non-temporal hint as well.
// (Separate builds: a flag in the parameters would make the compiler merge the two stores of an if / else and drop the hint.)
template <typename T, bool NT>
__device__ __forceinline__ void swiglu_vec(const SwigluParams &p) {  // T: f16 or bf16
    if constexpr (NT) {
        // one vector per thread over the whole tensor (a row's vectors seldom fill whole workgroups: 11008 columns are
        // 5.4 of them; 16384 rows of them at 76 % of 8 TB/s against 71 % row by row, and two vectors per thread 75 %)
        const uint32_t g = blockIdx.x * WG_THREADS + threadIdx.x;
        if (g >= p.total) return;
        const uint32_t row = fastdiv(g, p.per_row), v = g - row * p.per_row.d;
        char *gp = reinterpret_cast<char *>(p.gate) + (int64_t)row * p.sgn + (size_t)v * 16;
        const char *up = reinterpret_cast<const char *>(p.up) + (int64_t)row * p.sun + (size_t)v * 16;
        PackOf<T> a, b, o;
        a.u = ld128_nt(gp);
        b.u = ld128_nt(up);
#pragma unroll
        for (int i = 0; i < 8; ++i) o.e[i] = (T)swiglu_f32((float)a.e[i], (float)b.e[i]);
        st128_nt(gp, o.u);
        return;
    }
    const uint32_t nvec = p.d / 8;
    for (uint32_t row = blockIdx.y; row < p.n; row += gridDim.y) {
        char *g = reinterpret_cast<char *>(p.gate) + (int64_t)row * p.sgn;
        const char *u = reinterpret_cast<const char *>(p.up) + (int64_t)row * p.sun;
        for (uint32_t v = blockIdx.x * WG_THREADS + threadIdx.x; v < nvec; v += gridDim.x * WG_THREADS) {
            PackOf<T> a, b, o;
            a.u = ld128_nt(g + (size_t)v * 16);
            b.u = ld128_nt(u + (size_t)v * 16);
#pragma unroll
            for (int i = 0; i < 8; ++i) o.e[i] = (T)swiglu_f32((float)a.e[i], (float)b.e[i]);
            st128(g + (size_t)v * 16, o.u);
        }
    }
}
extern "C" __global__ void __launch_bounds__(256) swiglu_f16_vec(SwigluParams p) { swiglu_vec<f16, false>(p); }
extern "C" __global__ void __launch_bounds__(256) swiglu_f16_vec_nt(SwigluParams p) { swiglu_vec<f16, true>(p); }
// bf16: neither backend of the reference has it for this operator; the f16 kernels on bf16 elements (f32 inside, one rounding)
extern "C" __global__ void __launch_bounds__(256) swiglu_bf16_vec(SwigluParams p) { swiglu_vec<bf16, false>(p); }
extern "C" __global__ void __launch_bounds__(256) swiglu_bf16_vec_nt(SwigluParams p) { swiglu_vec<bf16, true>(p); }

// f64 data is computed in f64, as the reference does (swiglu/common_cpu/mod.rs:74-76): the library's exp, an IEEE division
__device__ __forceinline__ double swiglu_f64(double a, double b) { return (a * (1.0 / (1.0 + exp(-a)))) * b; }

template <typename T>
__device__ __forceinline__ void swiglu_scalar(const SwigluParams &p) {
    for (uint32_t row = blockIdx.y; row < p.n; row += gridDim.y) {
        T *g = reinterpret_cast<T *>(reinterpret_cast<char *>(p.gate) + (int64_t)row * p.sgn);
        const T *u = reinterpret_cast<const T *>(reinterpret_cast<const char *>(p.up) + (int64_t)row * p.sun);
        for (uint32_t j = blockIdx.x * WG_THREADS + threadIdx.x; j < p.d; j += gridDim.x * WG_THREADS) {
            if constexpr (sizeof(T) == 8) g[j] = swiglu_f64(g[j], u[j]);
            else g[j] = (T)swiglu_f32((float)g[j], (float)u[j]);
        }
    }
}

extern "C" __global__ void __launch_bounds__(256) swiglu_f16_scalar(SwigluParams p) { swiglu_scalar<f16>(p); }
extern "C" __global__ void __launch_bounds__(256) swiglu_bf16_scalar(SwigluParams p) { swiglu_scalar<bf16>(p); }
extern "C" __global__ void __launch_bounds__(256) swiglu_f32_scalar(SwigluParams p) { swiglu_scalar<float>(p); }
extern "C" __global__ void __launch_bounds__(256) swiglu_f64_scalar(SwigluParams p) { swiglu_scalar<double>(p); }
