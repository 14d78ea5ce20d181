// gelu (tanh form) for gfx950, in place:
//   x <- 0.5 * x * (1 + tanh(sqrt(2/pi) * (x + 0.044715 * x^3)))     (gelu/common_cpu/mod.rs:112-116)
// Pure streaming: one 16-byte vector per thread step.  tanh(u) = 1 - 2 / (exp(2u) + 1) with the
// hardware exp2 and reciprocal; the result is rounded to the storage type.
#include "device_util.h"

__device__ __forceinline__ float gelu_f32(float x) {
    const float c = 0.7978845608028654f;  // sqrt(2 / pi)
    const float u = c * (x + 0.044715f * (x * x * x));
    const float t = 1.0f - 2.0f * __builtin_amdgcn_rcpf(fast_exp(2.0f * u) + 1.0f);  // exp -> inf gives 1, -> 0 gives -1
    return (0.5f * x) * (1.0f + t);
}

template <typename T>
__device__ __forceinline__ void gelu_vec(const GeluParams &p) {  // T: f16 or bf16
    const uint32_t nvec = p.d / 8;
    for (uint32_t row = blockIdx.y; row < p.n; row += gridDim.y) {
        char *r = reinterpret_cast<char *>(p.base) + (int64_t)row * p.sn;
        for (uint32_t v = blockIdx.x * WG_THREADS + threadIdx.x; v < nvec; v += gridDim.x * WG_THREADS) {
            PackOf<T> a, o;
            a.u = ld128_nt(r + (size_t)v * 16);
#pragma unroll
            for (int i = 0; i < 8; ++i) o.e[i] = (T)gelu_f32((float)a.e[i]);
            st128(r + (size_t)v * 16, o.u);  // (with the non-temporal hint on this store too a 360 MB row set loses 11 points)
        }
    }
}
extern "C" __global__ void __launch_bounds__(256) gelu_f16_vec(GeluParams p) { gelu_vec<f16>(p); }
// bf16: neither backend of the reference has it for this operator; the f16 kernel on bf16 elements
extern "C" __global__ void __launch_bounds__(256) gelu_bf16_vec(GeluParams p) { gelu_vec<bf16>(p); }

// f64 data in f64 (gelu/common_cpu/mod.rs:62-64), sqrt(2 / pi) from the f64 constant
__device__ __forceinline__ double gelu_f64(double x) {
    const double c = 0.79788456080286535588;
    return 0.5 * x * (1.0 + tanh(c * (x + 0.044715 * (x * x * x))));
}

template <typename T>
__device__ __forceinline__ void gelu_scalar(const GeluParams &p) {
    for (uint32_t row = blockIdx.y; row < p.n; row += gridDim.y) {
        T *r = reinterpret_cast<T *>(reinterpret_cast<char *>(p.base) + (int64_t)row * p.sn);
        for (uint32_t j = blockIdx.x * WG_THREADS + threadIdx.x; j < p.d; j += gridDim.x * WG_THREADS) {
            if constexpr (sizeof(T) == 8) r[j] = gelu_f64(r[j]);
            else r[j] = (T)gelu_f32((float)r[j]);
        }
    }
}

extern "C" __global__ void __launch_bounds__(256) gelu_f16_scalar(GeluParams p) { gelu_scalar<f16>(p); }
extern "C" __global__ void __launch_bounds__(256) gelu_bf16_scalar(GeluParams p) { gelu_scalar<bf16>(p); }
extern "C" __global__ void __launch_bounds__(256) gelu_f32_scalar(GeluParams p) { gelu_scalar<float>(p); }
extern "C" __global__ void __launch_bounds__(256) gelu_f64_scalar(GeluParams p) { gelu_scalar<double>(p); }
