// add for gfx950:  c = a + b, element-wise over N-d strided tensors (broadcast = stride 0 in a or b).
//
// The host merges the three layouts into at most 8 dimensions (add/args.rs:42-167) and counts
// items in the innermost one: single elements, or 16-byte vectors when that dimension is
// contiguous in all three tensors.  Item g is decoded into per-dimension indices with
// multiply-high divisions; dimensions are ordered by descending c stride, so consecutive
// threads write ascending addresses.  f16 (and bf16) sums are formed in f32 and rounded once, as
// half's `f16 + f16` does.
#include <type_traits>

#include "device_util.h"

struct AddOffsets {
    int64_t c, a, b;
};

__device__ __forceinline__ AddOffsets add_decode(const AddParams &p, uint32_t g) {
    AddOffsets o{0, 0, 0};
    uint32_t rem = g;
    for (uint32_t q = 0; q < p.ndim; ++q) {
        const uint32_t k = fastdiv(rem, p.idx_div[q]);
        rem -= k * p.idx_div[q].d;
        o.c += (int64_t)k * p.c_s[q];
        o.a += (int64_t)k * p.a_s[q];
        o.b += (int64_t)k * p.b_s[q];
    }
    return o;
}

// NT: a sum larger than the caches (the host decides): stores with the non-temporal hint.  (Separate builds: a flag
// in the parameters would make the compiler merge the two stores of an if / else and drop the hint.)
template <typename T, bool NT>
__device__ __forceinline__ void add_h_vec_impl(const AddParams &p) {  // T: f16 or bf16
    for (uint32_t g = blockIdx.x * WG_THREADS + threadIdx.x; g < p.total; g += gridDim.x * WG_THREADS) {
        const AddOffsets o = add_decode(p, g);
        PackOf<T> a, b, c;
        a.u = ld128_nt(reinterpret_cast<const char *>(p.a) + o.a);
        b.u = ld128_nt(reinterpret_cast<const char *>(p.b) + o.b);
#pragma unroll
        for (int i = 0; i < 8; ++i) c.e[i] = (T)((float)a.e[i] + (float)b.e[i]);
        if constexpr (NT) st128_nt(reinterpret_cast<char *>(p.c) + o.c, c.u);
        else st128(reinterpret_cast<char *>(p.c) + o.c, c.u);
    }
}
extern "C" __global__ void __launch_bounds__(256) add_f16_vec(AddParams p) { add_h_vec_impl<f16, false>(p); }
extern "C" __global__ void __launch_bounds__(256) add_f16_vec_nt(AddParams p) { add_h_vec_impl<f16, true>(p); }
// bf16: the reference's CUDA backend adds any named type (add/cuda/mod.rs:105-123); its CPU backend has no bf16
extern "C" __global__ void __launch_bounds__(256) add_bf16_vec(AddParams p) { add_h_vec_impl<bf16, false>(p); }
extern "C" __global__ void __launch_bounds__(256) add_bf16_vec_nt(AddParams p) { add_h_vec_impl<bf16, true>(p); }

template <bool NT>
__device__ __forceinline__ void add_f32_vec_impl(const AddParams &p) {
    for (uint32_t g = blockIdx.x * WG_THREADS + threadIdx.x; g < p.total; g += gridDim.x * WG_THREADS) {
        const AddOffsets o = add_decode(p, g);
        Pack4f a, b, c;
        a.u = ld128_nt(reinterpret_cast<const char *>(p.a) + o.a);
        b.u = ld128_nt(reinterpret_cast<const char *>(p.b) + o.b);
        c.f = a.f + b.f;
        if constexpr (NT) st128_nt(reinterpret_cast<char *>(p.c) + o.c, c.u);
        else st128(reinterpret_cast<char *>(p.c) + o.c, c.u);
    }
}
extern "C" __global__ void __launch_bounds__(256) add_f32_vec(AddParams p) { add_f32_vec_impl<false>(p); }
extern "C" __global__ void __launch_bounds__(256) add_f32_vec_nt(AddParams p) { add_f32_vec_impl<true>(p); }

template <typename T>
__device__ __forceinline__ void add_scalar(const AddParams &p) {
    for (uint32_t g = blockIdx.x * WG_THREADS + threadIdx.x; g < p.total; g += gridDim.x * WG_THREADS) {
        const AddOffsets o = add_decode(p, g);
        using Calc = std::conditional_t<sizeof(T) == 8, double, float>;  // f64 data adds in f64
        const Calc a = (Calc)*reinterpret_cast<const T *>(reinterpret_cast<const char *>(p.a) + o.a);
        const Calc b = (Calc)*reinterpret_cast<const T *>(reinterpret_cast<const char *>(p.b) + o.b);
        *reinterpret_cast<T *>(reinterpret_cast<char *>(p.c) + o.c) = (T)(a + b);
    }
}

extern "C" __global__ void __launch_bounds__(256) add_f16_scalar(AddParams p) { add_scalar<f16>(p); }
extern "C" __global__ void __launch_bounds__(256) add_bf16_scalar(AddParams p) { add_scalar<bf16>(p); }
extern "C" __global__ void __launch_bounds__(256) add_f32_scalar(AddParams p) { add_scalar<float>(p); }
extern "C" __global__ void __launch_bounds__(256) add_f64_scalar(AddParams p) { add_scalar<double>(p); }

// Integer and bool elements: the reference's CUDA backend compiles `c[idx] = a[idx] + b[idx]` for any named type
// (add/cuda/mod.rs:105-123 with handle/cuda/mod.rs:188-210), which for integers is the sum modulo 2^bits (signed and
// unsigned alike in two's complement: one kernel per width) and for bool "either is set".  Its CPU backend has floats only.
template <typename U, bool IS_BOOL = false>
__device__ __forceinline__ void add_int_scalar(const AddParams &p) {
    for (uint32_t g = blockIdx.x * WG_THREADS + threadIdx.x; g < p.total; g += gridDim.x * WG_THREADS) {
        const AddOffsets o = add_decode(p, g);
        const U a = *reinterpret_cast<const U *>(reinterpret_cast<const char *>(p.a) + o.a);
        const U b = *reinterpret_cast<const U *>(reinterpret_cast<const char *>(p.b) + o.b);
        *reinterpret_cast<U *>(reinterpret_cast<char *>(p.c) + o.c) = IS_BOOL ? (U)((a | b) != 0) : (U)(a + b);
    }
}
extern "C" __global__ void __launch_bounds__(256) add_i8_scalar(AddParams p) { add_int_scalar<uint8_t>(p); }
extern "C" __global__ void __launch_bounds__(256) add_i16_scalar(AddParams p) { add_int_scalar<uint16_t>(p); }
extern "C" __global__ void __launch_bounds__(256) add_i32_scalar(AddParams p) { add_int_scalar<uint32_t>(p); }
extern "C" __global__ void __launch_bounds__(256) add_i64_scalar(AddParams p) { add_int_scalar<uint64_t>(p); }
extern "C" __global__ void __launch_bounds__(256) add_bool_scalar(AddParams p) { add_int_scalar<uint8_t, true>(p); }
