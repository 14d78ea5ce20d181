// Device-side helpers for the gfx950 kernels: 128-bit vector types, wave64 and
// workgroup reductions, f16 conversions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "params.h"

typedef _Float16 f16;
typedef __bf16 bf16;  // conversions from and to float are the hardware's (to bf16: nearest even)
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define WAVE 64

// Waits until every vector-memory operation the wave has issued is acknowledged (stores included).  Written out where a
// kernel publishes data to other workgroups: a workgroup-scope fence compiles to no such wait on gfx950.  (A build of
// the kernels for the host, which the CPU tests run work-item by work-item, has no such instruction: a fence there.)
#ifdef OPHIP_CPU_SIM
#define OPHIP_WAIT_VMEM() std::atomic_thread_fence(std::memory_order_seq_cst)
#else
#define OPHIP_WAIT_VMEM() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")
#endif

// Where a wave reads from LDS what other lanes of the same wave have just stored there, with no workgroup barrier in
// between: nothing on the GPU, where the LDS operations of a wave complete in the order they were issued for all of
// its lanes; a meeting point of the wave's lanes in the build of the kernels for the host, which runs the lanes one
// after another.
#ifdef OPHIP_CPU_SIM
#define OPHIP_WAVE_LOCKSTEP() cpusim_wave_sync()
#else
#define OPHIP_WAVE_LOCKSTEP() ((void)0)
#endif

// Threads per workgroup of every kernel that strides by its workgroup size (the host launches them with exactly this
// many).  A constant rather than blockDim.x: inside a __device__ function the compiler fetches blockDim.x with a vector
// load from the implicit arguments and waits for it before the first address is known, which costs a streaming kernel of
// many small workgroups a fifth of its rate (gelu at [16384, 11008]: 145 against 114 us).
constexpr uint32_t WG_THREADS = 256;

__device__ __forceinline__ u32x4 ld128(const void *p) { return *reinterpret_cast<const u32x4 *>(p); }
__device__ __forceinline__ void st128(void *p, u32x4 v) { *reinterpret_cast<u32x4 *>(p) = v; }
// the same with the non-temporal hint: for output that the kernel writes once and that is too large to be found in a
// cache by whoever reads it next
__device__ __forceinline__ void st128_nt(void *p, u32x4 v) { __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p)); }
// Streaming load for data touched once per launch (GEMM weights): the non-temporal hint keeps
// such lines from displacing reusable ones in L2 and the Infinity Cache, and raises read-only
// streaming bandwidth (5.8 -> 6.6 TB/s measured on 1 GiB).
__device__ __forceinline__ u32x4 ld128_nt(const void *p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p)); }

__device__ __forceinline__ float h2f(f16 h) { return (float)h; }
// round-to-nearest-even, subnormals kept (v_cvt_f16_f32)
__device__ __forceinline__ f16 f2h(float f) { return (f16)f; }

union Pack8 {
    u32x4 u;
    f16x8 h;
    f16 e[8];
};
union Pack4f {
    u32x4 u;
    f32x4 f;
    float e[4];
};
// 16 bytes of T (f16, bf16: 8 elements; f32: 4)
template <typename T>
union PackOf {
    u32x4 u;
    T e[16 / sizeof(T)];
};

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// The same reductions with the first four steps as DPP operand modifiers (lane ^ 1, lane ^ 2, mirror inside 8, mirror
// inside 16: no LDS crossbar, no extra instruction) and only the last two as cross-lane reads: a third of the
// instructions, for kernels whose reductions are a visible share of their work.  Every lane ends with the result.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_HALF_MIRROR = 0x141, DPP_MIRROR = 0x140;
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v += dpp_move<DPP_XOR1>(v);
    v += dpp_move<DPP_XOR2>(v);
    v += dpp_move<DPP_HALF_MIRROR>(v);
    v += dpp_move<DPP_MIRROR>(v);
    v += __shfl_xor(v, 16, WAVE);
    v += __shfl_xor(v, 32, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max_dpp(float v) {
    v = fmaxf(v, dpp_move<DPP_XOR1>(v));
    v = fmaxf(v, dpp_move<DPP_XOR2>(v));
    v = fmaxf(v, dpp_move<DPP_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_move<DPP_MIRROR>(v));
    v = fmaxf(v, __shfl_xor(v, 16, WAVE));
    v = fmaxf(v, __shfl_xor(v, 32, WAVE));
    return v;
}

// Sum over a group of G consecutive threads (G = 64 * 2^k, G <= blockDim).
// Groups wider than a wave combine their per-wave partials through `smem`
// (one float per wave of the block) in a fixed order; all threads must call.
template <int G>
__device__ __forceinline__ float group_sum(float v, float *smem) {
    v = wave_sum_dpp(v);
    if constexpr (G > WAVE) {
        const int wave = threadIdx.x / WAVE;
        __syncthreads();
        if ((threadIdx.x & (WAVE - 1)) == 0) smem[wave] = v;
        __syncthreads();
        const int first = (threadIdx.x / G) * (G / WAVE);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < G / WAVE; ++i) s += smem[first + i];
        v = s;
    }
    return v;
}
template <int G>
__device__ __forceinline__ float group_max(float v, float *smem) {
    v = wave_max_dpp(v);
    if constexpr (G > WAVE) {
        const int wave = threadIdx.x / WAVE;
        __syncthreads();
        if ((threadIdx.x & (WAVE - 1)) == 0) smem[wave] = v;
        __syncthreads();
        const int first = (threadIdx.x / G) * (G / WAVE);
        float s = smem[first];
#pragma unroll
        for (int i = 1; i < G / WAVE; ++i) s = fmaxf(s, smem[first + i]);
        v = s;
    }
    return v;
}

// exp(x) through the hardware base-2 exponential (about 1 ulp plus |x| * 2^-24 from the
// scaling by log2(e)): two instructions instead of libm's range reduction.  The
// streaming kernels whose result is rounded to f16 use it; at 8 TB/s the accurate
// expf alone would exceed their per-element instruction budget.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDivU32 &d) {
    uint32_t t = __umulhi(d.m, n);
    return (t + ((n - t) >> d.s1)) >> d.s2;
}
