// A CPU stand-in for <hip/hip_runtime.h>, found first on the include path when a kernel source of the library is
// compiled for the host (tests only): just enough of the device side of the programming model to run the kernels as
// they are written, work-item by work-item (cpusim_core.h says how), on small problems.
//
//   * what crosses lanes (MFMA, shuffles, DPP moves, ballots, the transposing LDS read) is emulated per wave of 64;
//   * buffer loads and stores honour the resource's record count (out of range: zeros / dropped, as the hardware
//     does) and count how often that happened; every other access is an ordinary host access: the test's allocator
//     (guard pages) or AddressSanitizer watches it;
//   * LDS is thread-local static storage (all work-items of a workgroup are fibers of one OS thread).
// Nothing in the library includes this.
#pragma once
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../cpusim_core.h"

#ifndef __global__  // (the build defines it to a marker when it lists a source's kernels)
#define __global__
#endif
#define __device__
#define __host__
#define __forceinline__ inline
#define __noinline__ __attribute__((noinline))
// block scope: implies static; file scope (`extern __shared__ T name[]`, the launch's dynamic LDS): declares an array that
// the generated translation unit of the module defines, at the size of a whole CU's LDS
#define __shared__ thread_local
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))

using std::max;
using std::min;

#define threadIdx (cpusim::worker().cur->tid)
#define blockIdx (cpusim::worker().block_idx)
#define blockDim (cpusim::worker().block_dim)
#define gridDim (cpusim::worker().grid_dim)

inline void __syncthreads() { cpusim::barrier(); }
// the lanes of the caller's wave meet (the kernels mark the places where they rely on a wave running in lockstep)
inline void cpusim_wave_sync(int line = __builtin_LINE()) { cpusim::wave_exchange((uint32_t)line, nullptr, 0); }

// ---- vector types
struct float2 {
    float x, y;
};
struct double2 {
    double x, y;
};
typedef uint32_t cpusim_u32x4 __attribute__((ext_vector_type(4)));
typedef float cpusim_f32x4 __attribute__((ext_vector_type(4)));
typedef float cpusim_f32x16 __attribute__((ext_vector_type(16)));
typedef short cpusim_s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 cpusim_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 cpusim_bf16x8 __attribute__((ext_vector_type(8)));

// ---- scalar helpers of the device library
inline uint32_t __float_as_uint(float f) { return __builtin_bit_cast(uint32_t, f); }
inline float __uint_as_float(uint32_t u) { return __builtin_bit_cast(float, u); }
inline double __longlong_as_double(long long v) { return __builtin_bit_cast(double, v); }
inline long long __double_as_longlong(double v) { return __builtin_bit_cast(long long, v); }
inline uint32_t __umulhi(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }
inline int __ffsll(long long v) { return __builtin_ffsll(v); }
inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
inline double rsqrt(double x) { return 1.0 / sqrt(x); }
#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_sched_barrier(mask) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_fence(order, scope) std::atomic_thread_fence(std::memory_order_seq_cst)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_s_setprio(x) ((void)0)

// v_perm_b32: byte k of the result is byte sel[k] of the eight bytes {s1 (0..3), s0 (4..7)}; selector 0x0c: 0x00, 0x0d and up: 0xff
inline uint32_t cpusim_perm(uint32_t s0, uint32_t s1, uint32_t sel) {
    const uint64_t both = ((uint64_t)s0 << 32) | s1;
    uint32_t out = 0;
    for (int k = 0; k < 4; ++k) {
        const uint32_t s = (sel >> (8 * k)) & 0xff;
        uint32_t byte;
        if (s < 8) byte = (uint32_t)(both >> (8 * s)) & 0xff;
        else if (s == 0x0c) byte = 0;
        else if (s >= 0x0d) byte = 0xff;
        else {
            std::fprintf(stderr, "cpusim: v_perm selector %#x is not emulated\n", s);
            std::abort();
        }
        out |= byte << (8 * k);
    }
    return out;
}
#define __builtin_amdgcn_perm(s0, s1, sel) cpusim_perm(s0, s1, sel)

// ---- atomics (on memory any workgroup may touch: workgroups run one after another here, but keep them atomic)
inline uint32_t atomicAdd(uint32_t *p, uint32_t v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
inline int atomicAdd(int *p, int v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
inline unsigned long long atomicAdd(unsigned long long *p, unsigned long long v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
inline float atomicAdd(float *p, float v) {
    float old = *p, want;
    do want = old + v;
    while (!__atomic_compare_exchange(p, &old, &want, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST));
    return old;
}
inline uint32_t atomicMax(uint32_t *p, uint32_t v) {
    uint32_t old = *p;
    while (old < v && !__atomic_compare_exchange_n(p, &old, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST)) {
    }
    return old;
}
inline uint32_t atomicMin(uint32_t *p, uint32_t v) {
    uint32_t old = *p;
    while (old > v && !__atomic_compare_exchange_n(p, &old, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST)) {
    }
    return old;
}

// ---- buffer resources: base, records (bytes); loads past the records read zeros, stores are dropped
struct __amdgpu_buffer_rsrc_t {
    char *base;
    uint32_t records;
};
inline __amdgpu_buffer_rsrc_t cpusim_make_rsrc(const void *base, int stride, uint32_t records, uint32_t) {
    if (stride != 0) {
        std::fprintf(stderr, "cpusim: only raw buffers (stride 0) are emulated\n");
        std::abort();
    }
    return {const_cast<char *>(static_cast<const char *>(base)), records};
}
#define __builtin_amdgcn_make_buffer_rsrc(base, stride, records, flags) cpusim_make_rsrc(base, stride, records, flags)
inline int cpusim_cache_policy(int aux) { return (aux & 16) ? 2 : (aux & 2) ? 1 : 0; }  // sc1, nt, neither
inline cpusim_u32x4 cpusim_buffer_load_b128(__amdgpu_buffer_rsrc_t r, uint32_t voffset, uint32_t soffset, int aux) {
    cpusim_u32x4 v = {0, 0, 0, 0};
    const uint64_t off = (uint64_t)voffset + soffset;
    if (off + 16 > r.records) {
        if (r.records) cpusim::worker().out_of_range_loads++;  // (a resource of zero records is how a kernel asks for zeros)
        return v;
    }
    std::memcpy(&v, r.base + off, 16);
    cpusim::worker().buffer_load_bytes[cpusim_cache_policy(aux)] += 16;
    return v;
}
inline void cpusim_buffer_store_b128(cpusim_u32x4 v, __amdgpu_buffer_rsrc_t r, uint32_t voffset, uint32_t soffset, int aux) {
    const uint64_t off = (uint64_t)voffset + soffset;
    if (off + 16 > r.records) {
        cpusim::worker().out_of_range_stores++;
        return;
    }
    std::memcpy(r.base + off, &v, 16);
    cpusim::worker().buffer_store_bytes[cpusim_cache_policy(aux)] += 16;
}
#define __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, aux) cpusim_buffer_load_b128(r, voff, soff, aux)
#define __builtin_amdgcn_raw_buffer_store_b128(v, r, voff, soff, aux) cpusim_buffer_store_b128(v, r, voff, soff, aux)

// ---- cross-lane
// value of `v` held by lane `src` of the caller's wave
template <class T>
inline T cpusim_read_lane(int line, T v, uint32_t src) {
    static_assert(sizeof(T) <= cpusim::SLOT_BYTES, "operand too wide");
    const cpusim::WaveView w = cpusim::wave_exchange((uint32_t)line, &v, sizeof(T));
    T out;
    std::memcpy(&out, w.a[src % cpusim::WAVE_LANES], sizeof(T));
    return out;
}
// (the last parameter of each: the line of the call, by which the scheduler checks that the lanes that meet are at the
// same operation)
template <class T>
inline T __shfl_xor(T v, int mask, int = 64, int line = __builtin_LINE()) {
    return cpusim_read_lane(line, v, cpusim::lane_id() ^ (uint32_t)mask);
}
template <class T>
inline T __shfl(T v, int src, int = 64, int line = __builtin_LINE()) {
    return cpusim_read_lane(line, v, (uint32_t)src);
}
template <class T>
inline T __shfl_up(T v, unsigned delta, int = 64, int line = __builtin_LINE()) {
    const uint32_t lane = cpusim::lane_id();
    return cpusim_read_lane(line, v, lane >= delta ? lane - delta : lane);
}
template <class T>
inline T __shfl_down(T v, unsigned delta, int = 64, int line = __builtin_LINE()) {
    const uint32_t lane = cpusim::lane_id();
    return cpusim_read_lane(line, v, lane + delta < cpusim::WAVE_LANES ? lane + delta : lane);
}
// A lane that is not at the ballot (masked out, or returned) counts as 0: a slot it left from an earlier operation
// must not be read, so every lane deposits a marker that carries the wave's operation number.
inline uint64_t __ballot(int pred, int line = __builtin_LINE()) {
    cpusim::Worker &wk = cpusim::worker();
    const uint32_t gen = wk.waves[wk.cur->flat / cpusim::WAVE_LANES].generation;
    const uint32_t mine[2] = {gen, pred ? 1u : 0u};
    const cpusim::WaveView w = cpusim::wave_exchange((uint32_t)line, mine, sizeof(mine));
    uint64_t out = 0;
    for (uint32_t l = 0; l < cpusim::WAVE_LANES; ++l) {
        uint32_t theirs[2];
        std::memcpy(theirs, w.a[l], sizeof(theirs));
        if (theirs[0] == gen && theirs[1]) out |= 1ull << l;
    }
    return out;
}
#define __builtin_amdgcn_ballot_w64(p) __ballot(p, __LINE__)
// DPP moves: quad permutes (ctrl < 0x100), row_mirror (0x140), row_half_mirror (0x141); full masks, bound_ctrl set
inline int cpusim_update_dpp(int line, int, int src, int ctrl, int row_mask, int bank_mask, bool) {
    const uint32_t lane = cpusim::lane_id();
    uint32_t from;
    if (ctrl < 0x100) from = (lane & ~3u) | ((uint32_t)(ctrl >> (2 * (lane & 3))) & 3u);
    else if (ctrl == 0x140) from = (lane & ~15u) | (15u - (lane & 15u));
    else if (ctrl == 0x141) from = (lane & ~7u) | (7u - (lane & 7u));
    else {
        std::fprintf(stderr, "cpusim: DPP control %#x is not emulated\n", ctrl);
        std::abort();
    }
    if (row_mask != 0xf || bank_mask != 0xf) {
        std::fprintf(stderr, "cpusim: partial DPP masks are not emulated\n");
        std::abort();
    }
    return cpusim_read_lane(line, src, from);
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound) cpusim_update_dpp(__LINE__, old, src, ctrl, row_mask, bank_mask, bound)

// ds_read_b64_tr_b16: the 16 lanes of a group each address four 16-bit elements; seen as a [4 rows][16 columns] matrix
// (lane 4 r + m of the group addresses row r, columns 4 m .. 4 m + 3), lane c of the group receives column c, rows 0 .. 3.
inline cpusim_s16x4 cpusim_ds_read_tr16_b64(int line, const void *p) {
    unsigned char mine[8];
    std::memcpy(mine, p, 8);
    const cpusim::WaveView w = cpusim::wave_exchange((uint32_t)line, mine, 8);
    const uint32_t lane = cpusim::lane_id(), group = lane & ~15u, c = lane & 15u;
    cpusim_s16x4 out;
    for (uint32_t r = 0; r < 4; ++r) {
        short e;
        std::memcpy(&e, w.a[group + 4 * r + c / 4] + 2 * (c % 4), 2);
        out[r] = e;
    }
    return out;
}
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) cpusim_ds_read_tr16_b64(__LINE__, (const void *)(p))

// ---- MFMA.  v_mfma_f32_16x16x32_{f16,bf16}: D[16 x 16] = A[16 x 32] . B[32 x 16] + C.  Lane l holds A[l % 16][8 (l / 16) ..+8],
// B[8 (l / 16) ..+8][l % 16] and D[4 (l / 16) + q][l % 16], q = 0 .. 3.
template <class V>
inline cpusim_f32x4 cpusim_mfma_16x16x32(int line, V a, V b, cpusim_f32x4 c) {
    float af[8], bf[8];
    for (int k = 0; k < 8; ++k) af[k] = (float)a[k], bf[k] = (float)b[k];
    const cpusim::WaveView w = cpusim::wave_exchange((uint32_t)line, af, 32, bf, 32);
    const uint32_t lane = cpusim::lane_id(), j = lane % 16, i0 = 4 * (lane / 16);
    for (int q = 0; q < 4; ++q) {
        float acc = c[q];
        for (uint32_t g = 0; g < 4; ++g) {
            const float *ar = reinterpret_cast<const float *>(w.a[g * 16 + i0 + q]);
            const float *br = reinterpret_cast<const float *>(w.b[g * 16 + j]);
            for (int k = 0; k < 8; ++k) acc += ar[k] * br[k];
        }
        c[q] = acc;
    }
    return c;
}
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) cpusim_mfma_16x16x32<cpusim_f16x8>(__LINE__, a, b, c)
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) cpusim_mfma_16x16x32<cpusim_bf16x8>(__LINE__, a, b, c)
// v_mfma_f32_32x32x16_{f16,bf16}: D[32 x 32] = A[32 x 16] . B[16 x 32] + C.  Lane l holds A[l % 32][8 (l / 32) ..+8],
// B[8 (l / 32) ..+8][l % 32] and D[8 (r / 4) + 4 (l / 32) + r % 4][l % 32], r = 0 .. 15.
template <class V>
inline cpusim_f32x16 cpusim_mfma_32x32x16(int line, V a, V b, cpusim_f32x16 c) {
    float af[8], bf[8];
    for (int k = 0; k < 8; ++k) af[k] = (float)a[k], bf[k] = (float)b[k];
    const cpusim::WaveView w = cpusim::wave_exchange((uint32_t)line, af, 32, bf, 32);
    const uint32_t lane = cpusim::lane_id(), j = lane % 32, h = lane / 32;
    for (int r = 0; r < 16; ++r) {
        const uint32_t i = 8 * (r / 4) + 4 * h + r % 4;
        float acc = c[r];
        for (uint32_t g = 0; g < 2; ++g) {
            const float *ar = reinterpret_cast<const float *>(w.a[g * 32 + i]);
            const float *br = reinterpret_cast<const float *>(w.b[g * 32 + j]);
            for (int k = 0; k < 8; ++k) acc += ar[k] * br[k];
        }
        c[r] = acc;
    }
    return c;
}
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) cpusim_mfma_32x32x16<cpusim_f16x8>(__LINE__, a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) cpusim_mfma_32x32x16<cpusim_bf16x8>(__LINE__, a, b, c)

// ---- registration of a module's kernels (the generated file of each module lists them after including the source)
#define CPUSIM_REGISTER(module_name, kernel)                                                                       \
    static const bool cpusim_registered_##kernel = [] {                                                            \
        using P = std::remove_cv_t<std::remove_reference_t<cpusim::KernelOf<decltype(&kernel)>::Params>>;          \
        cpusim::registry()[#kernel] = cpusim::KernelInfo{[](const void *params) { kernel(*static_cast<const P *>(params)); }, sizeof(P), module_name}; \
        return true;                                                                                               \
    }();
