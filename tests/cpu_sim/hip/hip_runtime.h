// A CPU stand-in for <hip/hip_runtime.h>, found first on the include path when a kernel source is compiled for the
// host (tests/test_cpu_sim.py): just enough of the programming model to run the library's kernels as they are
// written, work-item by work-item, under AddressSanitizer, on small problems.
//
//   * one OS thread per work-item of a workgroup, workgroups one after another (so the workgroup of a strip that
//     runs last is the one that "arrives last"); __syncthreads() is a barrier over the threads still running;
//   * what crosses lanes (MFMA, shuffles, DPP moves) is emulated per wave of 64: every lane deposits its operands,
//     the wave meets, every lane computes its share from what the others deposited;
//   * buffer loads and stores honour the resource's record count (out of range: zeros / dropped, as the hardware
//     does) and count how often that happened; every other access is an ordinary host access, which
//     AddressSanitizer watches.
// Only test infrastructure: nothing in the library includes this.
#pragma once
#include <algorithm>
#include <atomic>
#include <barrier>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)

using std::max;
using std::min;

namespace cpusim {

struct Dim3u {
    uint32_t x = 1, y = 1, z = 1;
};

constexpr int WAVE_LANES = 64;

struct WaveState {
    std::unique_ptr<std::barrier<>> meet;
    alignas(16) unsigned char slot[2][WAVE_LANES][32];  // two operands of up to 32 bytes per lane
};
struct BlockState {
    std::unique_ptr<std::barrier<>> all;
    std::vector<WaveState> waves;
};

inline BlockState *&current_block() {
    static BlockState *b = nullptr;
    return b;
}
inline std::atomic<uint64_t> &out_of_range_loads() {
    static std::atomic<uint64_t> n{0};
    return n;
}
inline std::atomic<uint64_t> &out_of_range_stores() {
    static std::atomic<uint64_t> n{0};
    return n;
}

}  // namespace cpusim

inline thread_local cpusim::Dim3u threadIdx, blockIdx;
inline cpusim::Dim3u blockDim, gridDim;

namespace cpusim {

inline uint32_t flat_thread() { return threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z); }
inline WaveState &my_wave() { return current_block()->waves[flat_thread() / WAVE_LANES]; }
inline uint32_t my_lane() { return flat_thread() % WAVE_LANES; }
inline void wave_meet() { my_wave().meet->arrive_and_wait(); }

// Runs kernel(args...) for every workgroup of the grid, one workgroup at a time.
template <class F>
void launch(Dim3u grid, Dim3u block, F kernel) {
    gridDim = grid;
    blockDim = block;
    const uint32_t threads = block.x * block.y * block.z;
    if (threads % WAVE_LANES) {
        std::fprintf(stderr, "cpusim: workgroups of whole waves only\n");
        std::abort();
    }
    for (uint32_t bz = 0; bz < grid.z; ++bz)
        for (uint32_t by = 0; by < grid.y; ++by)
            for (uint32_t bx = 0; bx < grid.x; ++bx) {
                BlockState state;
                state.all = std::make_unique<std::barrier<>>(threads);
                state.waves.resize(threads / WAVE_LANES);
                for (auto &w : state.waves) w.meet = std::make_unique<std::barrier<>>(WAVE_LANES);
                current_block() = &state;
                std::vector<std::thread> pool;
                pool.reserve(threads);
                for (uint32_t t = 0; t < threads; ++t)
                    pool.emplace_back([&, t] {
                        threadIdx = Dim3u{t % block.x, (t / block.x) % block.y, t / (block.x * block.y)};
                        blockIdx = Dim3u{bx, by, bz};
                        kernel();
                        // a work-item that has ended no longer takes part in barriers, as on the device
                        state.all->arrive_and_drop();
                        state.waves[t / WAVE_LANES].meet->arrive_and_drop();
                    });
                for (auto &th : pool) th.join();
                current_block() = nullptr;
            }
}

// value of `v` held by lane `src` of the caller's wave (every lane of the wave must call)
template <class T>
T read_lane(T v, uint32_t src) {
    static_assert(sizeof(T) <= 32, "operand too wide");
    WaveState &w = my_wave();
    std::memcpy(w.slot[0][my_lane()], &v, sizeof(T));
    wave_meet();
    T out;
    std::memcpy(&out, w.slot[0][src % WAVE_LANES], sizeof(T));
    wave_meet();
    return out;
}

}  // namespace cpusim

inline void __syncthreads() { cpusim::current_block()->all->arrive_and_wait(); }

// ---- vector types used by the builtins below
typedef uint32_t cpusim_u32x4 __attribute__((ext_vector_type(4)));
typedef float cpusim_f32x4 __attribute__((ext_vector_type(4)));
typedef float cpusim_f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 cpusim_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 cpusim_bf16x8 __attribute__((ext_vector_type(8)));

// ---- scalar helpers of the device library
inline uint32_t __float_as_uint(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
inline float __uint_as_float(uint32_t u) {
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
inline uint32_t __umulhi(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }
#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_sched_barrier(mask) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_fence(order, scope) std::atomic_thread_fence(std::memory_order_seq_cst)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_s_setprio(x) ((void)0)

// v_perm_b32: byte k of the result is byte sel[k] of the eight bytes {s1 (0..3), s0 (4..7)}; selectors 0x0c .. : 0x00 / 0xff
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

// ---- atomics
inline uint32_t atomicAdd(uint32_t *p, uint32_t v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
inline float atomicAdd(float *p, float v) {
    float old = *p, want;
    do want = old + v;
    while (!__atomic_compare_exchange(p, &old, &want, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST));
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
inline cpusim_u32x4 cpusim_buffer_load_b128(__amdgpu_buffer_rsrc_t r, uint32_t voffset, uint32_t soffset, int) {
    cpusim_u32x4 v = {0, 0, 0, 0};
    const uint64_t off = (uint64_t)voffset + soffset;
    if (off + 16 > r.records) {
        if (r.records) cpusim::out_of_range_loads()++;  // (a resource of zero records is how a kernel asks for zeros)
        return v;
    }
    std::memcpy(&v, r.base + off, 16);
    return v;
}
inline void cpusim_buffer_store_b128(cpusim_u32x4 v, __amdgpu_buffer_rsrc_t r, uint32_t voffset, uint32_t soffset, int) {
    const uint64_t off = (uint64_t)voffset + soffset;
    if (off + 16 > r.records) {
        cpusim::out_of_range_stores()++;
        return;
    }
    std::memcpy(r.base + off, &v, 16);
}
#define __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, aux) cpusim_buffer_load_b128(r, voff, soff, aux)
#define __builtin_amdgcn_raw_buffer_store_b128(v, r, voff, soff, aux) cpusim_buffer_store_b128(v, r, voff, soff, aux)

// ---- cross-lane
template <class T>
inline T __shfl_xor(T v, int mask, int = 64) {
    return cpusim::read_lane(v, cpusim::my_lane() ^ (uint32_t)mask);
}
template <class T>
inline T __shfl(T v, int src, int = 64) {
    return cpusim::read_lane(v, (uint32_t)src);
}
// DPP moves: quad permutes (ctrl < 0x100), row_mirror (0x140), row_half_mirror (0x141); full masks, bound_ctrl set
inline int cpusim_update_dpp(int, int src, int ctrl, int row_mask, int bank_mask, bool) {
    const uint32_t lane = cpusim::my_lane();
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
    return cpusim::read_lane(src, from);
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound) cpusim_update_dpp(old, src, ctrl, row_mask, bank_mask, bound)

// ---- MFMA.  v_mfma_f32_16x16x32_{f16,bf16}: D[16 x 16] = A[16 x 32] . B[32 x 16] + C.  Lane l holds A[l % 16][8 (l / 16) ..+8],
// B[8 (l / 16) ..+8][l % 16] and D[4 (l / 16) + q][l % 16], q = 0 .. 3.
template <class V>
inline cpusim_f32x4 cpusim_mfma_16x16x32(V a, V b, cpusim_f32x4 c) {
    cpusim::WaveState &w = cpusim::my_wave();
    const uint32_t lane = cpusim::my_lane();
    float af[8], bf[8];
    for (int k = 0; k < 8; ++k) af[k] = (float)a[k], bf[k] = (float)b[k];
    std::memcpy(w.slot[0][lane], af, 32);
    std::memcpy(w.slot[1][lane], bf, 32);
    cpusim::wave_meet();
    const uint32_t j = lane % 16, i0 = 4 * (lane / 16);
    for (int q = 0; q < 4; ++q) {
        float acc = c[q];
        for (uint32_t g = 0; g < 4; ++g) {
            const float *ar = reinterpret_cast<const float *>(w.slot[0][g * 16 + i0 + q]);
            const float *br = reinterpret_cast<const float *>(w.slot[1][g * 16 + j]);
            for (int k = 0; k < 8; ++k) acc += ar[k] * br[k];
        }
        c[q] = acc;
    }
    cpusim::wave_meet();
    return c;
}
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) cpusim_mfma_16x16x32<cpusim_f16x8>(a, b, c)
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) cpusim_mfma_16x16x32<cpusim_bf16x8>(a, b, c)
// v_mfma_f32_32x32x16: not emulated (the tile kernels are not run here); declared so that sources which name it compile
template <class V>
inline cpusim_f32x16 cpusim_mfma_32x32x16(V, V, cpusim_f32x16) {
    std::fprintf(stderr, "cpusim: v_mfma_f32_32x32x16 is not emulated\n");
    std::abort();
}
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) cpusim_mfma_32x32x16<cpusim_f16x8>(a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) cpusim_mfma_32x32x16<cpusim_bf16x8>(a, b, c)
