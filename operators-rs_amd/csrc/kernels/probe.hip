// Measurement probes (no counterpart in the reference): what this machine gives a plain stream and a bare
// MFMA loop, so that the operators' rates can be set against ceilings measured in the same run rather than
// against nameplate figures.  Launched by ophip_probe; bench.py --ceilings runs them.
//   probe_read / probe_read_nt : every thread pulls 16-byte vectors, four loads in flight, grid-stride
//                                (`_nt`: with the non-temporal hint the GEMM weight loads carry)
//   probe_read16 / probe_read_nt16 : the same with sixteen loads in flight
//   probe_write                : 16-byte stores, grid-stride
//   probe_copy                 : loads four vectors, then stores them (the element-wise kernels' pattern)
//   probe_mfma                 : v_mfma_f32_32x32x16_f16 back to back on 16 independent accumulators per wave, the
//                                operands generated in registers (random-looking f16 of magnitude about 0.1, or
//                                zeros): the rate the matrix pipes sustain with nothing else in the way
#include "device_util.h"

extern "C" __global__ void __launch_bounds__(256) probe_read(ProbeParams p) {
    const u32x4 *w = reinterpret_cast<const u32x4 *>(p.src);
    const size_t nvec = p.bytes / 16, st = (size_t)gridDim.x * WG_THREADS;
    size_t i = (size_t)blockIdx.x * WG_THREADS + threadIdx.x;
    u32x4 acc = {0, 0, 0, 0};
    for (; i + 3 * st < nvec; i += 4 * st) {
        const u32x4 a = w[i], b = w[i + st], c = w[i + 2 * st], d = w[i + 3 * st];
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < nvec; i += st) acc ^= w[i];
    if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u) *reinterpret_cast<u32x4 *>(p.dst) = acc;  // keeps the loads alive
}

extern "C" __global__ void __launch_bounds__(256) probe_read_nt(ProbeParams p) {
    const u32x4 *w = reinterpret_cast<const u32x4 *>(p.src);
    const size_t nvec = p.bytes / 16, st = (size_t)gridDim.x * WG_THREADS;
    size_t i = (size_t)blockIdx.x * WG_THREADS + threadIdx.x;
    u32x4 acc = {0, 0, 0, 0};
    for (; i + 3 * st < nvec; i += 4 * st) {
        const u32x4 a = ld128_nt(w + i), b = ld128_nt(w + i + st), c = ld128_nt(w + i + 2 * st), d = ld128_nt(w + i + 3 * st);
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < nvec; i += st) acc ^= ld128_nt(w + i);
    if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u) *reinterpret_cast<u32x4 *>(p.dst) = acc;
}

// The same read with 16 vectors in flight per thread (64 KB per workgroup, the depth of the weight-streaming GEMM's
// register ring): what one CU can pull when the depth of its queue is not the limit.
template <bool NT>
__device__ __forceinline__ void probe_read_deep(const ProbeParams &p) {
    const u32x4 *w = reinterpret_cast<const u32x4 *>(p.src);
    const size_t nvec = p.bytes / 16, st = (size_t)gridDim.x * WG_THREADS;
    size_t i = (size_t)blockIdx.x * WG_THREADS + threadIdx.x;
    u32x4 acc = {0, 0, 0, 0};
    for (; i + 15 * st < nvec; i += 16 * st) {
        u32x4 v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = NT ? ld128_nt(w + i + u * st) : w[i + u * st];
#pragma unroll
        for (int u = 0; u < 16; ++u) acc ^= v[u];
    }
    for (; i < nvec; i += st) acc ^= NT ? ld128_nt(w + i) : w[i];
    if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u) *reinterpret_cast<u32x4 *>(p.dst) = acc;
}
extern "C" __global__ void __launch_bounds__(256) probe_read16(ProbeParams p) { probe_read_deep<false>(p); }
extern "C" __global__ void __launch_bounds__(256) probe_read_nt16(ProbeParams p) { probe_read_deep<true>(p); }

// The weight-streaming GEMM's access pattern and nothing else: `src` is a row-major [seed rows][iters columns] f16
// matrix; workgroup (x, y) reads the 128-column strip x over the y-th of gridDim.y equal row ranges, its four waves
// taking every fourth group of 32 rows, a lane 8 rows x 16 bytes per group, three groups in flight per wave.
extern "C" __global__ void __launch_bounds__(256) probe_strips(ProbeParams p) {
    const uint32_t wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, j = lane % 16, g = lane / 16;
    const uint32_t n = p.iters, rows = p.seed;
    const uint32_t per = rows / gridDim.y, kbeg = blockIdx.y * per, kend = kbeg + per;
    const uint32_t col = min(blockIdx.x * 128 + 8 * j, n - 8);
    const f16 *w = reinterpret_cast<const f16 *>(p.src) + col;
    u32x4 acc = {0, 0, 0, 0};
    uint32_t kb = kbeg + 32 * wave;
    for (; kb + 2 * 128 + 32 <= kend; kb += 3 * 128) {
        u32x4 v[3][8];
#pragma unroll
        for (int u = 0; u < 3; ++u)
#pragma unroll
            for (int r = 0; r < 8; ++r) v[u][r] = ld128_nt(w + (size_t)(kb + 128 * u + 8 * g + r) * n);
#pragma unroll
        for (int u = 0; u < 3; ++u)
#pragma unroll
            for (int r = 0; r < 8; ++r) acc ^= v[u][r];
    }
    for (; kb + 32 <= kend; kb += 128)
#pragma unroll
        for (int r = 0; r < 8; ++r) acc ^= ld128_nt(w + (size_t)(kb + 8 * g + r) * n);
    if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u) *reinterpret_cast<u32x4 *>(p.dst) = acc;
}

extern "C" __global__ void __launch_bounds__(256) probe_write(ProbeParams p) {
    u32x4 *d = reinterpret_cast<u32x4 *>(p.dst);
    const size_t nvec = p.bytes / 16, st = (size_t)gridDim.x * WG_THREADS;
    const u32x4 v = {p.seed, p.seed, p.seed, p.seed};
    for (size_t i = (size_t)blockIdx.x * WG_THREADS + threadIdx.x; i < nvec; i += st) d[i] = v;
}

extern "C" __global__ void __launch_bounds__(256) probe_copy(ProbeParams p) {
    const u32x4 *w = reinterpret_cast<const u32x4 *>(p.src);
    u32x4 *d = reinterpret_cast<u32x4 *>(p.dst);
    const size_t nvec = p.bytes / 16, st = (size_t)gridDim.x * WG_THREADS;
    size_t i = (size_t)blockIdx.x * WG_THREADS + threadIdx.x;
    for (; i + 3 * st < nvec; i += 4 * st) {
        const u32x4 a = w[i], b = w[i + st], c = w[i + 2 * st], e = w[i + 3 * st];
        d[i] = a, d[i + st] = b, d[i + 2 * st] = c, d[i + 3 * st] = e;
    }
    for (; i < nvec; i += st) d[i] = w[i];
}

typedef float f32x16 __attribute__((ext_vector_type(16)));

// 128 MFMA of 32 x 32 x 16 per trip and wave: 2 * 32 * 32 * 16 * 128 flop
extern "C" __global__ void __launch_bounds__(256) probe_mfma(ProbeParams p) {
    const uint32_t t = threadIdx.x + blockIdx.x * 256;
    auto rnd = [&](uint32_t x) {  // two f16 of magnitude 0.06 .. 0.12, either sign (zeros when the seed is 0)
        x *= 0x9E3779B1u;
        x ^= x >> 15;
        x *= 0x85EBCA77u;
        x ^= x >> 13;
        return p.seed ? (0x2c002c00u | (x & 0x83ff83ffu)) : 0u;
    };
    Pack8 a[8], b[8];
    for (int i = 0; i < 8; ++i)
        for (int j = 0; j < 4; ++j) {
            a[i].u[j] = rnd(p.seed + t * 64 + i * 4 + j);
            b[i].u[j] = rnd(p.seed + 7777 + t * 64 + i * 4 + j);
        }
    f32x16 acc[4][4];
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (uint32_t it = 0; it < p.iters; ++it) {
#pragma unroll
        for (int kk = 0; kk < 8; ++kk)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i + 4 * (kk & 1)].h, b[j + 4 * (kk & 1)].h, acc[i][j], 0, 0, 0);
        if (p.seed) {  // the operands change from trip to trip, as a real kernel's do
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a[i].u[it & 3] ^= 0x00010001u << (it & 7);
                b[i].u[(it + 1) & 3] ^= 0x00010001u << ((it + 3) & 7);
            }
        }
    }
    float s = 0.f;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int e = 0; e < 16; ++e) s += acc[i][j][e];
    if (s == 12345.f) reinterpret_cast<float *>(p.dst)[t] = s;
}
