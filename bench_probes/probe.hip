// Measurement probes for bench.py (no counterpart in the reference, and no part of the operator library): what this
// machine gives a plain stream and a bare MFMA loop, so that the operators' rates can be set against ceilings measured
// in the same run rather than against nameplate figures.  Built as a small library of its own (libbenchprobe.so, one
// entry point: bench_probe); bench.py --ceilings / --floors / --granules run it.
//   probe_read / probe_read_nt : every thread pulls 16-byte vectors, four loads in flight, grid-stride
//                                (`_nt`: with the non-temporal hint the GEMM weight loads carry)
//   probe_read16 / probe_read_nt16 : the same with sixteen loads in flight
//   probe_write                : 16-byte stores, grid-stride
//   probe_copy                 : loads four vectors, then stores them (the element-wise kernels' pattern)
//   probe_strips               : the weight-streaming GEMM's access pattern and nothing else
//   probe_granules             : one workgroup per 128-column strip of a matrix, walking down its rows, each noting how
//                                long it took: which 256-byte granule classes of the address space HBM serves slower
//                                under that pattern
//   probe_mfma                 : v_mfma_f32_32x32x16_f16 back to back on 16 independent accumulators per wave, the
//                                operands generated in registers (random-looking f16 of magnitude about 0.1, or
//                                zeros): the rate the matrix pipes sustain with nothing else in the way
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

typedef _Float16 f16;
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define WAVE 64
constexpr uint32_t WG_THREADS = 256;
union Pack8 {
    u32x4 u;
    f16x8 h;
};
__device__ __forceinline__ u32x4 ld128_nt(const void *p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p)); }

struct ProbeParams {
    void *dst;
    const void *src;
    uint64_t bytes;
    uint32_t iters, seed;
};

__global__ void __launch_bounds__(256) probe_read(ProbeParams p) {
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

__global__ void __launch_bounds__(256) probe_read_nt(ProbeParams p) {
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
__global__ void __launch_bounds__(256) probe_read16(ProbeParams p) { probe_read_deep<false>(p); }
__global__ void __launch_bounds__(256) probe_read_nt16(ProbeParams p) { probe_read_deep<true>(p); }

// The weight-streaming GEMM's access pattern and nothing else: `src` is a row-major [seed rows][iters columns] f16
// matrix; workgroup (x, y) reads the 128-column strip x over the y-th of gridDim.y equal row ranges, its four waves
// taking every fourth group of 32 rows, a lane 8 rows x 16 bytes per group, three groups in flight per wave.
__global__ void __launch_bounds__(256) probe_strips(ProbeParams p) {
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

__global__ void __launch_bounds__(256) probe_write(ProbeParams p) {
    u32x4 *d = reinterpret_cast<u32x4 *>(p.dst);
    const size_t nvec = p.bytes / 16, st = (size_t)gridDim.x * WG_THREADS;
    const u32x4 v = {p.seed, p.seed, p.seed, p.seed};
    for (size_t i = (size_t)blockIdx.x * WG_THREADS + threadIdx.x; i < nvec; i += st) d[i] = v;
}

__global__ void __launch_bounds__(256) probe_copy(ProbeParams p) {
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
__global__ void __launch_bounds__(256) probe_mfma(ProbeParams p) {
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

// One workgroup per 128-column strip of a row-major f16 matrix of `seed` rows and `iters` columns: the strip is read
// top to bottom as the weight-streaming GEMM reads it (four waves, 32 rows each per trip, 8 rows x 16 bytes per lane),
// and the workgroup writes the 100 MHz clock ticks it took to dst[strip].
__global__ void __launch_bounds__(256) probe_granules(ProbeParams p) {
    const uint32_t wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, j = lane % 16, g = lane / 16;
    const uint32_t n = p.iters, rows = p.seed;
    const uint32_t col = min(blockIdx.x * 128 + 8 * j, n - 8);
    const f16 *w = reinterpret_cast<const f16 *>(p.src) + col;
    const uint64_t t0 = wall_clock64();
    u32x4 acc = {0, 0, 0, 0};
    for (uint32_t kb = 32 * wave; kb + 32 <= rows; kb += 128) {
        u32x4 v[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) v[r] = ld128_nt(w + (size_t)(kb + 8 * g + r) * n);
#pragma unroll
        for (int r = 0; r < 8; ++r) acc ^= v[r];
    }
    uint32_t *out = reinterpret_cast<uint32_t *>(p.dst);
    if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u) out[gridDim.x] = acc[2];  // keeps the loads alive
    __syncthreads();
    if (threadIdx.x == 0) out[blockIdx.x] = (uint32_t)(wall_clock64() - t0);
}

// ---------------------------------------------------------------------------------------------------- host --
static thread_local std::string g_error;

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

extern "C" __attribute__((visibility("default"))) const char *bench_probe_error() { return g_error.c_str(); }

// One launch of the named probe on the current device: 0, or 1 with the reason in bench_probe_error().
// kind = "read", "read_nt", "read16", "read_nt16", "write", "copy": `blocks` workgroups of 256 threads stream `bytes` (a
// multiple of 16) from `src` and / or into `dst` (16-byte aligned; a read-only probe writes at most 16 bytes to dst).
// kind = "strips": `src` is a row-major f16 matrix of `seed` rows and `iters` columns (a multiple of 8) inside `bytes`,
// read in 128-column strips by one workgroup per strip and per each of `blocks` equal row ranges (`seed` a multiple of
// 32 * blocks).  kind = "granules": the same matrix, one workgroup per strip, dst gets one u32 of clock ticks (10 ns) per
// strip and needs 4 * (strips + 1) bytes.  kind = "mfma": `blocks` workgroups run `iters` trips of 128
// v_mfma_f32_32x32x16_f16 per wave on operands made in registers from `seed` (0: all-zero operands) = blocks * 4 *
// iters * 128 * 32768 flop; dst needs blocks * 1024 bytes.
extern "C" __attribute__((visibility("default"))) int bench_probe(const char *kind, void *dst, const void *src, size_t bytes,
                                                                  unsigned iters, unsigned seed, unsigned blocks, void *stream) {
    auto fail = [](const std::string &why) {
        g_error = why;
        return 1;
    };
    if (!kind) return fail("null argument");
    const std::string k = kind;
    const bool reads = k == "read" || k == "read_nt" || k == "read16" || k == "read_nt16" || k == "copy", writes = k == "write" || k == "copy";
    const bool matrix = k == "strips" || k == "granules";
    if (!reads && !writes && k != "mfma" && !matrix) return fail("unknown probe: " + k);
    if ((reads && !src) || !dst || blocks == 0) return fail("probe: null buffer or empty grid");
    if ((reads || writes) && (bytes % 16 != 0 || !aligned16(dst) || (reads && !aligned16(src))))
        return fail("probe: buffers in whole 16-byte vectors");
    const ProbeParams p{dst, src, (uint64_t)bytes, iters, seed};
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(blocks), block(256);
    if (matrix) {
        if (!src || iters < 8 || iters % 8 != 0 || seed % (32 * blocks) != 0 || (size_t)iters * seed * 2 > bytes || !aligned16(src))
            return fail("probe " + k + ": [seed][iters] f16 inside `bytes`, rows in whole groups of 32 per range");
        if (k == "granules" && blocks != 1) return fail("probe granules: one row range");
        grid = k == "strips" ? dim3((iters + 127) / 128, blocks) : dim3((iters + 127) / 128);
    }
    if (k == "read") hipLaunchKernelGGL(probe_read, grid, block, 0, s, p);
    else if (k == "read_nt") hipLaunchKernelGGL(probe_read_nt, grid, block, 0, s, p);
    else if (k == "read16") hipLaunchKernelGGL(probe_read16, grid, block, 0, s, p);
    else if (k == "read_nt16") hipLaunchKernelGGL(probe_read_nt16, grid, block, 0, s, p);
    else if (k == "write") hipLaunchKernelGGL(probe_write, grid, block, 0, s, p);
    else if (k == "copy") hipLaunchKernelGGL(probe_copy, grid, block, 0, s, p);
    else if (k == "strips") hipLaunchKernelGGL(probe_strips, grid, block, 0, s, p);
    else if (k == "granules") hipLaunchKernelGGL(probe_granules, grid, block, 0, s, p);
    else hipLaunchKernelGGL(probe_mfma, grid, block, 0, s, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(std::string("launch of probe ") + k + ": " + hipGetErrorString(e));
    return 0;
}
