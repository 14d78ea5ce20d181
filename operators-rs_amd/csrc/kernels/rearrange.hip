// rearrange (N-d strided copy) for gfx950.
//
// The host normalises the two layouts into `count` units of `unit` contiguous
// bytes plus per-dimension index/dst/src strides.  A unit is cut into chunks of
// B bytes (the largest of 16/8/4/2/1 that divides the unit and keeps every
// address aligned); chunk g belongs to unit g / chunks_per_unit.  Consecutive
// threads take consecutive chunks, and since dimensions are ordered by
// descending destination stride, consecutive chunks land on ascending
// destination addresses: the stores coalesce into full lines while the loads
// gather `unit`-byte runs.  Divisions by the launch-time constants use
// multiply-high, so the index decode costs a few integer ops per chunk.
// Byte-exact for any element type, negative strides and zero source strides.
#include "device_util.h"

template <int B>
struct Chunk;
template <>
struct Chunk<16> { typedef u32x4 T; };
template <>
struct Chunk<8> { typedef u32x2 T; };
template <>
struct Chunk<4> { typedef uint32_t T; };
template <>
struct Chunk<2> { typedef uint16_t T; };
template <>
struct Chunk<1> { typedef uint8_t T; };

// RE_ITEMS chunks per thread, loads issued before stores: 4 for large copies; 1 for mid-size ones, which would
// otherwise leave the machine with one workgroup per CU or less (8 MB: 256 workgroups at 4 chunks per thread).
// NT: a copy larger than the caches (the host decides): what it writes is not found in them by the next reader
// anyway, and the non-temporal hint on the stores is worth 3 % on such a copy.  (A flag in the parameters does
// not do: the compiler merges the two stores of an if / else and drops the hint.)
template <int B, int RE_ITEMS, bool NT = false>
__device__ __forceinline__ void rearrange32(const RearrangeParams &p) {
    typedef typename Chunk<B>::T T;
    const uint32_t total = (uint32_t)p.total;
    T val[RE_ITEMS];
    int64_t doff[RE_ITEMS];
    bool ok[RE_ITEMS];
#pragma unroll
    for (int it = 0; it < RE_ITEMS; ++it) {
        const uint32_t g = (blockIdx.x * RE_ITEMS + it) * WG_THREADS + threadIdx.x;
        ok[it] = g < total;
        doff[it] = 0;
        if (ok[it]) {
            const uint32_t u = fastdiv(g, p.cpu_div);
            const uint32_t c = g - u * p.chunks_per_unit;
            uint32_t rem = u;
            int64_t d = (int64_t)c * B, s = (int64_t)c * B;
            for (uint32_t q = 0; q < p.ndim; ++q) {
                const uint32_t k = fastdiv(rem, p.idx_div[q]);
                rem -= k * p.idx_div[q].d;
                d += (int64_t)k * p.dst_s[q];
                s += (int64_t)k * p.src_s[q];
            }
            doff[it] = d;
            val[it] = __builtin_nontemporal_load(reinterpret_cast<const T *>(reinterpret_cast<const char *>(p.src) + s));
        }
    }
#pragma unroll
    for (int it = 0; it < RE_ITEMS; ++it)
        if (ok[it]) {
            if constexpr (NT) __builtin_nontemporal_store(val[it], reinterpret_cast<T *>(reinterpret_cast<char *>(p.dst) + doff[it]));
            else *reinterpret_cast<T *>(reinterpret_cast<char *>(p.dst) + doff[it]) = val[it];
        }
}

// 64-bit indices: more than 2^32 chunks or an index stride beyond 32 bits.
template <int B>
__device__ __forceinline__ void rearrange64(const RearrangeParams &p) {
    typedef typename Chunk<B>::T T;
    for (uint64_t g = (uint64_t)blockIdx.x * WG_THREADS + threadIdx.x; g < p.total;
         g += (uint64_t)gridDim.x * WG_THREADS) {
        const uint64_t u = g / p.chunks_per_unit;
        const uint64_t c = g % p.chunks_per_unit;
        uint64_t rem = u;
        int64_t d = (int64_t)c * B, s = (int64_t)c * B;
        for (uint32_t q = 0; q < p.ndim; ++q) {
            const uint64_t k = rem / p.idx[q];
            rem %= p.idx[q];
            d += (int64_t)k * p.dst_s[q];
            s += (int64_t)k * p.src_s[q];
        }
        *reinterpret_cast<T *>(reinterpret_cast<char *>(p.dst) + d) =
            *reinterpret_cast<const T *>(reinterpret_cast<const char *>(p.src) + s);
    }
}

#define REARRANGE(B)                                                                             \
    extern "C" __global__ void __launch_bounds__(256) rearrange_b##B(RearrangeParams p) {       \
        rearrange32<B, 4>(p);                                                                    \
    }                                                                                            \
    extern "C" __global__ void __launch_bounds__(256) rearrange_nt_b##B(RearrangeParams p) {    \
        rearrange32<B, 4, true>(p);                                                              \
    }                                                                                            \
    extern "C" __global__ void __launch_bounds__(256) rearrange1_b##B(RearrangeParams p) {      \
        rearrange32<B, 1>(p);                                                                    \
    }                                                                                            \
    extern "C" __global__ void __launch_bounds__(256) rearrange64_b##B(RearrangeParams p) {     \
        rearrange64<B>(p);                                                                       \
    }

REARRANGE(16)
REARRANGE(8)
REARRANGE(4)
REARRANGE(2)
REARRANGE(1)

// memset on a stream, as a kernel: it is recorded into a launch graph like any other launch.
// A transposing copy of small units: element-wise, one side of it would move 2 .. 8 bytes per lane at a stride
// ([8192, 8192] f16: 0.23 TB/s).  A tile of 64 x 64 units is read in rows of the source's contiguous dimension,
// turned in LDS (rows padded by one unit: no bank conflicts either way) and written in rows of the destination's.
template <typename U>
__device__ __forceinline__ void rearrange_transpose(const TransposeParams &p) {
    __shared__ U tile[64][65];
    uint32_t id = blockIdx.x;
    const uint32_t outer = fastdiv(id, p.tiles_div);
    id -= outer * p.tiles_div.d;
    const uint32_t ta = fastdiv(id, p.tb_div), tb = id - ta * p.tb_div.d;
    int64_t d0 = 0, s0 = 0;
    uint32_t rem = outer;
    for (uint32_t q = 0; q < p.nouter; ++q) {
        const uint32_t k = fastdiv(rem, p.outer_div[q]);
        rem -= k * p.outer_div[q].d;
        d0 += (int64_t)k * p.outer_dst[q];
        s0 += (int64_t)k * p.outer_src[q];
    }
    const uint32_t a0 = ta * 64, b0 = tb * 64, tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    const char *src = reinterpret_cast<const char *>(p.src) + s0;
    char *dst = reinterpret_cast<char *>(p.dst) + d0;
    // source: rows along B (contiguous), one row per a
#pragma unroll 4
    for (uint32_t r = ty; r < 64; r += 4) {
        const uint32_t a = a0 + r, b = b0 + tx;
        if (a < p.len_a && b < p.len_b) tile[r][tx] = *reinterpret_cast<const U *>(src + (int64_t)a * p.src_a + (size_t)b * sizeof(U));
    }
    __syncthreads();
    // destination: rows along A (contiguous), one row per b
#pragma unroll 4
    for (uint32_t r = ty; r < 64; r += 4) {
        const uint32_t b = b0 + r, a = a0 + tx;
        if (a < p.len_a && b < p.len_b) *reinterpret_cast<U *>(dst + (int64_t)b * p.dst_b + (size_t)a * sizeof(U)) = tile[tx][r];
    }
}
extern "C" __global__ void __launch_bounds__(256) rearrange_transpose_b2(TransposeParams p) { rearrange_transpose<uint16_t>(p); }
extern "C" __global__ void __launch_bounds__(256) rearrange_transpose_b4(TransposeParams p) { rearrange_transpose<uint32_t>(p); }
extern "C" __global__ void __launch_bounds__(256) rearrange_transpose_b8(TransposeParams p) { rearrange_transpose<uint64_t>(p); }

extern "C" __global__ void __launch_bounds__(256) fill_bytes(FillBytesParams p) {
    const uint64_t gid = (uint64_t)blockIdx.x * 256 + threadIdx.x, stride = (uint64_t)gridDim.x * 256;
    char *dst = reinterpret_cast<char *>(p.dst);
    if (gid < p.head) dst[gid] = (char)p.value;
    char *body = dst + p.head;
    const u32x4 v = u32x4{p.value, p.value, p.value, p.value};
    for (uint64_t i = gid; i < p.body; i += stride) st128(body + 16 * i, v);
    if (gid < p.tail) body[16 * p.body + gid] = (char)p.value;
}
