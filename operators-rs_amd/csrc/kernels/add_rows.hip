// add_rows for gfx950:  dst[b, m, :] += src[idx[b, m], :]   (add_rows/common_cpu/mod.rs:131-147)
//
// blockIdx.y walks the b * m destination rows, blockIdx.x the row in 16-byte vectors (or single
// elements when the row is not 16-byte friendly).  The row index is read once per workgroup.
// An index >= k (the reference asserts) leaves the destination row unchanged.
#include <type_traits>

#include "device_util.h"

__device__ __forceinline__ bool add_rows_locate(const AddRowsParams &p, uint32_t bm, char *&dst, const char *&src) {
    const uint32_t b = bm / p.m, m = bm % p.m;
    const char *ip = reinterpret_cast<const char *>(p.idx) + (int64_t)b * p.bsi + (int64_t)m * p.msi;
    const uint64_t idx = p.idx_is_u64 ? *reinterpret_cast<const uint64_t *>(ip) : *reinterpret_cast<const uint32_t *>(ip);
    if (idx >= p.k) return false;
    dst = reinterpret_cast<char *>(p.dst) + (int64_t)b * p.bsd + (int64_t)m * p.msd;
    src = reinterpret_cast<const char *>(p.src) + (int64_t)idx * p.kss;
    return true;
}

template <typename T>
__device__ __forceinline__ void add_rows_h_vec(const AddRowsParams &p) {  // T: f16 or bf16
    const uint32_t nvec = p.n / 8;
    for (uint32_t bm = blockIdx.y; bm < p.batch * p.m; bm += gridDim.y) {
        char *dst;
        const char *src;
        if (!add_rows_locate(p, bm, dst, src)) continue;
        for (uint32_t v = blockIdx.x * WG_THREADS + threadIdx.x; v < nvec; v += gridDim.x * WG_THREADS) {
            PackOf<T> d, s;
            d.u = ld128_nt(dst + (size_t)v * 16);
            s.u = ld128(src + (size_t)v * 16);
#pragma unroll
            for (int i = 0; i < 8; ++i) d.e[i] = (T)((float)d.e[i] + (float)s.e[i]);
            st128(dst + (size_t)v * 16, d.u);
        }
    }
}
extern "C" __global__ void __launch_bounds__(256) add_rows_f16_vec(AddRowsParams p) { add_rows_h_vec<f16>(p); }
// bf16: the reference's CUDA backend compiles add_rows for any named type (add_rows/cuda/mod.rs:135-163); its CPU
// backend has no bf16
extern "C" __global__ void __launch_bounds__(256) add_rows_bf16_vec(AddRowsParams p) { add_rows_h_vec<bf16>(p); }

// element-wise; nsd / nss are the element strides of dst and src rows in bytes
template <typename T>
__device__ __forceinline__ void add_rows_scalar(const AddRowsParams &p, int64_t nsd, int64_t nss) {
    for (uint32_t bm = blockIdx.y; bm < p.batch * p.m; bm += gridDim.y) {
        char *dst;
        const char *src;
        if (!add_rows_locate(p, bm, dst, src)) continue;
        for (uint32_t j = blockIdx.x * WG_THREADS + threadIdx.x; j < p.n; j += gridDim.x * WG_THREADS) {
            T *d = reinterpret_cast<T *>(dst + (int64_t)j * nsd);
            const T *s = reinterpret_cast<const T *>(src + (int64_t)j * nss);
            using Calc = std::conditional_t<sizeof(T) == 8, double, float>;  // f64 data adds in f64
            *d = (T)((Calc)*d + (Calc)*s);
        }
    }
}

struct AddRowsScalarParams {
    AddRowsParams p;
    int64_t nsd, nss;
};
extern "C" __global__ void __launch_bounds__(256) add_rows_f16_scalar(AddRowsScalarParams q) {
    add_rows_scalar<f16>(q.p, q.nsd, q.nss);
}
extern "C" __global__ void __launch_bounds__(256) add_rows_bf16_scalar(AddRowsScalarParams q) {
    add_rows_scalar<bf16>(q.p, q.nsd, q.nss);
}
extern "C" __global__ void __launch_bounds__(256) add_rows_f32_scalar(AddRowsScalarParams q) {
    add_rows_scalar<float>(q.p, q.nsd, q.nss);
}
extern "C" __global__ void __launch_bounds__(256) add_rows_f64_scalar(AddRowsScalarParams q) {
    add_rows_scalar<double>(q.p, q.nsd, q.nss);
}

// Integer and bool rows, as the reference's CUDA backend would compile them (add_rows/cuda/mod.rs:135-163): sums modulo
// 2^bits, one kernel per width; bool: either is set.
template <typename U, bool IS_BOOL = false>
__device__ __forceinline__ void add_rows_int(const AddRowsParams &p, int64_t nsd, int64_t nss) {
    for (uint32_t bm = blockIdx.y; bm < p.batch * p.m; bm += gridDim.y) {
        char *dst;
        const char *src;
        if (!add_rows_locate(p, bm, dst, src)) continue;
        for (uint32_t j = blockIdx.x * WG_THREADS + threadIdx.x; j < p.n; j += gridDim.x * WG_THREADS) {
            U *d = reinterpret_cast<U *>(dst + (int64_t)j * nsd);
            const U s = *reinterpret_cast<const U *>(src + (int64_t)j * nss);
            *d = IS_BOOL ? (U)((*d | s) != 0) : (U)(*d + s);
        }
    }
}
extern "C" __global__ void __launch_bounds__(256) add_rows_i8_scalar(AddRowsScalarParams q) { add_rows_int<uint8_t>(q.p, q.nsd, q.nss); }
extern "C" __global__ void __launch_bounds__(256) add_rows_i16_scalar(AddRowsScalarParams q) { add_rows_int<uint16_t>(q.p, q.nsd, q.nss); }
extern "C" __global__ void __launch_bounds__(256) add_rows_i32_scalar(AddRowsScalarParams q) { add_rows_int<uint32_t>(q.p, q.nsd, q.nss); }
extern "C" __global__ void __launch_bounds__(256) add_rows_i64_scalar(AddRowsScalarParams q) { add_rows_int<uint64_t>(q.p, q.nsd, q.nss); }
extern "C" __global__ void __launch_bounds__(256) add_rows_bool_scalar(AddRowsScalarParams q) { add_rows_int<uint8_t, true>(q.p, q.nsd, q.nss); }
