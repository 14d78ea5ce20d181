// Element type of the MFMA kernels.  gemm.hip and gemm_tile.hip (and attention_prefill.hip, attention_decode.hip) are compiled twice: as they stand, on f16 elements
// (modules `gemm`, `gemm_tile`), and with -DGEMM_ELEM_BF16 on bf16 elements (modules `gemm_bf16`, `gemm_tile_bf16`,
// kernel names with `_bf16` appended, so that a trace tells the two apart).  The kernels move elements as 16-bit words, so the type matters in three places only: the MFMA
// instruction, and the two conversions of the epilogue (f32 -> element rounds to nearest even in both types).
#pragma once
#include <type_traits>

#include "device_util.h"

#ifdef GEMM_ELEM_BF16
typedef bf16 elem;
#define GEMM_KERNEL(name) name##_bf16
#else
typedef f16 elem;
#define GEMM_KERNEL(name) name
#endif
typedef elem elem8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

union PackE {
    u32x4 u;
    elem8 h;
    elem e[8];
};

__device__ __forceinline__ float e2f(elem v) { return (float)v; }
__device__ __forceinline__ elem f2e(float v) { return (elem)v; }

// 16 x 16 (x 32 deep) and 32 x 32 (x 16 deep) products with f32 accumulation
template <typename V>
__device__ __forceinline__ f32x4 mfma_16x16x32(V a, V b, f32x4 c) {
    if constexpr (std::is_same_v<V, f16x8>) return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
template <typename V>
__device__ __forceinline__ f32x16 mfma_32x32x16(V a, V b, f32x16 c) {
    if constexpr (std::is_same_v<V, f16x8>) return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
