// 16x16x32 MFMA on packed 16-bit operands and the chunking constants shared by the few-rows GEMM
// kernels (a weight fragment of 16 rows x 32 K elements is the A operand, 16 rows of x the B operand).
#pragma once
#include <hip/hip_runtime.h>

#include "ksa_cvt.h"


template <typename T>
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma16<KsaBf16>(u32x4 a, u32x4 b, f32x4 c) {
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma16<KsaF16>(u32x4 a, u32x4 b, f32x4 c) {
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                  0, 0, 0);
}

constexpr int kChunkSteps = 16;                 // K steps (of 32) per staged chunk of x
constexpr int kChunkK = 32 * kChunkSteps;       // 512 elements of K
constexpr int kRowB = (kChunkK + 8) * 2;        // padded LDS row of x in bytes (conflict-free b128 reads)
