// 16x16x32 MFMA on packed 16-bit operands and the chunking constants shared by the few-rows GEMM
// kernels (a weight fragment of 16 rows x 32 K elements is the A operand, 16 rows of x the B operand).
#pragma once
#include <hip/hip_runtime.h>

#include "ksa_api_internal.h"
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

// Where a lane finds its 16 bytes of a weight fragment (16 rows of w x 32 elements of K, the A operand of
// one MFMA; lane = (row r of the 16, quarter kq of the 32)).  Row-major w [N, K]: row n starts n * rs
// elements in, the fragment of K step s lies 32 s elements further - 64 bytes of each of 16 rows that are
// K elements apart.  Streaming layout (rs == kWTiled, made by ksa_tile_weights): the 1 KB of a fragment is
// contiguous and the K / 32 fragments of 16 rows follow one another, [ceil(N / 16)][K / 32][16][32], so a
// wave reads its rows' share of the matrix as one sequential run (rows past N are zeros).
struct KsaWeightLane {
    const uint16_t* p;  // this lane's piece of K step 0
    int step;           // elements from one K step to the next
};
__device__ __forceinline__ KsaWeightLane ksa_weight_lane(const uint16_t* w, int64_t rs, int K, int64_t row0, int r,
                                                         int kq, int64_t nrows) {
    KsaWeightLane l;
    if (rs == kWTiled) {  // (a wave whose 16 rows all lie past the matrix reads the last tile: nothing of it is stored)
        const int64_t last = (nrows - 1) / 16;
        l.p = w + (row0 / 16 < last ? row0 / 16 : last) * (int64_t)(K / 32) * 512 + r * 32 + 8 * kq;
        l.step = 512;
    } else {
        const int64_t row = row0 + r < nrows ? row0 + r : nrows - 1;
        l.p = w + row * rs + 8 * kq;
        l.step = 32;
    }
    return l;
}
