// 16-bit float <-> fp32 conversions with explicit rounding points, shared by the element-wise
// kernels that reproduce the rounding of the reference's 16-bit tensor ops.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ksa_tile.h"

template <typename T>
struct KsaCvt;
template <>
struct KsaCvt<KsaBf16> {
    static __device__ __forceinline__ float up(uint16_t u) {
        return __builtin_bit_cast(float, (uint32_t)u << 16);
    }
    static __device__ __forceinline__ uint16_t down(float f) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }
    // two values rounded into one word (low, high) and back
    static __device__ __forceinline__ uint32_t down2(float lo, float hi) { return KsaOps<KsaBf16>::pack2(lo, hi); }
    static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
    // a.lo * b.lo + a.hi * b.hi + c on packed pairs (the products of two 16-bit values are exact in fp32)
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
    }
    // Two / four such products with a zero addend.  The compiler only has the accumulating
    // two-operand form for a zero addend and clears its register first; the three-operand form
    // with an inline zero is written out here.  The wait states at the end cover a result read
    // by the next vector instruction (3 wait states, DOT -> VALU): the compiler's hazard handling
    // does not look inside an assembly statement.
    static __device__ __forceinline__ void dot2z_x2(uint32_t a0, uint32_t b0, uint32_t a1, uint32_t b1,
                                                    float& r0, float& r1) {
        asm("v_dot2_f32_bf16 %0, %2, %3, 0\n\tv_dot2_f32_bf16 %1, %4, %5, 0\n\ts_nop 2"
            : "=&v"(r0), "=&v"(r1)
            : "v"(a0), "v"(b0), "v"(a1), "v"(b1));
    }
    static __device__ __forceinline__ void dot2z_x4(uint32_t a0, uint32_t b0, uint32_t a1, uint32_t b1,
                                                    uint32_t a2, uint32_t b2, uint32_t a3, uint32_t b3,
                                                    float& r0, float& r1, float& r2, float& r3) {
        asm("v_dot2_f32_bf16 %0, %4, %5, 0\n\tv_dot2_f32_bf16 %1, %6, %7, 0\n\t"
            "v_dot2_f32_bf16 %2, %8, %9, 0\n\tv_dot2_f32_bf16 %3, %10, %11, 0\n\ts_nop 2"
            : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
            : "v"(a0), "v"(b0), "v"(a1), "v"(b1), "v"(a2), "v"(b2), "v"(a3), "v"(b3));
    }
    static constexpr uint32_t kOnes = 0x3f803f80u;  // (1.0, 1.0)
};
template <>
struct KsaCvt<KsaF16> {
    // Conversion instructions written out: with plain _Float16 casts the compiler may keep
    // excess precision across a down/up pair, which would drop the rounding points.
    static __device__ __forceinline__ float up(uint16_t u) {
        float f;
        asm("v_cvt_f32_f16 %0, %1" : "=v"(f) : "v"((uint32_t)u));
        return f;
    }
    static __device__ __forceinline__ uint16_t down(float f) {
        uint32_t h;
        // the wait states cover a packed-dot-product result as the input: the compiler's hazard
        // handling does not look inside an assembly statement (3 wait states, DOT -> VALU)
        asm("s_nop 2\n\tv_cvt_f16_f32 %0, %1" : "=v"(h) : "v"(f));
        return (uint16_t)h;
    }
    static __device__ __forceinline__ uint32_t down2(float lo, float hi) {
        return (uint32_t)down(lo) | ((uint32_t)down(hi) << 16);
    }
    static __device__ __forceinline__ float lo(uint32_t w) { return up((uint16_t)(w & 0xffffu)); }
    static __device__ __forceinline__ float hi(uint32_t w) { return up((uint16_t)(w >> 16)); }
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
    }
    static __device__ __forceinline__ void dot2z_x2(uint32_t a0, uint32_t b0, uint32_t a1, uint32_t b1,
                                                    float& r0, float& r1) {
        r0 = dot2(a0, b0, 0.f), r1 = dot2(a1, b1, 0.f);
    }
    static __device__ __forceinline__ void dot2z_x4(uint32_t a0, uint32_t b0, uint32_t a1, uint32_t b1,
                                                    uint32_t a2, uint32_t b2, uint32_t a3, uint32_t b3,
                                                    float& r0, float& r1, float& r2, float& r3) {
        r0 = dot2(a0, b0, 0.f), r1 = dot2(a1, b1, 0.f), r2 = dot2(a2, b2, 0.f), r3 = dot2(a3, b3, 0.f);
    }
    static constexpr uint32_t kOnes = 0x3c003c00u;
};

typedef float f32x4 __attribute__((ext_vector_type(4)));

// rows of one slice of the K-split partial sums of a product with `rows` rows: whole 16-row blocks
__host__ __device__ __forceinline__ int ksa_partial_rows(int rows) { return (rows + 15) / 16 * 16; }

// eight consecutive columns of a row of x = the rounded sum of fp32 slices [ksplit][prows][width]
// (the K-split partial sums of ksa_gemm_rows, prows = ksa_partial_rows(rows of x)), added in split
// order like its own reduction
template <typename T>
__device__ __forceinline__ u32x4 ksa_sum_partials8(const float* part, int ksplit, int prows, int width, int row, int col) {
    using C = KsaCvt<T>;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int sp0 = 0; sp0 < ksplit; sp0 += 8) {  // eight slices requested together
        f32x4 lo[8], hi[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int sp = min(sp0 + u, ksplit - 1);
            const float* src = part + ((int64_t)sp * prows + row) * width + col;
            lo[u] = *reinterpret_cast<const f32x4*>(src);
            hi[u] = *reinterpret_cast<const f32x4*>(src + 4);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (sp0 + u < ksplit) {
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[i] += lo[u][i], acc[4 + i] += hi[u][i];
            }
        }
    }
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = C::down2(acc[2 * i], acc[2 * i + 1]);
    return r;
}
