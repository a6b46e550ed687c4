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
    static constexpr uint32_t kOnes = 0x3c003c00u;
};

