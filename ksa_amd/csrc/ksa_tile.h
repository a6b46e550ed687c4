// Register / LDS tile conventions shared by the prefill and decode kernels (gfx950, wave64).
//
// Both kernels compute S^T = K Q^T and O^T = V^T P^T with v_mfma_f32_32x32x16_{bf16,f16}:
//   * A operand (32 x 16): lane l holds row (l % 32), contraction elements 8*(l/32) .. +8
//   * B operand (16 x 32): lane l holds col (l % 32), contraction elements 8*(l/32) .. +8
//   * C/D (32 x 32 fp32, 16 regs): lane l holds col (l % 32), reg i holds row
//         8*(i/4) + 4*(l/32) + (i % 4)
// Putting the query on the column side makes one lane own one query row's scores
// (16 per 32 keys), so the soft-max row reductions are in-register plus a single
// exchange between lane l and lane l^32.
//
// For the second product the contraction index is the key position.  The C layout
// above hands lane (q, h) the keys {16*ks + 8*a + 4*h + r : a<2, r<4} of k-step ks as
// its 8 B-operand elements e = 4*a + r.  V stays row-major in LDS ([key][dim], like K) and
// the matching A operand of lane (d, h) -- V[those 8 keys][d] -- is fetched with two
// ds_read_b64_tr_b16: within each group of 16 lanes, lane t supplies the address of 4
// consecutive dims of key (K0 + t/4) at dim D0 + 4*(t%4) and receives V[K0 + j][D0 + t],
// j = 0..3, i.e. a 4-key x 16-dim block transposed on the way out of LDS.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

struct KsaBf16 {};
struct KsaF16 {};

template <typename T>
struct KsaOps;

template <>
struct KsaOps<KsaBf16> {
    static __device__ __forceinline__ floatx16 mfma(u32x4 a, u32x4 b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    // Register-class pinned forms for kernels that run one wave per SIMD with both register
    // files: accumulators of the second product (`acc`) and the resident B operand of the
    // first (`b_acc`) live in AGPRs, scores and LDS-fed operands in VGPRs.  The compiler does
    // not see an MFMA in these statements, so the caller keeps MFMA results away from vector
    // instructions for the required wait states (ksa_mfma_settle), and each statement carries
    // the one wait state the hardware needs between a vector instruction and an MFMA (without
    // it the first MFMA after vector work computed garbage on gfx950).
    static __device__ __forceinline__ floatx16 mfma_v0(u32x4 a, u32x4 b_acc) {
        floatx16 d;
        asm volatile("s_nop 0\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b_acc));
        return d;
    }
    static __device__ __forceinline__ void mfma_v(floatx16& c, u32x4 a, u32x4 b_acc) {
        asm volatile("s_nop 0\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b_acc));
    }
    static __device__ __forceinline__ void mfma_a(floatx16& acc, u32x4 a, u32x4 b) {
        asm volatile("s_nop 0\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        bf16x2 v;
        v[0] = (__bf16)lo;
        v[1] = (__bf16)hi;
        return __builtin_bit_cast(uint32_t, v);
    }
    // acc + lo + hi of a packed pair (as rounded to 16 bit)
    static __device__ __forceinline__ float sum2(uint32_t pk, float acc) {
        bf16x2 one;
        one[0] = (__bf16)1.0f;
        one[1] = (__bf16)1.0f;
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pk), one, acc, false);
    }
};

template <>
struct KsaOps<KsaF16> {
    static __device__ __forceinline__ floatx16 mfma(u32x4 a, u32x4 b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ floatx16 mfma_v0(u32x4 a, u32x4 b_acc) {
        floatx16 d;
        asm volatile("s_nop 0\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b_acc));
        return d;
    }
    static __device__ __forceinline__ void mfma_v(floatx16& c, u32x4 a, u32x4 b_acc) {
        asm volatile("s_nop 0\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b_acc));
    }
    static __device__ __forceinline__ void mfma_a(floatx16& acc, u32x4 a, u32x4 b) {
        asm volatile("s_nop 0\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f16x2 v;
        v[0] = (_Float16)lo;
        v[1] = (_Float16)hi;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float sum2(uint32_t pk, float acc) {
        f16x2 one;
        one[0] = (_Float16)1.0f;
        one[1] = (_Float16)1.0f;
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pk), one, acc, false);
    }
};

typedef short ksa_short4 __attribute__((ext_vector_type(4)));

// A operand of O^T += V^T P^T for k-step ks and 32-dim block db, from row-major V in LDS
// (row stride VROW elements).  lq = lane % 32, lh = lane / 32.
template <int VROW>
__device__ __forceinline__ u32x4 ksa_read_vt_frag(const uint16_t* vs, int ks, int db, int lq, int lh) {
    const int t = lq & 15;
    const uint16_t* p = vs + (16 * ks + 4 * lh + (t >> 2)) * VROW + 32 * db + (lq & 16) + 4 * (t & 3);
    typedef __attribute__((address_space(3))) ksa_short4* lds_ptr;
    const ksa_short4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
    const ksa_short4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 8 * VROW));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo);
    const u32x2 h2 = __builtin_bit_cast(u32x2, hi);
    u32x4 r;
    r[0] = l2[0];
    r[1] = l2[1];
    r[2] = h2[0];
    r[3] = h2[1];
    return r;
}

// Wait states between an MFMA written as inline assembly and the first vector or memory
// instruction that touches its result (the hardware does not interlock these; 8-pass MFMAs
// need 11, this leaves a wide margin).
__device__ __forceinline__ void ksa_mfma_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

__device__ __forceinline__ float ksa_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float ksa_xor32(float x) { return __shfl_xor(x, 32); }

// Reductions over the lane pair (l, l ^ 32) with v_permlane32_swap: after the swap one
// result holds the lower half's value and the other the upper half's value in every lane.
__device__ __forceinline__ float ksa_pair_max(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float ksa_pair_sum(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

// fence that orders this wave's LDS writes before its later LDS reads (and the
// reverse) without involving the other waves of the workgroup
__device__ __forceinline__ void ksa_wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
