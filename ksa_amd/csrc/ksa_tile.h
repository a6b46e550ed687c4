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
// its 8 B-operand elements e = 4*a + r, so V^T is stored in LDS with key position
//   pos(kv) = 16*(kv/16) + 8*h + 4*a + r      for kv = 16*(kv/16) + 8*a + 4*h + r
// and the A operand of lane (d, h) is the 16 contiguous bytes at V^T[d][16*ks + 8*h].
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
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        bf16x2 v;
        v[0] = (__bf16)lo;
        v[1] = (__bf16)hi;
        return __builtin_bit_cast(uint32_t, v);
    }
};

template <>
struct KsaOps<KsaF16> {
    static __device__ __forceinline__ floatx16 mfma(u32x4 a, u32x4 b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f16x2 v;
        v[0] = (_Float16)lo;
        v[1] = (_Float16)hi;
        return __builtin_bit_cast(uint32_t, v);
    }
};

// low halves / high halves of two dwords -> one dword (lo16 from b, hi16 from a)
__device__ __forceinline__ uint32_t ksa_pack_lo(uint32_t a, uint32_t b) {
    return __builtin_amdgcn_perm(a, b, 0x05040100u);
}
__device__ __forceinline__ uint32_t ksa_pack_hi(uint32_t a, uint32_t b) {
    return __builtin_amdgcn_perm(a, b, 0x07060302u);
}

// LDS position of key (4*kv4 .. 4*kv4+3) inside a V^T row
__device__ __forceinline__ int ksa_vt_pos(int kv4) {
    return 16 * (kv4 >> 2) + 8 * (kv4 & 1) + 4 * ((kv4 >> 1) & 1);
}

// Four rows x eight columns held as four 16-byte registers -> eight 8-byte
// columns written to V^T rows d0 .. d0+7 at key position pos.
template <int VROW>
__device__ __forceinline__ void ksa_store_vt(uint16_t* vt, int d0, int pos, const u32x4 (&r)[4]) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        u32x2 even, odd;
        even[0] = ksa_pack_lo(r[1][w], r[0][w]);
        even[1] = ksa_pack_lo(r[3][w], r[2][w]);
        odd[0] = ksa_pack_hi(r[1][w], r[0][w]);
        odd[1] = ksa_pack_hi(r[3][w], r[2][w]);
        *reinterpret_cast<u32x2*>(vt + (d0 + 2 * w) * VROW + pos) = even;
        *reinterpret_cast<u32x2*>(vt + (d0 + 2 * w + 1) * VROW + pos) = odd;
    }
}

__device__ __forceinline__ float ksa_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float ksa_xor32(float x) { return __shfl_xor(x, 32); }

// fence that orders this wave's LDS writes before its later LDS reads (and the
// reverse) without involving the other waves of the workgroup
__device__ __forceinline__ void ksa_wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
