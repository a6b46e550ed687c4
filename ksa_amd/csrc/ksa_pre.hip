// Pre-attention step of a Qwen3 / KSA attention layer in one pass over HBM (gfx950):
// per-head RMSNorm of the query and key projections, rotary position embedding, and the
// write of q, k, v in the layout the attention kernels (or the KV cache) want.
//
// Replaces, at the reference's call site
//   examples/pretrain/hf_template/modeling_qwen3sa.py:660-666
//     q = q_norm(q_proj(x).view(.., H, D)).transpose(1, 2)      (Qwen3RMSNorm :64-79)
//     k = k_norm(k_proj(x).view(.., Hkv, D)).transpose(1, 2)
//     v = v_proj(x).view(.., Hkv, D).transpose(1, 2)
//     q, k = apply_rotary_pos_emb(q, k, cos, sin)                (:523-554, rotate_half form)
// plus the .transpose(1, 2).contiguous() copies in front of the prefill kernel, i.e. about
// ten element-wise passes, and keeps their rounding points: the normalised value is rounded
// to the 16-bit type, multiplied by the 16-bit weight and rounded, and the rotation is
// round(round(z cos) + round(rot(z) sin)) -- what the reference's 16-bit tensor ops produce.
//
// A head row (D 16-bit elements) is held by D/8 consecutive lanes, 8 elements each, so a wave
// instruction moves 1 KB of consecutive head rows of one token.  The RMS reduction and the
// rotate_half partner (element j +- D/2) are lane exchanges inside that group of lanes.
#include <hip/hip_runtime.h>

#include "ksa_api_internal.h"
#include "ksa_tile.h"

namespace {

struct PreParams {
    const uint16_t* src[3];   // q, k, v projections  [batch, S, H, D] by strides
    uint16_t* dst[3];         // q, k, v outputs
    const uint16_t* w[2];     // q_norm, k_norm weights [D]
    const uint16_t* cos;      // [batch or 1, S, D]
    const uint16_t* sin;
    int64_t s_bs[3], s_rs[3], s_hs[3];
    int64_t d_bs[3], d_rs[3], d_hs[3];
    int64_t c_bs, c_rs;
    int batch, S, Hq, Hkv;
    float eps;
};

template <typename T>
struct PreCvt;
template <>
struct PreCvt<KsaBf16> {
    static __device__ __forceinline__ float up(uint16_t u) {
        return __builtin_bit_cast(float, (uint32_t)u << 16);
    }
    static __device__ __forceinline__ uint16_t down(float f) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }
};
template <>
struct PreCvt<KsaF16> {
    static __device__ __forceinline__ float up(uint16_t u) {
        return (float)__builtin_bit_cast(_Float16, u);
    }
    static __device__ __forceinline__ uint16_t down(float f) {
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    }
};

template <typename T, int D>
__global__ __launch_bounds__(256) void ksa_pre_attention_kernel(const PreParams p) {
    using C = PreCvt<T>;
    constexpr int LPR = D / 8;          // lanes per head row
    constexpr int RPW = 64 / LPR;       // head rows per wave instruction
    const int lane = threadIdx.x & 63;
    const int sub = lane / LPR;         // which of the wave's rows
    const int t = lane % LPR;           // 16-byte chunk inside the row
    const int H_all = p.Hq + 2 * p.Hkv;
    const int G = (H_all + RPW - 1) / RPW;
    const int64_t items = (int64_t)p.batch * p.S * G;
    const int64_t wave0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;

    for (int64_t it = wave0; it < items; it += nwaves) {
        const int g = (int)(it % G);
        const int64_t tok = it / G;
        const int s = (int)(tok % p.S);
        const int b = (int)(tok / p.S);
        const int hh = g * RPW + sub;
        if (hh >= H_all) continue;  // the whole lane group has nothing to do (no exchange partner outside it)
        const int which = hh < p.Hq ? 0 : (hh < p.Hq + p.Hkv ? 1 : 2);
        const int h = which == 0 ? hh : (which == 1 ? hh - p.Hq : hh - p.Hq - p.Hkv);
        const uint16_t* sp = p.src[which] + b * p.s_bs[which] + (int64_t)s * p.s_rs[which] + h * p.s_hs[which] + 8 * t;
        uint16_t* dp = p.dst[which] + b * p.d_bs[which] + (int64_t)s * p.d_rs[which] + h * p.d_hs[which] + 8 * t;
        const u32x4 raw = *reinterpret_cast<const u32x4*>(sp);
        if (which == 2) {  // v: layout change only
            *reinterpret_cast<u32x4*>(dp) = raw;
            continue;
        }
        float x[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[2 * i] = C::up((uint16_t)(raw[i] & 0xffffu));
            x[2 * i + 1] = C::up((uint16_t)(raw[i] >> 16));
        }
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ss = fmaf(x[i], x[i], ss);
#pragma unroll
        for (int m = 1; m < LPR; m <<= 1) ss += __shfl_xor(ss, m);
        const float inv = rsqrtf(ss * (1.0f / D) + p.eps);
        const u32x4 wraw = *reinterpret_cast<const u32x4*>(p.w[which] + 8 * t);
        const uint16_t* cb = p.cos + b * p.c_bs + (int64_t)s * p.c_rs + 8 * t;
        const uint16_t* sb = p.sin + b * p.c_bs + (int64_t)s * p.c_rs + 8 * t;
        const u32x4 craw = *reinterpret_cast<const u32x4*>(cb);
        const u32x4 sraw = *reinterpret_cast<const u32x4*>(sb);
        // z = round(w * round(x * inv)), packed again for the exchange
        u32x4 zp;
        float z[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float w0 = C::up((uint16_t)(wraw[i] & 0xffffu)), w1 = C::up((uint16_t)(wraw[i] >> 16));
            const uint16_t y0 = C::down(x[2 * i] * inv), y1 = C::down(x[2 * i + 1] * inv);
            const uint16_t z0 = C::down(w0 * C::up(y0)), z1 = C::down(w1 * C::up(y1));
            z[2 * i] = C::up(z0);
            z[2 * i + 1] = C::up(z1);
            zp[i] = (uint32_t)z0 | ((uint32_t)z1 << 16);
        }
        // rotate_half: the first half of the row takes -z[j + D/2], the second half z[j - D/2]
        u32x4 pp;
#pragma unroll
        for (int i = 0; i < 4; ++i) pp[i] = (uint32_t)__shfl_xor((int)zp[i], LPR / 2);
        const float sgn = t < LPR / 2 ? -1.f : 1.f;
        u32x4 outp;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float r0 = sgn * C::up((uint16_t)(pp[i] & 0xffffu)), r1 = sgn * C::up((uint16_t)(pp[i] >> 16));
            const float c0 = C::up((uint16_t)(craw[i] & 0xffffu)), c1 = C::up((uint16_t)(craw[i] >> 16));
            const float s0 = C::up((uint16_t)(sraw[i] & 0xffffu)), s1 = C::up((uint16_t)(sraw[i] >> 16));
            const float a0 = C::up(C::down(z[2 * i] * c0)) + C::up(C::down(r0 * s0));
            const float a1 = C::up(C::down(z[2 * i + 1] * c1)) + C::up(C::down(r1 * s1));
            outp[i] = (uint32_t)C::down(a0) | ((uint32_t)C::down(a1) << 16);
        }
        *reinterpret_cast<u32x4*>(dp) = outp;
    }
}

template <typename T, int D>
int launch_pre(const PreParams& p, hipStream_t stream) {
    constexpr int RPW = 64 / (D / 8);
    const int H_all = p.Hq + 2 * p.Hkv;
    const int64_t items = (int64_t)p.batch * p.S * ((H_all + RPW - 1) / RPW);
    int64_t blocks = (items + 3) / 4;                    // 4 waves per block, one item per wave
    const int64_t cap = 256 * 32;                        // grid-stride beyond that
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((ksa_pre_attention_kernel<T, D>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
    return ksa_check_launch();
}

}  // namespace

extern "C" int ksa_pre_attention(const void* q, const void* k, const void* v, const void* q_weight,
                                 const void* k_weight, const void* cos, const void* sin, void* q_out,
                                 void* k_out, void* v_out, int batch, int S, int Hq, int Hkv, int D,
                                 int dtype, const int64_t* q_strides, const int64_t* k_strides,
                                 const int64_t* v_strides, const int64_t* q_out_strides,
                                 const int64_t* k_out_strides, const int64_t* v_out_strides,
                                 const int64_t* cos_strides, float eps, void* stream) {
    if (!q || !k || !v || !q_weight || !k_weight || !cos || !sin || !q_out || !k_out || !v_out)
        return KSA_ERR_NULL;
    if (!q_strides || !k_strides || !v_strides || !q_out_strides || !k_out_strides || !v_out_strides ||
        !cos_strides)
        return KSA_ERR_NULL;
    if (batch <= 0 || S <= 0 || Hq <= 0 || Hkv <= 0 || !(eps >= 0.f)) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if (D != 64 && D != 128) return KSA_ERR_UNSUPPORTED;
    const void* ptrs[] = {q, k, v, q_weight, k_weight, cos, sin, q_out, k_out, v_out};
    for (const void* ptr : ptrs)
        if (reinterpret_cast<uintptr_t>(ptr) & 15) return KSA_ERR_ALIGN;
    const int64_t* st[] = {q_strides, k_strides, v_strides, q_out_strides, k_out_strides, v_out_strides};
    for (const int64_t* s3 : st)
        for (int i = 0; i < 3; ++i)
            if (s3[i] % 8) return KSA_ERR_ALIGN;
    if (cos_strides[0] % 8 || cos_strides[1] % 8) return KSA_ERR_ALIGN;

    PreParams p{};
    p.src[0] = (const uint16_t*)q, p.src[1] = (const uint16_t*)k, p.src[2] = (const uint16_t*)v;
    p.dst[0] = (uint16_t*)q_out, p.dst[1] = (uint16_t*)k_out, p.dst[2] = (uint16_t*)v_out;
    p.w[0] = (const uint16_t*)q_weight, p.w[1] = (const uint16_t*)k_weight;
    p.cos = (const uint16_t*)cos, p.sin = (const uint16_t*)sin;
    const int64_t* in[] = {q_strides, k_strides, v_strides};
    const int64_t* out[] = {q_out_strides, k_out_strides, v_out_strides};
    for (int i = 0; i < 3; ++i) {
        p.s_bs[i] = in[i][0], p.s_rs[i] = in[i][1], p.s_hs[i] = in[i][2];
        p.d_bs[i] = out[i][0], p.d_rs[i] = out[i][1], p.d_hs[i] = out[i][2];
    }
    p.c_bs = cos_strides[0], p.c_rs = cos_strides[1];
    p.batch = batch, p.S = S, p.Hq = Hq, p.Hkv = Hkv;
    p.eps = eps;
    hipStream_t stp = (hipStream_t)stream;
    if (dtype == KSA_DTYPE_BF16) {
        if (D == 128) return launch_pre<KsaBf16, 128>(p, stp);
        return launch_pre<KsaBf16, 64>(p, stp);
    }
    if (D == 128) return launch_pre<KsaF16, 128>(p, stp);
    return launch_pre<KsaF16, 64>(p, stp);
}
