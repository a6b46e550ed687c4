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
#include "ksa_cvt.h"

namespace {

struct PreParams {
    const uint16_t* src[3];   // q, k, v projections  [batch, S, H, D] by strides
    uint16_t* dst[3];         // q, k, v outputs
    const uint16_t* w[2];     // q_norm, k_norm weights [D]
    const int32_t* kv_row;    // null, or [batch]: row added to the k / v destination of a sequence, or
    int kv_row_per_token;     // (flag) [batch][S]: the k / v destination row of every token, in place of its position
    const float* part;        // if set: q | k | v rows as K-split partial sums [ksplit][ksa_partial_rows(batch S)][(Hq + 2 Hkv) D], src unused
    int ksplit;
    const uint16_t* cos;      // [batch or 1, S, D]
    const uint16_t* sin;
    int64_t s_bs[3], s_rs[3], s_hs[3];
    int64_t d_bs[3], d_rs[3], d_hs[3];
    int64_t c_bs, c_rs;
    int batch, S, Hq, Hkv;
    int tok_per_pass;  // tokens per workgroup pass: 4 / gcd(row groups per token, 4)
    float eps;
    int passes_per_wg;  // passes of tok_per_pass consecutive tokens that one workgroup takes
};

template <typename T>
using PreCvt = KsaCvt<T>;

// value of the lane `n` places further inside the same row of 16 lanes (cyclic)
template <int N>
__device__ __forceinline__ uint32_t pre_row_ror(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x120 + N, 0xf, 0xf, false);
}

// sum over the LPR lanes that hold one head row; every lane of the row gets the total
template <int LPR>
__device__ __forceinline__ float pre_row_sum(float ss) {
    if constexpr (LPR == 16) {  // rotations inside a DPP row (16 lanes)
        ss += __builtin_bit_cast(float, pre_row_ror<8>(__builtin_bit_cast(uint32_t, ss)));
        ss += __builtin_bit_cast(float, pre_row_ror<4>(__builtin_bit_cast(uint32_t, ss)));
        ss += __builtin_bit_cast(float, pre_row_ror<2>(__builtin_bit_cast(uint32_t, ss)));
        ss += __builtin_bit_cast(float, pre_row_ror<1>(__builtin_bit_cast(uint32_t, ss)));
    } else {
#pragma unroll
        for (int m = 1; m < LPR; m <<= 1) ss += __shfl_xor(ss, m);
    }
    return ss;
}

// One workgroup takes a few consecutive tokens; its four waves share
// their head rows, RPW rows of one of q / k / v per wave instruction, the same number for every
// wave.  Which tensor a wave instruction works on, the token's base addresses and the weights
// are wave-uniform (scalar registers); a lane only adds its row's offset, so no index division
// or 64-bit multiply sits in the inner loop.  Products of two 16-bit values are taken with
// packed dot products against operands that hold one element and a zero, straight from the
// packed words (exact in fp32), and the final sum of the two rounded terms is a dot product
// with (1, 1).
// kPartials: the rows come as K-split partial sums (a variant of its own, so that the streaming
// variant does not carry its registers).
template <typename T, int D, bool kPartials>
__global__ __launch_bounds__(256) void ksa_pre_attention_kernel(const PreParams p) {
    using C = PreCvt<T>;
    constexpr int LPR = D / 8;          // lanes per head row
    constexpr int RPW = 64 / LPR;       // head rows per wave instruction
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sub = lane / LPR;         // which of the wave's rows
    const int t = lane % LPR;           // 16-byte chunk inside the row
    const int Gq = (p.Hq + RPW - 1) / RPW, Gk = (p.Hkv + RPW - 1) / RPW;
    const int G = Gq + 2 * Gk;
    const int ntok = p.batch * p.S;
    // rotate_half: the first half of a row takes -z[j + D/2], the second half +z[j - D/2];
    // the sign goes into the sine once per token
    const uint32_t sgn_bits = t < LPR / 2 ? 0x80008000u : 0u;
    // this lane's slice of the two weight vectors, each packed word split into (low, 0) and
    // (0, high): a packed dot product with such a word is the exact fp32 product of one element,
    // taken straight from packed operands
    uint32_t wlo[2][4], whi[2][4];
    {
        const u32x4 wq = *reinterpret_cast<const u32x4*>(p.w[0] + 8 * t);
        const u32x4 wk = *reinterpret_cast<const u32x4*>(p.w[1] + 8 * t);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            wlo[0][i] = wq[i] & 0xffffu;
            whi[0][i] = wq[i] & 0xffff0000u;
            wlo[1][i] = wk[i] & 0xffffu;
            whi[1][i] = wk[i] & 0xffff0000u;
        }
    }
    // element offset of this lane's row inside a wave instruction's block of rows
    uint32_t lsrc[3], ldst[3];
#pragma unroll
    for (int w = 0; w < 3; ++w) {
        lsrc[w] = (uint32_t)sub * (uint32_t)p.s_hs[w] + 8 * t;
        ldst[w] = (uint32_t)sub * (uint32_t)p.d_hs[w] + 8 * t;
    }

    // A pass covers TOK consecutive tokens, TOK * G row groups in all, a multiple of four, so
    // that the four waves get the same number of groups (G = 12 with 32 + 8 + 8 heads of 128: one
    // token, three groups per wave); a workgroup takes a few consecutive passes and ends.
    // (token, group) advance by four per wave step.  A wave walks its groups as one sequence and
    // requests the rows of the next group (and the rotary row, when the token changes) before
    // it works on the current one, so two of its row requests are in flight.
    const int TOK = p.tok_per_pass;
    const int span = p.passes_per_wg * TOK;  // consecutive tokens of one workgroup
    // (a handful of tokens: gridDim.y workgroups share a token, each taking every gridDim.y-th set
    // of four row groups, so that no wave has more than one group to do)
    const int gstep = 4 * gridDim.y;
    int gi = (wave + 4 * blockIdx.y) % G, tl = (wave + 4 * blockIdx.y) / G, t0 = blockIdx.x * span;
    const int t_end = min(ntok, t0 + span);
    struct Group {
        bool live;             // wave-uniform: there is such a group
        int which, tok, h0;
        int col0;              // partial-sum input: first column of the group's first head
        const uint16_t* sbase;
        uint16_t* dbase;
    };
    int nb = 0, ns = 0, ntk = -1;  // batch index and position of the token of the last group
    auto next_group = [&]() {
        Group g;
        while (gi >= G) {
            gi -= G;
            ++tl;
        }
        if (tl >= TOK) {  // groups per wave and pass are equal, so tl < 2 * TOK here
            tl -= TOK;
            t0 += TOK;
        }
        g.tok = t0 + tl;
        g.live = g.tok < t_end;  // tokens only grow along the sequence: the first miss ends it
        if (g.live && g.tok != ntk) {
            ntk = g.tok;
            nb = g.tok / p.S;
            ns = g.tok - nb * p.S;
        }
        g.which = gi < Gq ? 0 : (gi < Gq + Gk ? 1 : 2);
        g.h0 = (gi - (g.which == 0 ? 0 : (g.which == 1 ? Gq : Gq + Gk))) * RPW;
        g.col0 = ((g.which == 0 ? 0 : (g.which == 1 ? p.Hq : p.Hq + p.Hkv)) + g.h0) * D;
        g.sbase = p.src[g.which] + nb * p.s_bs[g.which] + (int64_t)ns * p.s_rs[g.which] + (int64_t)g.h0 * p.s_hs[g.which];
        // (k and v may go to a row of their sequence that the host does not know: a cache cursor)
        int64_t drow = ns;
        if (g.which != 0 && p.kv_row) drow = p.kv_row_per_token ? p.kv_row[g.tok] : ns + p.kv_row[nb];
        g.dbase = p.dst[g.which] + nb * p.d_bs[g.which] + drow * p.d_rs[g.which] + (int64_t)g.h0 * p.d_hs[g.which];
        gi += gstep;
        return g;
    };
    auto pick = [](int which, const uint32_t (&a)[3]) { return which == 0 ? a[0] : (which == 1 ? a[1] : a[2]); };
    // a lane group beyond the last head is idle as a whole, exchange partners included
    auto lane_ok = [&](const Group& g) { return g.h0 + sub < (g.which == 0 ? p.Hq : p.Hkv); };
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    // this lane's 16 bytes of a group's rows: from the projection output, or (decode steps) from
    // the K-split partial sums of the projection, added and rounded as its own reduction would
    auto fetch = [&](const Group& g) {
        if constexpr (kPartials)
            return ksa_sum_partials8<T>(p.part, p.ksplit, ksa_partial_rows(ntok), (p.Hq + 2 * p.Hkv) * D, g.tok, g.col0 + sub * D + 8 * t);
        return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(g.sbase + pick(g.which, lsrc)));
    };

    Group g = next_group();
    u32x4 raw = zero4, craw = zero4, sraw = zero4;
    if (g.live) {
        craw = *reinterpret_cast<const u32x4*>(p.cos + nb * p.c_bs + (int64_t)ns * p.c_rs + 8 * t);
        sraw = *reinterpret_cast<const u32x4*>(p.sin + nb * p.c_bs + (int64_t)ns * p.c_rs + 8 * t);
        // every byte of q, k, v is touched once: non-temporal accesses
        if (lane_ok(g)) raw = fetch(g);
    }
    int cur = -1;  // token whose rotary row is split below
    uint32_t clo[4], chi[4], slo[4], shi[4];
    while (g.live) {
        const Group n = next_group();
        u32x4 raw_n = zero4, craw_n = craw, sraw_n = sraw;
        if (n.live) {
            if (n.tok != g.tok) {
                craw_n = *reinterpret_cast<const u32x4*>(p.cos + nb * p.c_bs + (int64_t)ns * p.c_rs + 8 * t);
                sraw_n = *reinterpret_cast<const u32x4*>(p.sin + nb * p.c_bs + (int64_t)ns * p.c_rs + 8 * t);
            }
            if (lane_ok(n)) raw_n = fetch(n);
        }
        if (g.tok != cur) {  // wave-uniform: the rotary row of this token, split like the weights
            cur = g.tok;
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // the sine carries the rotate_half sign
                clo[i] = craw[i] & 0xffffu;
                chi[i] = craw[i] & 0xffff0000u;
                slo[i] = (sraw[i] ^ sgn_bits) & 0xffffu;
                shi[i] = (sraw[i] ^ sgn_bits) & 0xffff0000u;
            }
        }
        if (lane_ok(g)) {
            uint16_t* dp = g.dbase + pick(g.which, ldst);
            if (g.which == 2) {  // v: layout change only
                __builtin_nontemporal_store(raw, reinterpret_cast<u32x4*>(dp));
            } else {
                float ss = 0.f;
#pragma unroll
                for (int i = 0; i < 4; ++i) ss = C::dot2(raw[i], raw[i], ss);
                ss = pre_row_sum<LPR>(ss);
                const float inv = rsqrtf(ss * (1.0f / D) + p.eps);
                // z = round(w * round(x * inv)), kept packed for the exchange
                u32x4 zp;
                auto scale_rows = [&](const uint32_t (&wl)[4], const uint32_t (&wh)[4]) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint32_t y = C::down2(C::lo(raw[i]) * inv, C::hi(raw[i]) * inv);
                        float z0, z1;
                        C::dot2z_x2(y, wl[i], y, wh[i], z0, z1);
                        zp[i] = C::down2(z0, z1);
                    }
                };
                if (g.which == 0) scale_rows(wlo[0], whi[0]);
                else scale_rows(wlo[1], whi[1]);
                // out = round(round(z cos) + round(rot(z) sin)); the two rounded terms of an
                // element are packed together and added by a dot product with (1, 1)
                u32x4 outp;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    uint32_t pp;  // the partner half of the row
                    if constexpr (LPR == 16) pp = pre_row_ror<8>(zp[i]);
                    else pp = (uint32_t)__shfl_xor((int)zp[i], LPR / 2);
                    float c0, s0, c1, s1, o0, o1;
                    C::dot2z_x4(zp[i], clo[i], pp, slo[i], zp[i], chi[i], pp, shi[i], c0, s0, c1, s1);
                    const uint32_t e0 = C::down2(c0, s0), e1 = C::down2(c1, s1);
                    C::dot2z_x2(e0, C::kOnes, e1, C::kOnes, o0, o1);
                    outp[i] = C::down2(o0, o1);
                }
                __builtin_nontemporal_store(outp, reinterpret_cast<u32x4*>(dp));
            }
        }
        g = n;
        raw = raw_n, craw = craw_n, sraw = sraw_n;
    }
}

template <typename T, int D>
int launch_pre(PreParams p, hipStream_t stream) {
    constexpr int RPW = 64 / (D / 8);
    const int G = (p.Hq + RPW - 1) / RPW + 2 * ((p.Hkv + RPW - 1) / RPW);
    p.tok_per_pass = (G % 4 == 0) ? 1 : (G % 2 == 0 ? 2 : 4);
    // Short-lived workgroups over consecutive tokens, in launch order, keep the window of
    // addresses in flight narrow: measured 5 % faster than a grid-stride loop of long-lived
    // workgroups over the same accesses (a plain copy shows the same preference, 6.2 against
    // 4.9 TB/s).  Four passes amortise a workgroup's set-up; 2 .. 8 measure alike.
    // (a handful of tokens - a decode step - get one pass per workgroup: all the parallelism there is)
    p.passes_per_wg = (int64_t)p.batch * p.S / p.tok_per_pass >= 4 * 1024 ? 4 : 1;
    const int64_t span = (int64_t)p.passes_per_wg * p.tok_per_pass;
    const int64_t blocks = ((int64_t)p.batch * p.S + span - 1) / span;
    // a decode step (one pass of one token per workgroup): one workgroup per four row groups of a
    // token instead of one per token - the groups of a wave are a chain of dependent loads
    const int parts = (p.passes_per_wg == 1 && p.tok_per_pass == 1 && blocks <= kMaxPartialRows) ? G / 4 : 1;
    const dim3 grid((unsigned)blocks, (unsigned)parts);
    if (p.part)
        hipLaunchKernelGGL((ksa_pre_attention_kernel<T, D, true>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((ksa_pre_attention_kernel<T, D, false>), grid, dim3(256), 0, stream, p);
    return ksa_check_launch();
}

int dispatch_pre(const PreParams& p, int D, int dtype, hipStream_t stp) {
    if (dtype == KSA_DTYPE_BF16) {
        if (D == 128) return launch_pre<KsaBf16, 128>(p, stp);
        return launch_pre<KsaBf16, 64>(p, stp);
    }
    if (D == 128) return launch_pre<KsaF16, 128>(p, stp);
    return launch_pre<KsaF16, 64>(p, stp);
}

}  // namespace

extern "C" int ksa_pre_attention(const void* q, const void* k, const void* v, const void* q_weight,
                                 const void* k_weight, const void* cos, const void* sin, void* q_out,
                                 void* k_out, void* v_out, int batch, int S, int Hq, int Hkv, int D,
                                 int dtype, const int64_t* q_strides, const int64_t* k_strides,
                                 const int64_t* v_strides, const int64_t* q_out_strides,
                                 const int64_t* k_out_strides, const int64_t* v_out_strides,
                                 const int64_t* cos_strides, const int32_t* kv_out_row_seq, int kv_out_row_per_token,
                                 float eps, void* stream) {
    if (!q || !k || !v || !q_weight || !k_weight || !cos || !sin || !q_out || !k_out || !v_out)
        return KSA_ERR_NULL;
    if (!q_strides || !k_strides || !v_strides || !q_out_strides || !k_out_strides || !v_out_strides ||
        !cos_strides)
        return KSA_ERR_NULL;
    if (batch <= 0 || S <= 0 || Hq <= 0 || Hkv <= 0 || !(eps >= 0.f)) return KSA_ERR_INVALID;
    if ((int64_t)batch * S >= (1ll << 31) - 64) return KSA_ERR_INVALID;  // token indices, plus a workgroup's span, in 32 bits
    // a lane's row offset inside one wave instruction (at most 8 head rows) is kept in 32 bits
    for (const int64_t* s3 : {q_strides, k_strides, v_strides, q_out_strides, k_out_strides, v_out_strides})
        if (s3[2] < 0 || s3[2] * 8 + 128 >= (1ll << 32)) return KSA_ERR_INVALID;
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
    p.kv_row = kv_out_row_seq;
    p.kv_row_per_token = kv_out_row_per_token != 0;
    const int64_t* in[] = {q_strides, k_strides, v_strides};
    const int64_t* out[] = {q_out_strides, k_out_strides, v_out_strides};
    for (int i = 0; i < 3; ++i) {
        p.s_bs[i] = in[i][0], p.s_rs[i] = in[i][1], p.s_hs[i] = in[i][2];
        p.d_bs[i] = out[i][0], p.d_rs[i] = out[i][1], p.d_hs[i] = out[i][2];
    }
    p.c_bs = cos_strides[0], p.c_rs = cos_strides[1];
    p.batch = batch, p.S = S, p.Hq = Hq, p.Hkv = Hkv;
    p.eps = eps;
    return dispatch_pre(p, D, dtype, (hipStream_t)stream);
}

extern "C" int ksa_pre_attention_partials(const float* partials, int ksplit, const void* q_weight,
                                          const void* k_weight, const void* cos, const void* sin, void* q_out,
                                          void* k_out, void* v_out, int batch, int S, int Hq, int Hkv, int D,
                                          int dtype, const int64_t* q_out_strides, const int64_t* k_out_strides,
                                          const int64_t* v_out_strides, const int64_t* cos_strides,
                                          const int32_t* kv_out_row_seq, int kv_out_row_per_token, float eps,
                                          void* stream) {
    if (!partials || !q_weight || !k_weight || !cos || !sin || !q_out || !k_out || !v_out) return KSA_ERR_NULL;
    if (!q_out_strides || !k_out_strides || !v_out_strides || !cos_strides) return KSA_ERR_NULL;
    if (batch <= 0 || S <= 0 || (int64_t)batch * S > kMaxPartialRows || Hq <= 0 || Hkv <= 0 || ksplit < 1 || ksplit > 64 ||
        !(eps >= 0.f))
        return KSA_ERR_INVALID;
    for (const int64_t* s3 : {q_out_strides, k_out_strides, v_out_strides})
        if (s3[2] < 0 || s3[2] * 8 + 128 >= (1ll << 32)) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if (D != 64 && D != 128) return KSA_ERR_UNSUPPORTED;
    const void* ptrs[] = {partials, q_weight, k_weight, cos, sin, q_out, k_out, v_out};
    for (const void* ptr : ptrs)
        if (reinterpret_cast<uintptr_t>(ptr) & 15) return KSA_ERR_ALIGN;
    for (const int64_t* s3 : {q_out_strides, k_out_strides, v_out_strides})
        for (int i = 0; i < 3; ++i)
            if (s3[i] % 8) return KSA_ERR_ALIGN;
    if (cos_strides[0] % 8 || cos_strides[1] % 8) return KSA_ERR_ALIGN;
    PreParams p{};
    p.part = partials;
    p.ksplit = ksplit;
    p.dst[0] = (uint16_t*)q_out, p.dst[1] = (uint16_t*)k_out, p.dst[2] = (uint16_t*)v_out;
    p.w[0] = (const uint16_t*)q_weight, p.w[1] = (const uint16_t*)k_weight;
    p.cos = (const uint16_t*)cos, p.sin = (const uint16_t*)sin;
    p.kv_row = kv_out_row_seq;
    p.kv_row_per_token = kv_out_row_per_token != 0;
    const int64_t* out[] = {q_out_strides, k_out_strides, v_out_strides};
    for (int i = 0; i < 3; ++i) {
        p.s_hs[i] = D;  // (only the lane offsets are derived from it; the source is `partials`)
        p.d_bs[i] = out[i][0], p.d_rs[i] = out[i][1], p.d_hs[i] = out[i][2];
    }
    p.c_bs = cos_strides[0], p.c_rs = cos_strides[1];
    p.batch = batch, p.S = S, p.Hq = Hq, p.Hkv = Hkv;
    p.eps = eps;
    return dispatch_pre(p, D, dtype, (hipStream_t)stream);
}
