// Block-sparse Summary-Attention prefill forward for gfx950.
//
// Replaces, for the forward pass, what the reference reaches through
//   summary_attn wheel, summary_attn/interface.py:70-91   (SummaryAttnFunc.forward)
//   flash_attn_cute wheel, flash_attn/cute/flash_fwd.py:1162-2480 (FlashAttentionForwardSm90)
//   flash_attn_cute wheel, flash_attn/cute/block_sparse_utils.py:134-476 (tile walk)
//   flash_attn_cute wheel, flash_attn/cute/softmax.py:52-146 (online soft-max)
// and keeps its numerics: 16-bit inputs, fp32 scores and soft-max state, exp2 with
// the scale folded in, probabilities rounded to 16 bit before the second product,
// fp32 output accumulator, one reciprocal per row at the end.
//
// One workgroup (4 waves) owns a 128-row query tile of one query head; wave w owns
// rows 32w .. 32w+31.  It walks the tile's non-empty key tiles (64 keys each) taken
// from the block index, staging K and V row-major in LDS (two buffers); V is transposed
// on the way out of LDS by ds_read_b64_tr_b16, see ksa_tile.h for the operand layouts.  The summary prefix of the key axis is
// read in place from the in-line summary rows (or from a separate prefix buffer),
// never concatenated.
//
// Partial tiles are masked from a 64-bit visibility word per query row; when every
// row of the wave is all-or-nothing in the tile (the common case: summary rows do
// not see old summaries, text rows see all of them) no per-element work is done.
#include <hip/hip_runtime.h>
#include <math.h>

#include "ksa_api_internal.h"
#include "ksa_mask.h"
#include "ksa_tile.h"

namespace {

struct PrefillParams {
    const uint16_t* q;
    const uint16_t* k;        // in-line keys   [Sq rows]
    const uint16_t* v;
    const uint16_t* kprefix;  // separate prefix rows [P rows] or null (read in place)
    const uint16_t* vprefix;
    uint16_t* out;
    float* lse;  // may be null
    const int32_t* mask_cnt;
    const int32_t* mask_idx;
    const int32_t* full_cnt;
    const int32_t* full_idx;
    int idx_stride;  // N
    int M, Hq, Hkv, g;
    int64_t q_bs, q_rs, q_hs;  // element strides: batch, row, head
    int64_t k_bs, k_rs, k_hs;
    int64_t v_bs, v_rs, v_hs;
    int64_t kp_bs, kp_rs, kp_hs;
    int64_t vp_bs, vp_rs, vp_hs;
    int64_t o_bs, o_rs, o_hs;
    int64_t lse_bs, lse_hs;
    KsaMask mk;
    float scale;
    float scale_log2;
};

constexpr int kThreads = 256;
constexpr int kTileM = 128;
constexpr int kTileN = 64;

template <typename T, int D>
__global__ __launch_bounds__(kThreads, 2) void ksa_prefill_kernel(const PrefillParams p) {
    using Ops = KsaOps<T>;
    constexpr int KS = D / 16;       // contraction steps of K Q^T
    constexpr int DB = D / 32;       // 32-row blocks of O^T
    constexpr int KROW = D + 8;      // padded LDS row of K (elements)
    constexpr int VROW = D + 16;     // padded LDS row of V (stride = 8 banks mod 64)
    constexpr int CPR = D / 8;       // 16-byte chunks per K/V row
    constexpr int KLD = (kTileN * CPR) / kThreads;  // K (and V) loads per thread

    __shared__ __attribute__((aligned(16))) uint16_t Ks[2][kTileN * KROW];
    __shared__ __attribute__((aligned(16))) uint16_t Vs[2][kTileN * VROW];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lq = lane & 31;
    const int lh = lane >> 5;

    // workgroup -> (kv head, query head in group, m tile); kv head fastest so that
    // the workgroups sharing K/V land on one XCD; heavy (late) m tiles first.
    const int bz = blockIdx.y;
    const int id = blockIdx.x;
    const int kvh = id % p.Hkv;
    const int rest = id / p.Hkv;
    const int gi = rest % p.g;
    const int mt = p.M - 1 - rest / p.g;
    const int head = kvh * p.g + gi;
    const KsaMask mk = p.mk;

    const int qrow = mt * kTileM + wave * 32 + lq;
    const int qrow_c = min(qrow, mk.Sq - 1);

    // Q as B operand, resident in registers for the whole tile walk
    u32x4 qf[KS];
    {
        const uint16_t* qp = p.q + bz * p.q_bs + (int64_t)qrow_c * p.q_rs + head * p.q_hs + 8 * lh;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const u32x4*>(qp + 16 * s);
    }

    const uint16_t* kbase = p.k + bz * p.k_bs + kvh * p.k_hs;
    const uint16_t* vbase = p.v + bz * p.v_bs + kvh * p.v_hs;
    const uint16_t* kpbase = p.kprefix ? p.kprefix + bz * p.kp_bs + kvh * p.kp_hs : nullptr;
    const uint16_t* vpbase = p.vprefix ? p.vprefix + bz * p.vp_bs + kvh * p.vp_hs : nullptr;
    const int Bblk = mk.C + mk.S;

    const int npart = p.mask_cnt[mt];
    const int ntiles = npart + p.full_cnt[mt];
    const int32_t* plist = p.mask_idx + (int64_t)mt * p.idx_stride;
    const int32_t* flist = p.full_idx + (int64_t)mt * p.idx_stride;

    u32x4 kreg[KLD];
    u32x4 vreg[KLD];

    auto row_ptrs = [&](int kv, const uint16_t*& kr, const uint16_t*& vr) {
        kv = min(kv, mk.Sk - 1);
        if (kv < mk.P) {
            if (kpbase) {
                kr = kpbase + (int64_t)kv * p.kp_rs;
                vr = vpbase + (int64_t)kv * p.vp_rs;
            } else {  // prefix row j lives at in-line row (j/S)*B + C + j%S
                const int r = (kv / mk.S) * Bblk + mk.C + (kv % mk.S);
                kr = kbase + (int64_t)r * p.k_rs;
                vr = vbase + (int64_t)r * p.v_rs;
            }
        } else {
            kr = kbase + (int64_t)(kv - mk.P) * p.k_rs;
            vr = vbase + (int64_t)(kv - mk.P) * p.v_rs;
        }
    };

    auto load_tile = [&](int n) {
        const int n0 = n * kTileN;
#pragma unroll
        for (int i = 0; i < KLD; ++i) {
            const int u = tid + kThreads * i;
            const int row = u / CPR, c = u % CPR;
            const uint16_t *kr, *vr;
            row_ptrs(n0 + row, kr, vr);
            kreg[i] = *reinterpret_cast<const u32x4*>(kr + 8 * c);
            vreg[i] = *reinterpret_cast<const u32x4*>(vr + 8 * c);
        }
    };

    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < KLD; ++i) {
            const int u = tid + kThreads * i;
            const int row = u / CPR, c = u % CPR;
            *reinterpret_cast<u32x4*>(&Ks[buf][row * KROW + 8 * c]) = kreg[i];
            *reinterpret_cast<u32x4*>(&Vs[buf][row * VROW + 8 * c]) = vreg[i];
        }
    };

    auto tile_at = [&](int i) { return i < npart ? plist[i] : flist[i - npart]; };

    floatx16 oacc[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[b][i] = 0.f;
    float m_run = -INFINITY;
    float l_run = 0.f;
    const float c2 = p.scale_log2;

    if (ntiles > 0) load_tile(tile_at(0));

    for (int it = 0; it < ntiles; ++it) {
        const int buf = it & 1;
        const int n = tile_at(it);
        const int n0 = n * kTileN;
        store_tile(buf);
        __syncthreads();
        if (it + 1 < ntiles) load_tile(tile_at(it + 1));

        // ---- S^T = K Q^T ----
        floatx16 sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(
                    &Ks[buf][(kb * 32 + lq) * KROW + 16 * s + 8 * lh]);
                sacc[kb] = Ops::mfma(a, qf[s], sacc[kb]);
            }
        }

        // ---- mask ----
        bool row_vis = true;
        const bool need_mask = (it < npart) || (n0 + kTileN > mk.Sk);
        if (need_mask) {
            uint64_t text, valid;
            ksa_tile_column_bits(mk, n0, lane, text, valid);
            const uint64_t bits = ksa_row_bits(mk, qrow_c, n0, text, valid);
            const bool uniform = __all(bits == 0ull || bits == ~0ull);
            if (uniform) {
                row_vis = bits != 0ull;
            } else {
                const uint64_t sh = bits >> (4 * lh);
                const uint32_t w0 = (uint32_t)sh, w1 = (uint32_t)(sh >> 32);
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t bit = 1u << (8 * (i / 4) + (i % 4));
                    sacc[0][i] = (w0 & bit) ? sacc[0][i] : -INFINITY;
                    sacc[1][i] = (w1 & bit) ? sacc[1][i] : -INFINITY;
                }
            }
        }

        // ---- online soft-max (one query row per lane pair l, l^32) ----
        float mloc = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, fmaxf(sacc[0][i], sacc[1][i]));
        if (!row_vis) mloc = -INFINITY;
        mloc = fmaxf(mloc, ksa_xor32(mloc));
        const float m_new = fmaxf(m_run, mloc);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = ksa_exp2((m_run - m_safe) * c2);
        const float mc = row_vis ? m_safe * c2 : INFINITY;
        m_run = m_new;

        float rowsum = 0.f;
        u32x4 pf[4];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                const float p0 = ksa_exp2(fmaf(sacc[kb][i], c2, -mc));
                const float p1 = ksa_exp2(fmaf(sacc[kb][i + 1], c2, -mc));
                rowsum += p0 + p1;
                pf[kb * 2 + i / 8][(i % 8) / 2] = Ops::pack2(p0, p1);
            }
        l_run = l_run * alpha + rowsum;

        if (__any(alpha != 1.f)) {
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[b][i] *= alpha;
        }

        // ---- O^T += V^T P^T ----
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int b = 0; b < DB; ++b) {
                const u32x4 a = ksa_read_vt_frag<VROW>(Vs[buf], ks, b, lq, lh);
                oacc[b] = Ops::mfma(a, pf[ks], oacc[b]);
            }
        }
    }

    // ---- epilogue ----
    const float l_tot = l_run + ksa_xor32(l_run);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (qrow < mk.Sq) {
        uint16_t* op = p.out + bz * p.o_bs + (int64_t)qrow * p.o_rs + head * p.o_hs;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32x2 w;
                w[0] = Ops::pack2(oacc[b][4 * j] * inv, oacc[b][4 * j + 1] * inv);
                w[1] = Ops::pack2(oacc[b][4 * j + 2] * inv, oacc[b][4 * j + 3] * inv);
                *reinterpret_cast<u32x2*>(op + 32 * b + 8 * j + 4 * lh) = w;
            }
        if (p.lse && lh == 0)
            p.lse[bz * p.lse_bs + head * p.lse_hs + qrow] =
                l_tot > 0.f ? m_run * p.scale + logf(l_tot) : -INFINITY;
    }
}

template <typename T, int D>
int launch(const PrefillParams& p, int batch, hipStream_t stream) {
    dim3 grid(p.M * p.Hq, batch);
    hipLaunchKernelGGL((ksa_prefill_kernel<T, D>), grid, dim3(kThreads), 0, stream, p);
    return ksa_check_launch();
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool stride_ok(int64_t s) { return (s % 8) == 0; }

}  // namespace

extern "C" int ksa_prefill_fwd(const void* q, const void* k, const void* v, const void* kprefix,
                               const void* vprefix, void* out, float* lse, int batch, int Sq,
                               int Hq, int Hkv, int D, int dtype, const int64_t* q_strides,
                               const int64_t* k_strides, const int64_t* v_strides,
                               const int64_t* kprefix_strides, const int64_t* vprefix_strides,
                               const int64_t* out_strides, int C, int S, int W, int P,
                               int skip_old, const int32_t* mask_cnt, const int32_t* mask_idx,
                               const int32_t* full_cnt, const int32_t* full_idx, int idx_stride,
                               float scale, void* stream) {
    if (!q || !k || !v || !out || !mask_cnt || !mask_idx || !full_cnt || !full_idx) return KSA_ERR_NULL;
    if (!q_strides || !k_strides || !v_strides || !out_strides) return KSA_ERR_NULL;
    if ((kprefix == nullptr) != (vprefix == nullptr)) return KSA_ERR_NULL;
    if (kprefix && (!kprefix_strides || !vprefix_strides)) return KSA_ERR_NULL;
    if (batch <= 0 || Sq <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return KSA_ERR_INVALID;
    if (C <= 0 || S <= 0 || W < 0 || P < 0) return KSA_ERR_INVALID;
    if ((int64_t)Sq + P >= (1ll << 30)) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    const int Sk = Sq + P;
    const int N = (Sk + kTileN - 1) / kTileN;
    if (idx_stride < N) return KSA_ERR_INVALID;
    if (!kprefix && P > 0) {
        // in-place prefix: row j is in-line row (j/S)*B + C + j%S, which must exist
        const int64_t last = (int64_t)((P - 1) / S) * (C + S) + C + (P - 1) % S;
        if (last >= Sq) return KSA_ERR_INVALID;
    }
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return KSA_ERR_ALIGN;
    if (kprefix && (!aligned16(kprefix) || !aligned16(vprefix))) return KSA_ERR_ALIGN;
    for (int i = 0; i < 3; ++i) {
        if (!stride_ok(q_strides[i]) || !stride_ok(k_strides[i]) || !stride_ok(v_strides[i]) ||
            !stride_ok(out_strides[i]))
            return KSA_ERR_ALIGN;
        if (kprefix && (!stride_ok(kprefix_strides[i]) || !stride_ok(vprefix_strides[i])))
            return KSA_ERR_ALIGN;
    }

    PrefillParams p{};
    p.q = (const uint16_t*)q;
    p.k = (const uint16_t*)k;
    p.v = (const uint16_t*)v;
    p.kprefix = (const uint16_t*)kprefix;
    p.vprefix = (const uint16_t*)vprefix;
    p.out = (uint16_t*)out;
    p.lse = lse;
    p.mask_cnt = mask_cnt;
    p.mask_idx = mask_idx;
    p.full_cnt = full_cnt;
    p.full_idx = full_idx;
    p.idx_stride = idx_stride;
    p.M = (Sq + kTileM - 1) / kTileM;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.g = Hq / Hkv;
    p.q_bs = q_strides[0], p.q_rs = q_strides[1], p.q_hs = q_strides[2];
    p.k_bs = k_strides[0], p.k_rs = k_strides[1], p.k_hs = k_strides[2];
    p.v_bs = v_strides[0], p.v_rs = v_strides[1], p.v_hs = v_strides[2];
    if (kprefix) {
        p.kp_bs = kprefix_strides[0], p.kp_rs = kprefix_strides[1], p.kp_hs = kprefix_strides[2];
        p.vp_bs = vprefix_strides[0], p.vp_rs = vprefix_strides[1], p.vp_hs = vprefix_strides[2];
    }
    p.o_bs = out_strides[0], p.o_rs = out_strides[1], p.o_hs = out_strides[2];
    p.lse_bs = (int64_t)Hq * Sq;
    p.lse_hs = Sq;
    p.mk = KsaMask{C, S, W, P, skip_old ? 1 : 0, Sq, Sk};
    p.scale = scale;
    p.scale_log2 = scale * 1.4426950408889634f;

    hipStream_t st = (hipStream_t)stream;
    if (dtype == KSA_DTYPE_BF16) {
        if (D == 128) return launch<KsaBf16, 128>(p, batch, st);
        if (D == 64) return launch<KsaBf16, 64>(p, batch, st);
    } else {
        if (D == 128) return launch<KsaF16, 128>(p, batch, st);
        if (D == 64) return launch<KsaF16, 64>(p, batch, st);
    }
    return KSA_ERR_UNSUPPORTED;
}
