// Decode attention over the contiguous ring-buffer KV slice for gfx950.
//
// Replaces the reference's decode attention function
//   examples/pretrain/hf_template/modeling_qwen3sa.py:591-612 (_sdpa_attention_forward)
//   examples/pretrain/hf_template/modeling_qwen3sa.py:557-566 (repeat_kv)
// i.e. softmax(q K^T * scale) V without any mask over rows [start_b, end_b) of the
// cache slice returned by Qwen3RingBufferCache.get_attention_kv (:402-434).  The
// reference materialises g copies of K and V per step; here every K/V row is read
// from HBM exactly once per kv head and shared by the g query heads (and by all
// query tokens of a chunk-boundary step) as columns of one MFMA tile.
//
// Split-K: a workgroup owns (sequence, kv head, split); its 4 waves stream disjoint
// 32-row tiles with private LDS staging (no workgroup barrier in the loop) and keep
// private (max, sum, O^T) state that is merged across the waves through LDS at the
// end; with more than one split the un-normalised partials go to a workspace and a
// second kernel merges them.
#include <hip/hip_runtime.h>
#include <math.h>

#include <mutex>

#include "ksa_api_internal.h"
#include "ksa_tile.h"

namespace {

struct DecodeParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* out;
    const int32_t* start;  // per sequence or null
    const int32_t* end;
    int start0, end0;
    int Hq, Hkv, g, Q;
    int ncols;   // Q * g columns per kv head
    int nsplit;
    int64_t q_bs, q_hs, q_qs;   // element strides of q [B,Hq,Q,D]
    int64_t k_bs, k_hs, k_rs;   // cache [B,Hkv,rows,D]
    int64_t v_bs, v_hs, v_rs;
    int64_t o_bs, o_qs, o_hs;   // out [B,Q,Hq,D]
    float* ws_o;   // [B,Hkv,nsplit,ncols_pad,D] un-normalised partial outputs
    float* ws_ml;  // [B,Hkv,nsplit,ncols_pad,2]  (max in log2 units, sum)
    int ncols_pad;
    float scale_log2;
    // Chunk-boundary form (split_q != 0): query token 0 (the chunk's last text token) attends the rows
    // [start, end) and has column block 0 to itself (g columns); the other Q - 1 query tokens (the
    // chunk's summary tokens) attend [start2, end2) and fill the column blocks behind it.
    int split_q;
    const int32_t* start2;
    const int32_t* end2;
    int start20, end20;
};

// column lq of column block colblk -> (query token, head in the group); false: no such column
__device__ __forceinline__ bool ksa_decode_column(const DecodeParams& p, int colblk, int lq, int& qi, int& gi) {
    if (!p.split_q) {
        const int col = colblk * 32 + lq;
        qi = col / p.g, gi = col % p.g;
        return col < p.ncols;
    }
    if (colblk == 0) {
        qi = 0, gi = lq;
        return lq < p.g;
    }
    const int c = (colblk - 1) * 32 + lq;
    qi = 1 + c / p.g, gi = c % p.g;
    return c < (p.Q - 1) * p.g;
}
// slot of the logical column (query token qi, head gi) in the workspace's column axis
__device__ __forceinline__ int ksa_decode_slot(const DecodeParams& p, int qi, int gi) {
    if (!p.split_q) return qi * p.g + gi;
    return qi == 0 ? gi : 32 + (qi - 1) * p.g + gi;
}

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kRows = 32;  // key rows per wave tile

template <typename T, int D>
__global__ __launch_bounds__(kThreads, (D <= 128 ? 2 : 1)) void ksa_decode_kernel(const DecodeParams p) {
    using Ops = KsaOps<T>;
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int KROW = D + 8;
    constexpr int VROW = D + 16;
    constexpr int CPR = D / 8;
    constexpr int KLD = (kRows * CPR) / 64;          // K (and V) loads per lane
    constexpr int kStage = kRows * (KROW + VROW);    // elements of one wave's staging area
    constexpr int kMergeFloats = kWaves * 32 * (D + 2);
    constexpr int kSmemBytes = (kWaves * kStage * 2 > kMergeFloats * 4) ? kWaves * kStage * 2
                                                                        : kMergeFloats * 4;
    __shared__ __attribute__((aligned(16))) unsigned char smem[kSmemBytes];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lq = lane & 31;
    const int lh = lane >> 5;

    const int split = blockIdx.x;
    const int kvh = blockIdx.y % p.Hkv;
    const int bz = blockIdx.z;

    uint16_t* Kw = reinterpret_cast<uint16_t*>(smem) + wave * kStage;
    uint16_t* Vw = Kw + kRows * KROW;

    // One column block per workgroup - except in the chunk-boundary form, where the workgroup of the text
    // token's block takes the summary tokens' blocks behind it (their row range is one chunk: a tile or two
    // for two of the splits, nothing for the others).  As workgroups of their own, scattered between the long
    // ones, those short blocks held places of a CU for a chain of memory round trips under full load, and the
    // long workgroups that had to wait for the places ended late: +8 us per small-window layer and +27 us
    // per large-window layer of a boundary step.
    const int colblk_first = p.split_q ? 0 : blockIdx.y / p.Hkv;
    const int colblk_last = p.split_q ? p.ncols_pad / 32 - 1 : colblk_first;
    for (int colblk = colblk_first; colblk <= colblk_last; ++colblk) {
    if (colblk != colblk_first) __syncthreads();  // the previous block's merge area becomes staging again
    const bool second = p.split_q && colblk > 0;  // the summary tokens' columns and their own row range
    const int r_begin = second ? (p.start2 ? p.start2[bz] : p.start20) : (p.start ? p.start[bz] : p.start0);
    const int r_end = second ? (p.end2 ? p.end2[bz] : p.end20) : (p.end ? p.end[bz] : p.end0);
    const int L = max(r_end - r_begin, 0);
    // rows per split: a multiple of the 128 rows the four waves cover per round
    const int per = ((L + p.nsplit - 1) / p.nsplit + kWaves * kRows - 1) / (kWaves * kRows) *
                    (kWaves * kRows);
    const int s0 = r_begin + split * per;
    const int s1 = min(r_end, s0 + per);

    if (p.nsplit > 1 && s0 >= s1) {
        // an empty slice (a short range: the summary tokens' chunk at a boundary step, a sequence with few
        // rows): the merge only needs to know that there is nothing here (it does not read the sums then)
        const int ncol = !p.split_q ? min(32, p.ncols - colblk * 32)
                                    : (colblk == 0 ? p.g : min(32, (p.Q - 1) * p.g - (colblk - 1) * 32));
        if (tid < ncol) {
            const int64_t slot = (((int64_t)bz * p.Hkv + kvh) * p.nsplit + split) * p.ncols_pad + colblk * 32 + tid;
            p.ws_ml[slot * 2] = -INFINITY;
            p.ws_ml[slot * 2 + 1] = 0.f;
        }
        continue;
    }

    // column (query token qi, head gi of the group) owned by this lane
    int qi, gi;
    const bool col_ok = ksa_decode_column(p, colblk, lq, qi, gi);
    if (!col_ok) qi = 0, gi = 0;
    const int head = kvh * p.g + gi;

    u32x4 qf[KS];
    {
        const uint16_t* qp = p.q + bz * p.q_bs + head * p.q_hs + qi * p.q_qs + 8 * lh;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            u32x4 z = {0u, 0u, 0u, 0u};
            qf[s] = col_ok ? *reinterpret_cast<const u32x4*>(qp + 16 * s) : z;
        }
    }

    const uint16_t* kbase = p.k + bz * p.k_bs + kvh * p.k_hs;
    const uint16_t* vbase = p.v + bz * p.v_bs + kvh * p.v_hs;
    const int last_row = max(r_end - 1, r_begin);

    u32x4 kreg[KLD];
    u32x4 vreg[KLD];

    // K/V rows are read once and never again: non-temporal loads
    auto load_piece = [&](int row0, int i) {
        const int u = lane + 64 * i;
        const int row = min(row0 + u / CPR, last_row);
        kreg[i] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4*>(kbase + (int64_t)row * p.k_rs + 8 * (u % CPR)));
        vreg[i] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4*>(vbase + (int64_t)row * p.v_rs + 8 * (u % CPR)));
    };
    auto load_tile = [&](int row0) {
#pragma unroll
        for (int i = 0; i < KLD; ++i) load_piece(row0, i);
    };

    floatx16 oacc[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[b][i] = 0.f;
    float m_run = -INFINITY;  // in raw score units
    float l_run = 0.f;
    const float c2 = p.scale_log2;

    int row0 = s0 + wave * kRows;
    if (row0 < s1) load_tile(row0);

    for (; row0 < s1; row0 += kWaves * kRows) {
        ksa_wave_lds_fence();
        // registers -> LDS, and each register pair is refilled with the next tile right behind
        // its store, so the loads of the next tile are in flight for the whole step
        const int next = row0 + kWaves * kRows;
        const bool has_next = next < s1;
#pragma unroll
        for (int i = 0; i < KLD; ++i) {
            const int u = lane + 64 * i;
            *reinterpret_cast<u32x4*>(Kw + (u / CPR) * KROW + 8 * (u % CPR)) = kreg[i];
            *reinterpret_cast<u32x4*>(Vw + (u / CPR) * VROW + 8 * (u % CPR)) = vreg[i];
            if (has_next) load_piece(next, i);
        }
        ksa_wave_lds_fence();

        floatx16 sacc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const u32x4 a = *reinterpret_cast<const u32x4*>(Kw + lq * KROW + 16 * s + 8 * lh);
            sacc = Ops::mfma(a, qf[s], sacc);
        }
        if (row0 + kRows > s1) {  // tail tile: rows past the slice end do not exist
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int r = row0 + 8 * (i / 4) + 4 * lh + (i % 4);
                if (r >= s1) sacc[i] = -INFINITY;
            }
        }
        float mloc = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, sacc[i]);
        mloc = fmaxf(mloc, ksa_xor32(mloc));
        const float m_new = fmaxf(m_run, mloc);  // finite: every tile has >= 1 real row
        const float alpha = ksa_exp2((m_run - m_new) * c2);
        const float mc = m_new * c2;
        m_run = m_new;
        float rowsum = 0.f;
        u32x4 pf[2];
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const float p0 = ksa_exp2(fmaf(sacc[i], c2, -mc));
            const float p1 = ksa_exp2(fmaf(sacc[i + 1], c2, -mc));
            rowsum += p0 + p1;
            pf[i / 8][(i % 8) / 2] = Ops::pack2(p0, p1);
        }
        l_run = l_run * alpha + rowsum;
        if (__any(alpha != 1.f)) {
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[b][i] *= alpha;
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int b = 0; b < DB; ++b) {
                const u32x4 a = ksa_read_vt_frag<VROW>(Vw, ks, b, lq, lh);
                oacc[b] = Ops::mfma(a, pf[ks], oacc[b]);
            }
    }

    // ---- merge the four waves through LDS ----
    l_run += ksa_xor32(l_run);
    __syncthreads();  // staging areas are dead from here on
    float* mg = reinterpret_cast<float*>(smem);  // [wave][col 32][D + 2]
    {
        float* row = mg + (wave * 32 + lq) * (D + 2);
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) row[32 * b + 8 * (i / 4) + 4 * lh + (i % 4)] = oacc[b][i];
        if (lh == 0) {
            row[D] = m_run * c2;  // log2 units; -inf if this wave saw no row
            row[D + 1] = l_run;
        }
    }
    __syncthreads();
    const int ncol_here = !p.split_q ? min(32, p.ncols - colblk * 32)
                                     : (colblk == 0 ? p.g : min(32, (p.Q - 1) * p.g - (colblk - 1) * 32));
    for (int e = tid; e < ncol_here * D; e += kThreads) {
        const int c = e / D, d = e % D;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) mx = fmaxf(mx, mg[(w * 32 + c) * (D + 2) + D]);
        float acc = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float* row = mg + (w * 32 + c) * (D + 2);
            const float f = (row[D] == -INFINITY) ? 0.f : ksa_exp2(row[D] - mx);
            acc += row[d] * f;
            l += row[D + 1] * f;
        }
        const int cg = colblk * 32 + c;
        if (p.nsplit == 1) {
            int oq, og;
            ksa_decode_column(p, colblk, c, oq, og);
            const float val = l > 0.f ? acc / l : 0.f;
            uint16_t* op = p.out + bz * p.o_bs + oq * p.o_qs + (kvh * p.g + og) * p.o_hs + d;
            const uint32_t pk = Ops::pack2(val, 0.f);
            *op = (uint16_t)(pk & 0xffffu);
        } else {
            const int64_t slot = (((int64_t)bz * p.Hkv + kvh) * p.nsplit + split) * p.ncols_pad + cg;
            p.ws_o[slot * D + d] = acc;
            if (d == 0) {
                p.ws_ml[slot * 2] = mx;
                p.ws_ml[slot * 2 + 1] = l;
            }
        }
    }
    }  // column blocks of this workgroup
}

// second stage: merge the splits of one (sequence, kv head, column)
template <typename T, int D>
__global__ __launch_bounds__(D) void ksa_decode_merge_kernel(const DecodeParams p) {
    using Ops = KsaOps<T>;
    const int oq = blockIdx.x / p.g, og = blockIdx.x % p.g;  // logical column: query token, head in the group
    const int cg = ksa_decode_slot(p, oq, og);
    const int kvh = blockIdx.y;
    const int bz = blockIdx.z;
    const int d = threadIdx.x;
    const int64_t base = (((int64_t)bz * p.Hkv + kvh) * p.nsplit) * p.ncols_pad + cg;
    // the loads of eight splits are requested together (two passes: maximum, then weighted sums)
    float mx = -INFINITY;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        float m[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) m[u] = p.ws_ml[(base + (int64_t)min(s0 + u, p.nsplit - 1) * p.ncols_pad) * 2];
#pragma unroll
        for (int u = 0; u < 8; ++u) mx = fmaxf(mx, m[u]);
    }
    float acc = 0.f, l = 0.f;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        float m[8], ls[8], o[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int64_t slot = base + (int64_t)min(s0 + u, p.nsplit - 1) * p.ncols_pad;
            m[u] = p.ws_ml[slot * 2];
            ls[u] = p.ws_ml[slot * 2 + 1];
            o[u] = p.ws_o[slot * D + d];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (s0 + u < p.nsplit) {
                // (an empty slice leaves its sums unwritten: nothing of it may enter, not even times zero)
                const bool some = m[u] != -INFINITY;
                const float f = some ? ksa_exp2(m[u] - mx) : 0.f;
                acc = some ? fmaf(o[u], f, acc) : acc;
                l = some ? fmaf(ls[u], f, l) : l;
            }
        }
    }
    const float val = l > 0.f ? acc / l : 0.f;
    uint16_t* op = p.out + bz * p.o_bs + oq * p.o_qs + (kvh * p.g + og) * p.o_hs + d;
    *op = (uint16_t)(Ops::pack2(val, 0.f) & 0xffffu);
}

template <typename T, int D>
int launch(const DecodeParams& p, int batch, hipStream_t stream) {
    const int colblks = p.split_q ? 1 : p.ncols_pad / 32;  // (boundary form: a workgroup walks its column blocks)
    dim3 grid(p.nsplit, p.Hkv * colblks, batch);
    hipLaunchKernelGGL((ksa_decode_kernel<T, D>), grid, dim3(kThreads), 0, stream, p);
    if (p.nsplit > 1) {
        dim3 g2(p.ncols, p.Hkv, batch);
        hipLaunchKernelGGL((ksa_decode_merge_kernel<T, D>), g2, dim3(D), 0, stream, p);
    }
    return ksa_check_launch();
}

int pad_cols(int ncols) { return (ncols + 31) / 32 * 32; }
// column slots of the chunk-boundary form: a block of 32 for the text token, the summary tokens behind it
int pad_cols_boundary(int Q, int g) { return 32 + pad_cols((Q - 1) * g); }

}  // namespace

extern "C" size_t ksa_decode_workspace_bytes(int batch, int Hq, int Hkv, int Q, int D, int nsplit) {
    if (nsplit <= 1 || batch <= 0 || Hkv <= 0 || Hq % Hkv != 0) return 0;
    const size_t cols = (size_t)pad_cols(Q * (Hq / Hkv));
    return (size_t)batch * Hkv * nsplit * cols * (D + 2) * sizeof(float);
}

// Heuristic number of splits: at least two workgroups per CU of the current device (256 CUs
// assumed when no device can be asked), but never splits shorter than 256 rows.
extern "C" int ksa_decode_auto_splits(int batch, int Hkv, int max_rows) {
    if (batch <= 0 || Hkv <= 0 || max_rows <= 0) return 1;
    const int units = batch * Hkv;
    const int want = 2 * ksa_cu_count_or(256);
    int n = (want + units - 1) / units;
    const int cap = max_rows / 256 > 1 ? max_rows / 256 : 1;
    if (n > cap) n = cap;
    if (n > 64) n = 64;
    return n < 1 ? 1 : n;
}

namespace {

int decode_fwd_impl(const void* q, const void* kcache, const void* vcache, void* out,
                    const int32_t* start, const int32_t* end, int start0, int end0, int batch, int Hq,
                    int Hkv, int Q, int D, int dtype, const int64_t* q_strides,
                    const int64_t* k_strides, const int64_t* v_strides, const int64_t* out_strides,
                    float scale, int nsplit, void* workspace, size_t workspace_bytes, void* stream,
                    bool boundary = false, const int32_t* start2 = nullptr, const int32_t* end2 = nullptr,
                    int start20 = 0, int end20 = 0) {
    if (!q || !kcache || !vcache || !out || !q_strides || !k_strides || !v_strides || !out_strides)
        return KSA_ERR_NULL;
    if ((start == nullptr) != (end == nullptr)) return KSA_ERR_NULL;
    if (boundary) {
        if ((start2 == nullptr) != (end2 == nullptr)) return KSA_ERR_NULL;
        if (Q < 2 || Hkv <= 0 || Hq % Hkv != 0 || Hq / Hkv > 32) return KSA_ERR_INVALID;
        if (!start2 && (start20 < 0 || end20 <= start20)) return KSA_ERR_INVALID;
    }
    if (batch <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || Q <= 0 || nsplit < 1) return KSA_ERR_INVALID;
    if (!start && (start0 < 0 || end0 <= start0)) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kcache) |
         reinterpret_cast<uintptr_t>(vcache)) & 15)
        return KSA_ERR_ALIGN;
    for (int i = 0; i < 3; ++i)
        if ((q_strides[i] % 8) || (k_strides[i] % 8) || (v_strides[i] % 8)) return KSA_ERR_ALIGN;

    DecodeParams p{};
    p.q = (const uint16_t*)q;
    p.k = (const uint16_t*)kcache;
    p.v = (const uint16_t*)vcache;
    p.out = (uint16_t*)out;
    p.start = start;
    p.end = end;
    p.start0 = start0;
    p.end0 = end0;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.g = Hq / Hkv;
    p.Q = Q;
    p.ncols = Q * p.g;
    p.ncols_pad = boundary ? pad_cols_boundary(Q, p.g) : pad_cols(p.ncols);
    p.split_q = boundary ? 1 : 0;
    p.start2 = start2, p.end2 = end2, p.start20 = start20, p.end20 = end20;
    p.nsplit = nsplit;
    p.q_bs = q_strides[0], p.q_hs = q_strides[1], p.q_qs = q_strides[2];
    p.k_bs = k_strides[0], p.k_hs = k_strides[1], p.k_rs = k_strides[2];
    p.v_bs = v_strides[0], p.v_hs = v_strides[1], p.v_rs = v_strides[2];
    p.o_bs = out_strides[0], p.o_qs = out_strides[1], p.o_hs = out_strides[2];
    p.scale_log2 = scale * 1.4426950408889634f;
    if (nsplit > 1) {
        const size_t need = (size_t)batch * Hkv * nsplit * p.ncols_pad * (D + 2) * sizeof(float);
        if (!workspace || workspace_bytes < need) return KSA_ERR_WORKSPACE;
        p.ws_o = (float*)workspace;
        p.ws_ml = p.ws_o + (size_t)batch * Hkv * nsplit * p.ncols_pad * D;
    }
    hipStream_t st = (hipStream_t)stream;
    if (dtype == KSA_DTYPE_BF16) {
        if (D == 128) return launch<KsaBf16, 128>(p, batch, st);
        if (D == 64) return launch<KsaBf16, 64>(p, batch, st);
        if (D == 256) return launch<KsaBf16, 256>(p, batch, st);
    } else {
        if (D == 128) return launch<KsaF16, 128>(p, batch, st);
        if (D == 64) return launch<KsaF16, 64>(p, batch, st);
        if (D == 256) return launch<KsaF16, 256>(p, batch, st);
    }
    return KSA_ERR_UNSUPPORTED;
}

// ---- scratch of the entry point that allocates nothing ----
// Split-K partials of ksa_decode_fwd_noalloc live in this array instead of a caller-provided
// workspace.  Every GPU the library is loaded on holds its own copy at its own address; the
// array's name is only a host-side handle, so the device address is asked for once per device
// (hipGetSymbolAddress) and kept.
constexpr size_t kNoAllocScratchBytes = KSA_DECODE_NOALLOC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the current device, or null
void* noalloc_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

}  // namespace

extern "C" int ksa_decode_fwd(const void* q, const void* kcache, const void* vcache, void* out,
                              const int32_t* start, const int32_t* end, int start0, int end0,
                              int batch, int Hq, int Hkv, int Q, int D, int dtype,
                              const int64_t* q_strides, const int64_t* k_strides,
                              const int64_t* v_strides, const int64_t* out_strides, float scale,
                              int nsplit, void* workspace, size_t workspace_bytes, void* stream) {
    return decode_fwd_impl(q, kcache, vcache, out, start, end, start0, end0, batch, Hq, Hkv, Q, D, dtype,
                           q_strides, k_strides, v_strides, out_strides, scale, nsplit, workspace,
                           workspace_bytes, stream);
}

// Chunk-boundary step (HF:831-876): the chunk's last text token and its summary tokens in one launch.
// Query token 0 attends rows [text_start, text_end) (the slice of get_attention_kv after update_text,
// HF:844-856), query tokens 1 .. Q - 1 attend [sum_start, sum_end) (the [own summaries | chunk] rows of
// get_summary_attention_kv, HF:858-870), un-masked both, as the reference's two calls of its decode
// attention function do; out [batch, Q, Hq, D] is their torch.cat (HF:875).
extern "C" size_t ksa_decode_boundary_workspace_bytes(int batch, int Hq, int Hkv, int Q, int D, int nsplit) {
    if (nsplit <= 1 || batch <= 0 || Hkv <= 0 || Hq % Hkv != 0 || Q < 2) return 0;
    return (size_t)batch * Hkv * nsplit * (size_t)pad_cols_boundary(Q, Hq / Hkv) * (D + 2) * sizeof(float);
}

extern "C" int ksa_decode_boundary_fwd(const void* q, const void* kcache, const void* vcache, void* out,
                                       const int32_t* text_start, const int32_t* text_end, int text_start0,
                                       int text_end0, const int32_t* sum_start, const int32_t* sum_end,
                                       int sum_start0, int sum_end0, int batch, int Hq, int Hkv, int Q, int D,
                                       int dtype, const int64_t* q_strides, const int64_t* k_strides,
                                       const int64_t* v_strides, const int64_t* out_strides, float scale,
                                       int nsplit, void* workspace, size_t workspace_bytes, void* stream) {
    return decode_fwd_impl(q, kcache, vcache, out, text_start, text_end, text_start0, text_end0, batch, Hq, Hkv, Q, D,
                           dtype, q_strides, k_strides, v_strides, out_strides, scale, nsplit, workspace,
                           workspace_bytes, stream, true, sum_start, sum_end, sum_start0, sum_end0);
}

extern "C" size_t ksa_decode_noalloc_max_workspace_bytes(void) { return kNoAllocScratchBytes; }

// ksa_decode_fwd without the workspace arguments: the split-K partials go to the library's own
// fixed device array.  Nothing is allocated, freed or synchronised here; the kernels are the
// ones ksa_decode_fwd launches and receive the array's device address as their workspace.
// Every (sequence, kv head, split, column) slot the merge kernel reads is written by the
// decode kernel of the same call, so nothing has to be cleared between calls.
extern "C" int ksa_decode_fwd_noalloc(const void* q, const void* kcache, const void* vcache, void* out,
                                      const int32_t* start, const int32_t* end, int start0, int end0,
                                      int batch, int Hq, int Hkv, int Q, int D, int dtype,
                                      const int64_t* q_strides, const int64_t* k_strides,
                                      const int64_t* v_strides, const int64_t* out_strides,
                                      float scale, int nsplit, void* stream) {
    if (nsplit <= 1)
        return decode_fwd_impl(q, kcache, vcache, out, start, end, start0, end0, batch, Hq, Hkv, Q, D,
                               dtype, q_strides, k_strides, v_strides, out_strides, scale, nsplit,
                               nullptr, 0, stream);
    if (batch <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || Q <= 0) return KSA_ERR_INVALID;
    const size_t need = ksa_decode_workspace_bytes(batch, Hq, Hkv, Q, D, nsplit);
    if (need > kNoAllocScratchBytes) return KSA_ERR_WORKSPACE;
    void* ws = noalloc_scratch();
    if (!ws) return KSA_ERR_LAUNCH;
    return decode_fwd_impl(q, kcache, vcache, out, start, end, start0, end0, batch, Hq, Hkv, Q, D, dtype,
                           q_strides, k_strides, v_strides, out_strides, scale, nsplit, ws,
                           kNoAllocScratchBytes, stream);
}
