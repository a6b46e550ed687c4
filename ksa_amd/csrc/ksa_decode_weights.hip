// Attention probabilities of the decode step, for callers that ask for them (gfx950).
//
// The reference has a second decode attention function that returns the probabilities next to
// the output:
//   examples/pretrain/hf_template/modeling_qwen3sa.py:569-588 (eager_attention_forward), selected
//   at :643-646 when config._attn_implementation == "eager":
//     w = softmax(q K^T * scaling (+ mask), dim=-1, dtype=float32).to(q.dtype)     [b, Hq, q_len, L]
// The output itself comes from ksa_decode_fwd; this file only makes w, in two small launches:
//   1. scores: S^T = K Q^T per 32-row tile with the MFMA formulation of the decode kernel (the g
//      query heads of a kv head and the query tokens are the columns, so K is read once per kv
//      head), times the scale, as fp32 into a workspace [b, Hq, Q, Lp];
//   2. row soft-max in fp32 (maximum, sum, normalise; optional additive mask), rounded to the
//      16-bit type; positions past a sequence's range get 0.
// K is read a second time for this (the decode kernel does not keep its scores): the price of
// asking for the probabilities, as in the reference, whose eager path is its slow path.
#include <hip/hip_runtime.h>
#include <math.h>

#include "ksa_api_internal.h"
#include "ksa_tile.h"

namespace {

struct WeightsParams {
    const uint16_t* q;
    const uint16_t* k;
    uint16_t* w;           // [b, Hq, Q, Lw]
    const uint16_t* mask;  // additive, 16-bit, element strides below (0 = broadcast); may be null
    float* sc;             // workspace [b, Hq, Q, Lp]
    const int32_t* start;
    const int32_t* end;
    int start0, end0;
    int Hq, Hkv, g, Q, ncols;
    int Lw, Lp;
    int64_t q_bs, q_hs, q_qs;
    int64_t k_bs, k_hs, k_rs;
    int64_t m_bs, m_hs, m_qs, m_ls;
    float scale;
};

constexpr int kRowsPerWave = 32;
constexpr int kWavesPerBlock = 4;

// grid: (row blocks of 128, kv head x column block, sequence)
template <typename T, int D>
__global__ __launch_bounds__(256) void ksa_decode_scores_kernel(const WeightsParams p) {
    using Ops = KsaOps<T>;
    constexpr int KS = D / 16;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int lq = lane & 31, lh = lane >> 5;
    const int colblk = blockIdx.y / p.Hkv;
    const int kvh = blockIdx.y % p.Hkv;
    const int bz = blockIdx.z;
    const int r_begin = p.start ? p.start[bz] : p.start0;
    const int r_end = p.end ? p.end[bz] : p.end0;
    const int L = min(max(r_end - r_begin, 0), p.Lw);  // (a longer range is cut at the width of the output)
    const int j0 = (blockIdx.x * kWavesPerBlock + wave) * kRowsPerWave;  // first position of this wave's tile
    if (j0 >= L) return;

    const int col = colblk * 32 + lq;
    const bool col_ok = col < p.ncols;
    const int qi = col_ok ? col / p.g : 0;
    const int gi = col_ok ? col % p.g : 0;
    const int head = kvh * p.g + gi;
    // A operand: lane (lq, lh) holds key row lq, elements 16 s + 8 lh .. + 8 of the head row
    const int krow = r_begin + min(j0 + lq, L - 1);
    const uint16_t* kp = p.k + bz * p.k_bs + kvh * p.k_hs + (int64_t)krow * p.k_rs + 8 * lh;
    const uint16_t* qp = p.q + bz * p.q_bs + head * p.q_hs + qi * p.q_qs + 8 * lh;
    u32x4 a[KS], b[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        a[s] = *reinterpret_cast<const u32x4*>(kp + 16 * s);
        const u32x4 z = {0u, 0u, 0u, 0u};
        b[s] = col_ok ? *reinterpret_cast<const u32x4*>(qp + 16 * s) : z;
    }
    floatx16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) acc = Ops::mfma(a[s], b[s], acc);
    if (!col_ok) return;
    // C layout: register i of lane (lq, lh) is key 8 (i / 4) + 4 lh + i % 4 of the tile, column lq
    float* dst = p.sc + (((int64_t)bz * p.Hq + head) * p.Q + qi) * p.Lp;
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
        const int j = j0 + 8 * i4 + 4 * lh;
        if (j + 3 < L) {
            float4 v4 = {acc[4 * i4] * p.scale, acc[4 * i4 + 1] * p.scale, acc[4 * i4 + 2] * p.scale,
                         acc[4 * i4 + 3] * p.scale};
            *reinterpret_cast<float4*>(dst + j) = v4;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (j + e < L) dst[j + e] = acc[4 * i4 + e] * p.scale;
        }
    }
}

__device__ __forceinline__ float block_reduce(float v, bool is_max, float* red) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float o = __shfl_xor(v, m);
        v = is_max ? fmaxf(v, o) : v + o;
    }
    __syncthreads();  // (red may still be read from the previous reduction)
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) r = is_max ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

template <typename T>
struct Cvt16;
template <>
struct Cvt16<KsaBf16> {
    static __device__ __forceinline__ float up(uint16_t x) { return __uint_as_float((uint32_t)x << 16); }
};
template <>
struct Cvt16<KsaF16> {
    static __device__ __forceinline__ float up(uint16_t x) {
        return (float)__builtin_bit_cast(_Float16, x);
    }
};

// grid: (query token, head, sequence); one workgroup per row of probabilities
template <typename T>
__global__ __launch_bounds__(256) void ksa_decode_softmax_rows_kernel(const WeightsParams p) {
    using Ops = KsaOps<T>;
    __shared__ float red[4];
    const int qi = blockIdx.x, head = blockIdx.y, bz = blockIdx.z;
    const int r_begin = p.start ? p.start[bz] : p.start0;
    const int r_end = p.end ? p.end[bz] : p.end0;
    const int L = min(max(r_end - r_begin, 0), p.Lw);
    const float* src = p.sc + (((int64_t)bz * p.Hq + head) * p.Q + qi) * p.Lp;
    uint16_t* dst = p.w + (((int64_t)bz * p.Hq + head) * p.Q + qi) * p.Lw;
    const uint16_t* mk = p.mask ? p.mask + bz * p.m_bs + head * p.m_hs + qi * p.m_qs : nullptr;
    auto score = [&](int j) { return src[j] + (mk ? Cvt16<T>::up(mk[(int64_t)j * p.m_ls]) : 0.f); };
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < L; j += 256) mx = fmaxf(mx, score(j));
    mx = block_reduce(mx, true, red);
    float sum = 0.f;
    for (int j = threadIdx.x; j < L; j += 256) sum += expf(score(j) - mx);
    sum = block_reduce(sum, false, red);
    // a row whose every position is masked to -inf has no defined soft-max (the reference gives NaN)
    const float inv = 1.f / sum;
    for (int j = threadIdx.x; j < p.Lw; j += 256) {
        const float v = j < L ? expf(score(j) - mx) * inv : 0.f;
        dst[j] = (uint16_t)(Ops::pack2(v, 0.f) & 0xffffu);
    }
}

template <typename T, int D>
int launch_weights(const WeightsParams& p, int batch, int max_len, hipStream_t st) {
    const int colblks = (p.ncols + 31) / 32;
    const int rowblks = (max_len + kRowsPerWave * kWavesPerBlock - 1) / (kRowsPerWave * kWavesPerBlock);
    hipLaunchKernelGGL((ksa_decode_scores_kernel<T, D>), dim3(rowblks, p.Hkv * colblks, batch), dim3(256), 0, st, p);
    hipLaunchKernelGGL((ksa_decode_softmax_rows_kernel<T>), dim3(p.Q, p.Hq, batch), dim3(256), 0, st, p);
    return ksa_check_launch();
}

}  // namespace

// fp32 scores [batch, Hq, Q, L rounded up to a multiple of 4]
extern "C" size_t ksa_decode_weights_workspace_bytes(int batch, int Hq, int Q, int L) {
    if (batch <= 0 || Hq <= 0 || Q <= 0 || L <= 0) return 0;
    return (size_t)batch * Hq * Q * (size_t)((L + 3) / 4 * 4) * sizeof(float);
}

extern "C" int ksa_decode_weights(const void* q, const void* kcache, void* weights, const void* mask,
                                  const int32_t* start, const int32_t* end, int start0, int end0, int batch, int Hq,
                                  int Hkv, int Q, int D, int dtype, int L, const int64_t* q_strides,
                                  const int64_t* k_strides, const int64_t* mask_strides, float scale, void* workspace,
                                  size_t workspace_bytes, void* stream) {
    if (!q || !kcache || !weights || !q_strides || !k_strides || !workspace) return KSA_ERR_NULL;
    if ((start == nullptr) != (end == nullptr)) return KSA_ERR_NULL;
    if (mask && !mask_strides) return KSA_ERR_NULL;
    if (batch <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || Q <= 0 || L <= 0) return KSA_ERR_INVALID;
    if (!start && (start0 < 0 || end0 <= start0 || end0 - start0 > L)) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kcache) | reinterpret_cast<uintptr_t>(workspace)) & 15)
        return KSA_ERR_ALIGN;
    for (int i = 0; i < 3; ++i)
        if ((q_strides[i] % 8) || (k_strides[i] % 8)) return KSA_ERR_ALIGN;
    if (workspace_bytes < ksa_decode_weights_workspace_bytes(batch, Hq, Q, L)) return KSA_ERR_WORKSPACE;
    WeightsParams p{};
    p.q = (const uint16_t*)q;
    p.k = (const uint16_t*)kcache;
    p.w = (uint16_t*)weights;
    p.mask = (const uint16_t*)mask;
    p.sc = (float*)workspace;
    p.start = start, p.end = end, p.start0 = start0, p.end0 = end0;
    p.Hq = Hq, p.Hkv = Hkv, p.g = Hq / Hkv, p.Q = Q, p.ncols = Q * p.g;
    p.Lw = L, p.Lp = (L + 3) / 4 * 4;
    p.q_bs = q_strides[0], p.q_hs = q_strides[1], p.q_qs = q_strides[2];
    p.k_bs = k_strides[0], p.k_hs = k_strides[1], p.k_rs = k_strides[2];
    if (mask) p.m_bs = mask_strides[0], p.m_hs = mask_strides[1], p.m_qs = mask_strides[2], p.m_ls = mask_strides[3];
    p.scale = scale;
    hipStream_t st = (hipStream_t)stream;
    // (the scores kernel covers positions [0, L); a sequence whose range is longer is cut at L by the
    // soft-max kernel, which the Python mirror never lets happen)
    if (dtype == KSA_DTYPE_BF16) {
        if (D == 128) return launch_weights<KsaBf16, 128>(p, batch, L, st);
        if (D == 64) return launch_weights<KsaBf16, 64>(p, batch, L, st);
        if (D == 256) return launch_weights<KsaBf16, 256>(p, batch, L, st);
    } else {
        if (D == 128) return launch_weights<KsaF16, 128>(p, batch, L, st);
        if (D == 64) return launch_weights<KsaF16, 64>(p, batch, L, st);
        if (D == 256) return launch_weights<KsaF16, 256>(p, batch, L, st);
    }
    return KSA_ERR_UNSUPPORTED;
}
