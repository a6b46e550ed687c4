// y = x W^T for a handful of rows (decode steps: one row per sequence), gfx950.
//
// The projections of a decode step (examples/pretrain/hf_template/modeling_qwen3sa.py: q/k/v
// and o projections :628-641, :879; the MLP :507-514; lm_head :1338, :1395) multiply at most a
// few rows by a weight matrix that has to be streamed from HBM once: the step is bound by the
// weight bytes.  A wave owns 16 output columns (16 rows of W, each K elements long); a weight
// fragment goes from global memory straight into the A operand of a 16x16x32 MFMA (lane = (row
// of W, quarter of the 32-wide K step): 16 contiguous bytes per lane, 64 contiguous bytes per
// row and instruction), the rows of x, staged in LDS, are the B operand.  With more than one K
// split per column tile the fp32 partial sums go to a workspace and a second kernel adds and
// rounds them.
#include <hip/hip_runtime.h>

#include "ksa_api_internal.h"
#include "ksa_cvt.h"
#include "ksa_rows_mfma.h"

namespace {

struct GemmParams {
    const uint16_t* x;   // [M, K], row stride xs
    const uint16_t* w;   // [N, K], row stride ws
    uint16_t* out;       // [M, N], row stride os
    float* part;         // [ksplit, 16, N] when ksplit > 1
    int64_t xs, ws, os;
    int M, N, K, ksplit;
};

// grid: (tiles of 64 output columns, K splits); block: 4 waves, each 16 columns over the whole K
// slice.  Per chunk of 512 K elements a wave first requests its 16 weight fragments (16 x 16
// bytes per lane in flight), the workgroup copies the chunk of x into LDS once, and the MFMAs
// then take their B operands from there: x is fetched once per 64 columns instead of once per
// wave and step, which is what held a first version of this kernel at 60 % of the rate below.
template <typename T>
__global__ __launch_bounds__(256) void ksa_gemm_rows_kernel(const GemmParams p) {
    using C = KsaCvt<T>;
    __shared__ __attribute__((aligned(16))) unsigned char xs[2][16 * kRowB];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r = lane & 15;   // row of W inside the tile (A operand) / row of x (B operand)
    const int kq = lane >> 4;  // which 8 of the 32 K elements of a step
    const int n0 = (blockIdx.x * 4 + wave) * 16;
    const int steps = p.K / 32;
    const int per_split = (steps + p.ksplit - 1) / p.ksplit;
    const int s_begin = blockIdx.y * per_split;
    const int s_end = min(steps, s_begin + per_split);

    const int nrow = min(n0 + r, p.N - 1);
    const uint16_t* wp = p.w + (int64_t)nrow * p.ws + 8 * kq;
    // rows of x beyond M repeat the last one: their columns of the product are never stored
    const int xrow = min(r, p.M - 1);

    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    int buf = 0;
    for (int c0 = s_begin; c0 < s_end; c0 += kChunkSteps) {
        const int nst = min(kChunkSteps, s_end - c0);
        u32x4 a[kChunkSteps];
#pragma unroll
        for (int u = 0; u < kChunkSteps; ++u) a[u] = *reinterpret_cast<const u32x4*>(wp + 32 * min(c0 + u, s_end - 1));
        // x[0:M][32 c0 .. 32 (c0 + nst)) -> LDS, 16 bytes per thread and pass
        for (int e = threadIdx.x; e < p.M * (kChunkK / 8); e += 256) {
            const int m = e / (kChunkK / 8), j = e % (kChunkK / 8);
            if (j < nst * 4)
                *reinterpret_cast<u32x4*>(xs[buf] + m * kRowB + 16 * j) =
                    *reinterpret_cast<const u32x4*>(p.x + (int64_t)m * p.xs + 32 * c0 + 8 * j);
        }
        // (one barrier per chunk is enough with two buffers: nobody passes the next chunk's
        // barrier before everybody has finished reading this one)
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kChunkSteps; ++u) {
            if (u < nst) {
                const u32x4 b = *reinterpret_cast<const u32x4*>(xs[buf] + xrow * kRowB + 64 * u + 16 * kq);
                acc = mfma16<T>(a[u], b, acc);
            }
        }
        buf ^= 1;
    }
    // C layout of the 16x16 tile: lane holds column (row of x) lane % 16, rows (of W) 4 * (lane / 16) + i
    if (r < p.M) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + 4 * kq + i;
            if (n < p.N) {
                if (p.ksplit == 1) p.out[(int64_t)r * p.os + n] = C::down(acc[i]);
                else p.part[((int64_t)blockIdx.y * 16 + r) * p.N + n] = acc[i];
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void ksa_gemm_rows_reduce_kernel(const GemmParams p) {
    using C = KsaCvt<T>;
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (int64_t)p.M * p.N) return;
    const int m = (int)(e / p.N), n = (int)(e % p.N);
    float v = 0.f;
    for (int sp = 0; sp < p.ksplit; ++sp) v += p.part[((int64_t)sp * 16 + m) * p.N + n];
    p.out[(int64_t)m * p.os + n] = C::down(v);
}

template <typename T>
int launch_gemm(const GemmParams& p, hipStream_t st) {
    dim3 grid((p.N + 63) / 64, p.ksplit);
    hipLaunchKernelGGL(ksa_gemm_rows_kernel<T>, grid, dim3(256), 0, st, p);
    if (p.ksplit > 1 && p.out) {
        const int64_t n = (int64_t)p.M * p.N;
        hipLaunchKernelGGL(ksa_gemm_rows_reduce_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p);
    }
    return ksa_check_launch();
}

// ---- gate | up projection with the MLP's activation folded in ----
// out[m][n] = round(SiLU(round(x . w[n]))) * round(x . w[I + n]) for the few rows of a decode step
// (examples/pretrain/hf_template/modeling_qwen3sa.py:507-514, act_fn(gate_proj(x)) * up_proj(x), with
// the rounding points of its 16-bit tensor ops).  A workgroup owns 16 columns of the hidden vector
// and the whole of K: wave (h, s) multiplies the chunks s, s + S, ... of 512 elements of K with the
// gate (h = 0) or up (h = 1) rows of w, where S = min(chunks of K, 8) - at K = 2560 ten waves with
// one chunk each and no loop, every weight load of the workgroup in flight at once.  x is staged in
// LDS once, whole; the partial sums of the 2 S waves meet in LDS (in place of x), and the first 256
// threads finish one output each.  Product, activation and multiply are one launch and no partial
// sums travel through memory.
struct GateUpParams {
    const uint16_t* x;   // [M, K]
    const uint16_t* w;   // [2 I, K]: gate rows, then up rows
    uint16_t* out;       // [M, I]
    int64_t xs, ws, os;
    int M, I, K, S;      // S: K slices = waves per half
};
constexpr int kGateUpMaxSlices = 8;

static inline size_t gate_up_lds_bytes(int M, int K, int S) {
    const size_t xb = (size_t)M * (K + 8) * 2;
    const size_t rb = (size_t)2 * S * 16 * 17 * sizeof(float);
    return xb > rb ? xb : rb;
}

template <typename T>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void ksa_gemm_gate_up_silu_kernel(const GateUpParams p) {
    using C = KsaCvt<T>;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r = lane & 15;
    const int kq = lane >> 4;
    const int half = wave / p.S;  // 0: gate rows of w, 1: up rows
    const int slice = wave - half * p.S;
    const int n0 = blockIdx.x * 16;
    const int steps = p.K / 32;
    const int chunks = (steps + kChunkSteps - 1) / kChunkSteps;
    const int rowb = (p.K + 8) * 2;
    const uint16_t* wp = p.w + ((int64_t)half * p.I + min(n0 + r, p.I - 1)) * p.ws + 8 * kq;
    const int xrow = min(r, p.M - 1);

    // eight K steps of weights in flight per wave (32 registers): with at most 64 registers a SIMD
    // holds eight waves, so three workgroups of ten waves per CU and the whole grid of a 4B-shape
    // MLP (608 workgroups) is resident at once
    constexpr int kB = 8;
    u32x4 a[kB];
    auto load_steps = [&](int s0) {
#pragma unroll
        for (int u = 0; u < kB; ++u) a[u] = *reinterpret_cast<const u32x4*>(wp + 32 * min(s0 + u, steps - 1));
    };
    load_steps(slice * kChunkSteps);  // in flight while x is staged (every slice has a first chunk: S <= chunks)
    const int per_row = p.K / 8;
    for (int e = threadIdx.x; e < p.M * per_row; e += blockDim.x) {
        const int m = e / per_row, j = e - m * per_row;
        *reinterpret_cast<u32x4*>(lds + m * rowb + 16 * j) =
            *reinterpret_cast<const u32x4*>(p.x + (int64_t)m * p.xs + 8 * j);
    }
    __syncthreads();
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int c = slice; c < chunks; c += p.S) {
        for (int s0 = c * kChunkSteps; s0 < min((c + 1) * kChunkSteps, steps); s0 += kB) {
            if (s0 != slice * kChunkSteps) load_steps(s0);
            const int nst = min(kB, steps - s0);
            const unsigned char* xb = lds + xrow * rowb + s0 * 64 + 16 * kq;
#pragma unroll
            for (int u = 0; u < kB; ++u) {
                if (u < nst) acc = mfma16<T>(a[u], *reinterpret_cast<const u32x4*>(xb + 64 * u), acc);
            }
        }
    }
    __syncthreads();  // x is no longer read: its place takes the partial sums
    // C layout of the 16x16 tile: lane holds row of x lane % 16, columns 4 * (lane / 16) + i
    float* red = reinterpret_cast<float*>(lds);  // [2 S][16 rows][17]
#pragma unroll
    for (int i = 0; i < 4; ++i) red[(wave * 16 + r) * 17 + 4 * kq + i] = acc[i];
    __syncthreads();
    if (threadIdx.x < 256) {
        const int m = threadIdx.x >> 4, n = n0 + (threadIdx.x & 15);
        if (m < p.M && n < p.I) {
            float g = 0.f, u = 0.f;
            for (int sl = 0; sl < p.S; ++sl) {
                g += red[(sl * 16 + m) * 17 + (threadIdx.x & 15)];
                u += red[((p.S + sl) * 16 + m) * 17 + (threadIdx.x & 15)];
            }
            g = C::up(C::down(g));
            u = C::up(C::down(u));
            const float act = C::up(C::down(g / (1.f + expf(-g))));
            p.out[(int64_t)m * p.os + n] = C::down(act * u);
        }
    }
}

}  // namespace

// K splits that give about two workgroups per CU of the current device (256 CUs assumed when no
// device can be asked) without slices shorter than one chunk
// of 512; when one chunk per workgroup is at least that many splits and still a moderate grid,
// that is taken instead: a workgroup then stages x once and has no loop (measured 11 % faster at
// N = 19456, K = 2560).
extern "C" int ksa_gemm_rows_auto_splits(int N, int K) {
    if (N <= 0 || K <= 0) return 1;
    const int tiles = (N + 63) / 64;
    const int want = 2 * ksa_cu_count_or(256);
    int sp = (want + tiles - 1) / tiles;
    const int chunks = K / 32 / 16 > 1 ? K / 32 / 16 : 1;
    if (sp > chunks) sp = chunks;
    if (sp > 16) sp = 16;
    if (sp < 1) sp = 1;
    if (sp > 1 && chunks >= sp && chunks <= 16 && (long long)tiles * chunks <= 2048 && K % (32 * 16) == 0) sp = chunks;
    return sp;
}

extern "C" size_t ksa_gemm_rows_workspace_bytes(int N, int ksplit) {
    return ksplit > 1 ? (size_t)ksplit * 16 * (size_t)N * sizeof(float) : 0;
}

extern "C" int ksa_gemm_rows(const void* x, const void* w, void* out, int M, int N, int K, long long x_row_stride,
                             long long w_row_stride, long long out_row_stride, int dtype, int ksplit,
                             void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !w) return KSA_ERR_NULL;
    if (!out && ksplit <= 1) return KSA_ERR_NULL;  // out may be null only to leave the partial sums to the caller
    if (M <= 0 || M > 16 || N <= 0 || K <= 0 || K % 32 != 0 || ksplit < 1 || ksplit > 64) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return KSA_ERR_ALIGN;
    if (x_row_stride % 8 || w_row_stride % 8) return KSA_ERR_ALIGN;
    GemmParams p{};
    p.x = (const uint16_t*)x;
    p.w = (const uint16_t*)w;
    p.out = (uint16_t*)out;
    p.xs = x_row_stride, p.ws = w_row_stride, p.os = out_row_stride;
    p.M = M, p.N = N, p.K = K, p.ksplit = ksplit;
    if (ksplit > 1) {
        if (!workspace || workspace_bytes < ksa_gemm_rows_workspace_bytes(N, ksplit)) return KSA_ERR_WORKSPACE;
        p.part = (float*)workspace;
    }
    return dtype == KSA_DTYPE_BF16 ? launch_gemm<KsaBf16>(p, (hipStream_t)stream)
                                   : launch_gemm<KsaF16>(p, (hipStream_t)stream);
}

extern "C" int ksa_gemm_rows_gate_up_silu(const void* x, const void* w, void* out, int M, int I, int K,
                                          long long x_row_stride, long long w_row_stride,
                                          long long out_row_stride, int dtype, void* stream) {
    if (!x || !w || !out) return KSA_ERR_NULL;
    if (M <= 0 || M > 16 || I <= 0 || K <= 0 || K % 32 != 0) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return KSA_ERR_ALIGN;
    if (x_row_stride % 8 || w_row_stride % 8) return KSA_ERR_ALIGN;
    GateUpParams p{};
    p.x = (const uint16_t*)x;
    p.w = (const uint16_t*)w;
    p.out = (uint16_t*)out;
    p.xs = x_row_stride, p.ws = w_row_stride, p.os = out_row_stride;
    p.M = M, p.I = I, p.K = K;
    const int chunks = (K / 32 + kChunkSteps - 1) / kChunkSteps;
    p.S = chunks < kGateUpMaxSlices ? chunks : kGateUpMaxSlices;
    const size_t lds = gate_up_lds_bytes(M, K, p.S);
    if (lds > 160 * 1024) return KSA_ERR_UNSUPPORTED;  // x does not fit LDS whole: M (K + 8) 2 bytes
    const dim3 grid((I + 15) / 16), block(128 * p.S);
    auto kern = dtype == KSA_DTYPE_BF16 ? ksa_gemm_gate_up_silu_kernel<KsaBf16> : ksa_gemm_gate_up_silu_kernel<KsaF16>;
    if (lds > 64 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return KSA_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, grid, block, lds, (hipStream_t)stream, p);
    return ksa_check_launch();
}
