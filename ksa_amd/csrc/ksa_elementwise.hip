// Two element-wise steps of a decoder layer around the attention path, one pass over HBM each
// (gfx950), with the rounding points of the reference's 16-bit tensor ops:
//   * residual add + RMSNorm over the hidden size
//       examples/pretrain/hf_template/modeling_qwen3sa.py:64-79 (Qwen3RMSNorm.forward: fp32
//       normalisation, result rounded to the 16-bit type, times the 16-bit weight) and the
//       residual adds of Qwen3DecoderLayer.forward :946, :952
//   * SiLU(gate) * up of the MLP (:507-514)
// Both replace chains of 3-8 library element-wise launches; at decode batch sizes a layer step
// is bound by the number of launches.
#include <hip/hip_runtime.h>

#include "ksa_api_internal.h"
#include "ksa_cvt.h"

namespace {

struct NormParams {
    const uint16_t* x;
    const float* part;     // partial-sum variant: x = rounded sum of `ksplit` fp32 slices [ksplit][ksa_partial_rows(rows)][H]
    int ksplit;
    const uint16_t* res;   // may be null
    const uint16_t* w;
    uint16_t* out_norm;
    uint16_t* out_sum;     // x + res (null if res is null)
    int64_t rows;
    int64_t xs, rs, ns, ss;  // row strides (elements)
    int H;
    float eps;
};

// One wave per row; the row (after the residual add) stays in registers between the
// sum-of-squares pass and the scaling pass.  NI = 16-byte items per lane.  Inputs are read once:
// non-temporal loads.
template <typename T, int NI>
__global__ __launch_bounds__(256) void ksa_add_rmsnorm_kernel(const NormParams p) {
    using C = KsaCvt<T>;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int items = p.H / 8;
    for (int64_t row = (int64_t)blockIdx.x * 4 + wave; row < p.rows; row += (int64_t)gridDim.x * 4) {
        u32x4 r[NI];
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int idx = lane + 64 * j;
            if (idx < items) {
                r[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.x + row * p.xs + 8 * idx));
                if (p.res) {
                    const u32x4 q = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.res + row * p.rs + 8 * idx));
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        r[j][i] = C::down2(C::lo(r[j][i]) + C::lo(q[i]), C::hi(r[j][i]) + C::hi(q[i]));
                    *reinterpret_cast<u32x4*>(p.out_sum + row * p.ss + 8 * idx) = r[j];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float a = C::lo(r[j][i]), b = C::hi(r[j][i]);
                    ss = fmaf(a, a, ss);
                    ss = fmaf(b, b, ss);
                }
            }
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
        const float inv = rsqrtf(ss / (float)p.H + p.eps);
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int idx = lane + 64 * j;
            if (idx < items) {
                const u32x4 wv = *reinterpret_cast<const u32x4*>(p.w + 8 * idx);
                u32x4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t y = C::down2(C::lo(r[j][i]) * inv, C::hi(r[j][i]) * inv);
                    o[i] = C::down2(C::lo(wv[i]) * C::lo(y), C::hi(wv[i]) * C::hi(y));
                }
                *reinterpret_cast<u32x4*>(p.out_norm + row * p.ns + 8 * idx) = o;
            }
        }
    }
}

// The same step for the few rows of a decode step when x is still the K-split partial sums of
// the GEMM that produced it (fp32 [ksplit][rows in whole 16-row blocks][H], as ksa_gemm_rows leaves them): one workgroup
// per row, as many threads as the row has 16-byte items (up to 512, then NJ = 2 items per thread),
// adds the slices in split order, rounds (which is what the GEMM's own reduction does), adds the
// residual and normalises.  Everything that does not depend on the sums is requested first.
template <typename T, int NJ>
__global__ __launch_bounds__(512) void ksa_add_rmsnorm_partials_kernel(const NormParams p) {
    using C = KsaCvt<T>;
    __shared__ float s_ss[8];
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int row = blockIdx.x;
    const int items = p.H / 8;
    u32x4 r[NJ], wv[NJ], q[NJ];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {  // the weights and the residual do not wait for the sums
        const int idx = tid + nthr * j;
        if (idx < items) {
            wv[j] = *reinterpret_cast<const u32x4*>(p.w + 8 * idx);
            q[j] = *reinterpret_cast<const u32x4*>(p.res + (int64_t)row * p.rs + 8 * idx);
        }
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int idx = tid + nthr * j;
        if (idx < items) {
            const u32x4 x = ksa_sum_partials8<T>(p.part, p.ksplit, ksa_partial_rows(p.rows), p.H, row, 8 * idx);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                r[j][i] = C::down2(C::lo(x[i]) + C::lo(q[j][i]), C::hi(x[i]) + C::hi(q[j][i]));
                const float a = C::lo(r[j][i]), b = C::hi(r[j][i]);
                ss = fmaf(a, a, ss);
                ss = fmaf(b, b, ss);
            }
            *reinterpret_cast<u32x4*>(p.out_sum + (int64_t)row * p.ss + 8 * idx) = r[j];
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
    if ((tid & 63) == 0) s_ss[tid >> 6] = ss;
    __syncthreads();
    ss = 0.f;
    for (int w = 0; w < nthr / 64; ++w) ss += s_ss[w];
    const float inv = rsqrtf(ss / (float)p.H + p.eps);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int idx = tid + nthr * j;
        if (idx < items) {
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t y = C::down2(C::lo(r[j][i]) * inv, C::hi(r[j][i]) * inv);
                o[i] = C::down2(C::lo(wv[j][i]) * C::lo(y), C::hi(wv[j][i]) * C::hi(y));
            }
            *reinterpret_cast<u32x4*>(p.out_norm + (int64_t)row * p.ns + 8 * idx) = o;
        }
    }
}

template <typename T>
int dispatch_norm_partials(const NormParams& p, hipStream_t st) {
    const int items = p.H / 8;
    const int threads = items >= 512 ? 512 : (items + 63) / 64 * 64;
    const int need = (items + threads - 1) / threads;
    const dim3 grid((unsigned)p.rows), block(threads);
    if (need <= 1) hipLaunchKernelGGL((ksa_add_rmsnorm_partials_kernel<T, 1>), grid, block, 0, st, p);
    else if (need <= 2) hipLaunchKernelGGL((ksa_add_rmsnorm_partials_kernel<T, 2>), grid, block, 0, st, p);
    else return KSA_ERR_UNSUPPORTED;
    return ksa_check_launch();
}

template <typename T, int NI>
int launch_norm(const NormParams& p, hipStream_t st) {
    const int64_t blocks = (p.rows + 3) / 4;
    // one short-lived workgroup per four rows (measured 5 % faster than a capped grid with a
    // grid-stride loop); the loop only serves row counts beyond the grid limit
    const int64_t cap = 0x7fffffff;
    hipLaunchKernelGGL((ksa_add_rmsnorm_kernel<T, NI>), dim3((unsigned)(blocks < cap ? blocks : cap)), dim3(256), 0,
                       st, p);
    return ksa_check_launch();
}

template <typename T>
int dispatch_norm(const NormParams& p, hipStream_t st) {
    const int need = (p.H / 8 + 63) / 64;
    if (need <= 1) return launch_norm<T, 1>(p, st);
    if (need <= 2) return launch_norm<T, 2>(p, st);
    if (need <= 4) return launch_norm<T, 4>(p, st);
    if (need <= 8) return launch_norm<T, 8>(p, st);
    if (need <= 16) return launch_norm<T, 16>(p, st);
    return KSA_ERR_UNSUPPORTED;
}

struct ActParams {
    const uint16_t* gate;
    const uint16_t* up;
    uint16_t* out;
    int64_t gs, us, os;  // row strides (elements)
    int I;
    const float* part;   // if set: gate | up as K-split partial sums, see the kernel
    int ksplit;
};

// blockIdx.x = row, blockIdx.y = block of 256 16-byte items inside the row
// kPartials: a variant of its own, so that the streaming variant does not carry its registers
template <typename T, bool kPartials>
__global__ __launch_bounds__(256) void ksa_silu_mul_kernel(const ActParams p) {
    using C = KsaCvt<T>;
    const int64_t row = blockIdx.x;
    const int idx = blockIdx.y * 256 + threadIdx.x;
    if (idx >= p.I / 8) return;
    u32x4 g, u;
    if constexpr (kPartials) {  // gate | up still as the partial sums of the fused projection [ksplit][ksa_partial_rows(rows)][2 I]
        g = ksa_sum_partials8<T>(p.part, p.ksplit, ksa_partial_rows((int)gridDim.x), 2 * p.I, (int)row, 8 * idx);
        u = ksa_sum_partials8<T>(p.part, p.ksplit, ksa_partial_rows((int)gridDim.x), 2 * p.I, (int)row, p.I + 8 * idx);
    } else {
        g = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.gate + row * p.gs + 8 * idx));
        u = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.up + row * p.us + 8 * idx));
    }
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float a = C::lo(g[i]), b = C::hi(g[i]);
        const uint32_t s = C::down2(a / (1.f + expf(-a)), b / (1.f + expf(-b)));
        o[i] = C::down2(C::lo(s) * C::lo(u[i]), C::hi(s) * C::hi(u[i]));
    }
    *reinterpret_cast<u32x4*>(p.out + row * p.os + 8 * idx) = o;
}

bool al16(const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; }

// ---- greedy token choice: index of the largest value of every row ----
// One workgroup of 1024 threads per row; a thread scans every 1024th 16-byte item (several
// requests in flight), then wave and workgroup reductions on (value, index) pairs.  Among equal
// values the lowest index wins and a NaN counts as the largest value, as torch.argmax has it.
struct ArgmaxParams {
    const uint16_t* x;
    long long* out;
    int64_t xs;
    int N;
};

__device__ __forceinline__ bool argmax_better(float a, int ia, float b, int ib) {
    // (the library is built without NaN-honouring float compares: test the bits)
    const bool na = (__builtin_bit_cast(uint32_t, a) & 0x7fffffffu) > 0x7f800000u;
    const bool nb = (__builtin_bit_cast(uint32_t, b) & 0x7fffffffu) > 0x7f800000u;
    if (na != nb) return na;
    if (!na && a != b) return a > b;
    return ia < ib;
}

template <typename T>
__global__ __launch_bounds__(1024) void ksa_argmax_rows_kernel(const ArgmaxParams p) {
    using C = KsaCvt<T>;
    const uint16_t* row = p.x + (int64_t)blockIdx.x * p.xs;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    const int items = p.N / 8;
    for (int j0 = threadIdx.x; j0 < items; j0 += 4 * 1024) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int j = j0 + 1024 * u;
            v[u] = *reinterpret_cast<const u32x4*>(row + 8 * (j < items ? j : j0));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int j = j0 + 1024 * u;
            if (j < items) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float lo = C::up((uint16_t)(v[u][i] & 0xffffu)), hi = C::up((uint16_t)(v[u][i] >> 16));
                    if (argmax_better(lo, 8 * j + 2 * i, best, bi)) best = lo, bi = 8 * j + 2 * i;
                    if (argmax_better(hi, 8 * j + 2 * i + 1, best, bi)) best = hi, bi = 8 * j + 2 * i + 1;
                }
            }
        }
    }
    for (int n = 8 * items + threadIdx.x; n < p.N; n += 1024) {  // a tail shorter than one item
        const float v = C::up(row[n]);
        if (argmax_better(v, n, best, bi)) best = v, bi = n;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ob = __shfl_xor(best, m);
        const int oi = __shfl_xor(bi, m);
        if (argmax_better(ob, oi, best, bi)) best = ob, bi = oi;
    }
    __shared__ float sv[16];
    __shared__ int si[16];
    if ((threadIdx.x & 63) == 0) sv[threadIdx.x >> 6] = best, si[threadIdx.x >> 6] = bi;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (argmax_better(sv[w], si[w], best, bi)) best = sv[w], bi = si[w];
        p.out[blockIdx.x] = bi;
    }
}

}  // namespace

extern "C" int ksa_add_rmsnorm(const void* x, const void* residual, const void* weight, void* out_norm,
                               void* out_sum, long long rows, int H, long long x_row_stride,
                               long long residual_row_stride, long long norm_row_stride,
                               long long sum_row_stride, int dtype, float eps, void* stream) {
    if (!x || !weight || !out_norm) return KSA_ERR_NULL;
    if (residual && !out_sum) return KSA_ERR_NULL;
    if (rows <= 0 || H <= 0 || H % 8 != 0 || !(eps >= 0.f)) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if (!al16(x) || !al16(weight) || !al16(out_norm) || (residual && (!al16(residual) || !al16(out_sum))))
        return KSA_ERR_ALIGN;
    if (x_row_stride % 8 || norm_row_stride % 8 || (residual && (residual_row_stride % 8 || sum_row_stride % 8)))
        return KSA_ERR_ALIGN;
    NormParams p{};
    p.x = (const uint16_t*)x;
    p.res = (const uint16_t*)residual;
    p.w = (const uint16_t*)weight;
    p.out_norm = (uint16_t*)out_norm;
    p.out_sum = residual ? (uint16_t*)out_sum : nullptr;
    p.rows = rows;
    p.xs = x_row_stride, p.rs = residual_row_stride, p.ns = norm_row_stride, p.ss = sum_row_stride;
    p.H = H;
    p.eps = eps;
    return dtype == KSA_DTYPE_BF16 ? dispatch_norm<KsaBf16>(p, (hipStream_t)stream)
                                   : dispatch_norm<KsaF16>(p, (hipStream_t)stream);
}

extern "C" int ksa_add_rmsnorm_partials(const float* partials, int ksplit, const void* residual,
                                        const void* weight, void* out_norm, void* out_sum, int rows, int H,
                                        long long residual_row_stride, long long norm_row_stride,
                                        long long sum_row_stride, int dtype, float eps, void* stream) {
    if (!partials || !residual || !weight || !out_norm || !out_sum) return KSA_ERR_NULL;
    if (rows <= 0 || rows > kMaxPartialRows || ksplit < 1 || ksplit > 64 || H <= 0 || H % 8 != 0 || !(eps >= 0.f))
        return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if (!al16(partials) || !al16(residual) || !al16(weight) || !al16(out_norm) || !al16(out_sum)) return KSA_ERR_ALIGN;
    if (residual_row_stride % 8 || norm_row_stride % 8 || sum_row_stride % 8) return KSA_ERR_ALIGN;
    NormParams p{};
    p.part = partials;
    p.ksplit = ksplit;
    p.res = (const uint16_t*)residual;
    p.w = (const uint16_t*)weight;
    p.out_norm = (uint16_t*)out_norm;
    p.out_sum = (uint16_t*)out_sum;
    p.rows = rows;
    p.rs = residual_row_stride, p.ns = norm_row_stride, p.ss = sum_row_stride;
    p.H = H;
    p.eps = eps;
    return dtype == KSA_DTYPE_BF16 ? dispatch_norm_partials<KsaBf16>(p, (hipStream_t)stream)
                                   : dispatch_norm_partials<KsaF16>(p, (hipStream_t)stream);
}

extern "C" int ksa_silu_mul(const void* gate, const void* up, void* out, long long rows, int I,
                            long long gate_row_stride, long long up_row_stride, long long out_row_stride,
                            int dtype, void* stream) {
    if (!gate || !up || !out) return KSA_ERR_NULL;
    if (rows <= 0 || rows >= (1ll << 31) || I <= 0 || I % 8 != 0) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if (!al16(gate) || !al16(up) || !al16(out) || gate_row_stride % 8 || up_row_stride % 8 || out_row_stride % 8)
        return KSA_ERR_ALIGN;
    const int yblocks = (I / 8 + 255) / 256;
    if (yblocks > 65535) return KSA_ERR_INVALID;
    ActParams p{(const uint16_t*)gate, (const uint16_t*)up, (uint16_t*)out, gate_row_stride, up_row_stride,
                out_row_stride, I, nullptr, 0};
    if (dtype == KSA_DTYPE_BF16)
        hipLaunchKernelGGL((ksa_silu_mul_kernel<KsaBf16, false>), dim3((unsigned)rows, yblocks), dim3(256), 0,
                           (hipStream_t)stream, p);
    else
        hipLaunchKernelGGL((ksa_silu_mul_kernel<KsaF16, false>), dim3((unsigned)rows, yblocks), dim3(256), 0,
                           (hipStream_t)stream, p);
    return ksa_check_launch();
}

extern "C" int ksa_silu_mul_partials(const float* partials, int ksplit, void* out, int rows, int I,
                                     long long out_row_stride, int dtype, void* stream) {
    if (!partials || !out) return KSA_ERR_NULL;
    if (rows <= 0 || rows > kMaxPartialRows || ksplit < 1 || ksplit > 64 || I <= 0 || I % 8 != 0) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if (!al16(partials) || !al16(out) || out_row_stride % 8) return KSA_ERR_ALIGN;
    const int yblocks = (I / 8 + 255) / 256;
    if (yblocks > 65535) return KSA_ERR_INVALID;
    ActParams p{nullptr, nullptr, (uint16_t*)out, 0, 0, out_row_stride, I, partials, ksplit};
    if (dtype == KSA_DTYPE_BF16)
        hipLaunchKernelGGL((ksa_silu_mul_kernel<KsaBf16, true>), dim3((unsigned)rows, yblocks), dim3(256), 0,
                           (hipStream_t)stream, p);
    else
        hipLaunchKernelGGL((ksa_silu_mul_kernel<KsaF16, true>), dim3((unsigned)rows, yblocks), dim3(256), 0,
                           (hipStream_t)stream, p);
    return ksa_check_launch();
}

extern "C" int ksa_argmax_rows(const void* x, long long* out, int rows, int N, long long x_row_stride,
                               int dtype, void* stream) {
    if (!x || !out) return KSA_ERR_NULL;
    if (rows <= 0 || rows > 65535 || N <= 0) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if (!al16(x) || x_row_stride % 8) return KSA_ERR_ALIGN;
    ArgmaxParams p{(const uint16_t*)x, out, x_row_stride, N};
    if (dtype == KSA_DTYPE_BF16)
        hipLaunchKernelGGL(ksa_argmax_rows_kernel<KsaBf16>, dim3(rows), dim3(1024), 0, (hipStream_t)stream, p);
    else
        hipLaunchKernelGGL(ksa_argmax_rows_kernel<KsaF16>, dim3(rows), dim3(1024), 0, (hipStream_t)stream, p);
    return ksa_check_launch();
}
