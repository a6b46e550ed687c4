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
// rounds them.  Up to 16 rows of x are one B operand; 17 to 128 rows (a decode step of a larger batch,
// the 9 tokens per sequence of a chunk-boundary step) take the `wide` kernel below, which feeds every
// weight fragment to one MFMA per 16-row block of x.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "ksa_api_internal.h"
#include "ksa_cvt.h"
#include "ksa_rows_mfma.h"

namespace {

struct GemmParams {
    const uint16_t* x;   // [M, K], row stride xs
    const uint16_t* w;   // [N, K], row stride ws
    uint16_t* out;       // [M, N], row stride os
    float* part;         // [ksplit, ksa_partial_rows(M), N] when ksplit > 1
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

    const KsaWeightLane wl = ksa_weight_lane(p.w, p.ws, p.K, n0, r, kq, p.N);
    // rows of x beyond M repeat the last one: their columns of the product are never stored
    const int xrow = min(r, p.M - 1);

    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    int buf = 0;
    for (int c0 = s_begin; c0 < s_end; c0 += kChunkSteps) {
        const int nst = min(kChunkSteps, s_end - c0);
        u32x4 a[kChunkSteps];
#pragma unroll
        for (int u = 0; u < kChunkSteps; ++u) a[u] = *reinterpret_cast<const u32x4*>(wl.p + wl.step * min(c0 + u, s_end - 1));
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
    const int prows = ksa_partial_rows(p.M);
    for (int sp = 0; sp < p.ksplit; ++sp) v += p.part[((int64_t)sp * prows + m) * p.N + n];
    p.out[(int64_t)m * p.os + n] = C::down(v);
}


// ---- 17 to 128 rows of x ----
// grid: (column tiles, K splits); block: eight waves, each 16 columns over the K slice of the
// workgroup, which it walks in chunks of 512 elements.  Per chunk the workgroup stages the rows of x in
// LDS once (one buffer: 1040 bytes per row, whole 16-row blocks, up to 130 KB) and every wave multiplies its 16 weight fragments
// with each of the MB 16-row blocks of x.  The stream from HBM does not stop at the two barriers between
// chunks: a weight fragment's register is refilled with the next chunk's fragment right behind its last
// MFMA, and the next chunk of x waits in registers, requested in front of those (so that the wait for it
// does not include them).
// kPair (the MLP's first half, out = SiLU(x Wg^T) * (x Wu^T) with w = [gate rows; up rows]): waves
// 0..3 take gate columns, waves 4..7 the same columns of up; they meet in LDS behind the walk and the
// up waves write the activation.  K is not split in this form.
struct WideParams {
    const uint16_t* x;
    const uint16_t* w;
    uint16_t* out;
    float* part;  // [ksplit, ksa_partial_rows(M), N] when ksplit > 1
    int64_t xs, ws, os;
    int M, N, K, ksplit, chunks_per_split;
};
constexpr int kWideWaves = 8;

template <typename T, int MB, bool kPair>
__global__ __launch_bounds__(64 * kWideWaves) void ksa_gemm_rows_wide_kernel(const WideParams p) {
    using C = KsaCvt<T>;
    extern __shared__ __attribute__((aligned(16))) unsigned char wide_lds[];
    constexpr int nw = kWideWaves;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r = lane & 15;   // row of W inside the wave's tile (A operand) / row of x inside a block (B operand)
    const int kq = lane >> 4;  // which 8 of the 32 K elements of a step
    int n0;                    // first output column of this wave (kPair: of the gate / up half)
    KsaWeightLane wl;          // this lane's piece of the wave's weight fragments
    if constexpr (kPair) {
        const int half = wave / (nw / 2);
        n0 = (blockIdx.x * (nw / 2) + wave % (nw / 2)) * 16;
        wl = ksa_weight_lane(p.w, p.ws, p.K, (int64_t)half * p.N + n0, r, kq, (int64_t)(half + 1) * p.N);
    } else {
        n0 = (blockIdx.x * nw + wave) * 16;
        wl = ksa_weight_lane(p.w, p.ws, p.K, n0, r, kq, p.N);
    }
    const int steps = p.K / 32;
    const int chunks = (steps + kChunkSteps - 1) / kChunkSteps;
    const int c_begin = blockIdx.y * p.chunks_per_split;
    const int c_end = min(chunks, c_begin + p.chunks_per_split);

    f32x4 acc[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    // rows of x beyond M repeat the last one: their columns of the product are never stored
    int xoff[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) xoff[b] = min(16 * b + r, p.M - 1) * kRowB + 16 * kq;

    // staging of a chunk of x: thread = (row tr of a pass of eight rows, 16-byte piece tj of the row's chunk).
    // No predicates: rows past M repeat the last row and pieces past a short last chunk its last piece
    // (LDS holds whole 16-row blocks; what lands there is never used).
    constexpr int XT = 2 * MB;
    const int tr = threadIdx.x >> 6, tj = threadIdx.x & 63;
    unsigned char* xdst = wide_lds + tr * kRowB + 16 * tj;
    int64_t xrow_off[XT];
#pragma unroll
    for (int i = 0; i < XT; ++i) xrow_off[i] = (int64_t)min(tr + nw * i, p.M - 1) * p.xs;
    u32x4 xt[XT];
    auto x_request = [&](int c) {
        const int nst = min(kChunkSteps, steps - c * kChunkSteps);
        const uint16_t* src = p.x + (int64_t)kChunkK * c + 8 * min(tj, 4 * nst - 1);
#pragma unroll
        for (int i = 0; i < XT; ++i) xt[i] = *reinterpret_cast<const u32x4*>(src + xrow_off[i]);
    };
    // (a short last chunk is filled up with zeros: its missing steps then add nothing, whatever weights
    // the clamped requests fetch for them)
    auto x_store = [&](int c) {
        const bool live = tj < 4 * min(kChunkSteps, steps - c * kChunkSteps);
#pragma unroll
        for (int i = 0; i < XT; ++i) {
            u32x4 v = xt[i];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = live ? v[e] : 0u;
            *reinterpret_cast<u32x4*>(xdst + nw * i * kRowB) = v;
        }
    };
    u32x4 a[kChunkSteps];
    auto w_request = [&](int c, int u) {
        a[u] = *reinterpret_cast<const u32x4*>(wl.p + wl.step * min(c * kChunkSteps + u, steps - 1));
    };
    // the products of one chunk; kMore: there is a next chunk, whose x and weights are requested on the way
    // (two copies of the loop body rather than a condition inside it: with branches between the MFMAs the
    // compiler waits for every outstanding load in front of each of them)
    auto chunk = [&](auto more_tag, int cn) __attribute__((always_inline)) {  // cn: the next chunk (kMore)
        constexpr bool kMore = decltype(more_tag)::value;
        if constexpr (kMore) x_request(cn);
        // the rows of x of step u + 1 are read from LDS while the MFMAs of step u run; the fences keep
        // the compiler from reading many steps ahead (which costs it more registers than there are)
        u32x4 bf[2][MB];
#pragma unroll
        for (int b = 0; b < MB; ++b) bf[0][b] = *reinterpret_cast<const u32x4*>(wide_lds + xoff[b]);
#pragma unroll
        for (int u = 0; u < kChunkSteps; ++u) {
            if (u + 1 < kChunkSteps) {
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    bf[(u + 1) & 1][b] = *reinterpret_cast<const u32x4*>(wide_lds + xoff[b] + 64 * (u + 1));
            }
#pragma unroll
            for (int b = 0; b < MB; ++b) acc[b] = mfma16<T>(a[u], bf[u & 1][b], acc[b]);
            if constexpr (kMore) w_request(cn, u);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if (c_begin < c_end) {  // (uniform; an empty slice does not exist in a grid made by wide_plan)
        x_request(c_begin);
#pragma unroll
        for (int u = 0; u < kChunkSteps; ++u) w_request(c_begin, u);
        x_store(c_begin);
        __syncthreads();
        for (int c = c_begin; c + 1 < c_end; ++c) {
            chunk(std::true_type{}, c + 1);
            __syncthreads();  // every wave is done with this chunk of x
            x_store(c + 1);
            __syncthreads();
        }
        chunk(std::false_type{}, c_end);
    }
    // C layout of a 16x16 tile: lane holds row (of x) lane % 16 of the block, columns n0 + 4 * (lane / 16) + i
    const int n = n0 + 4 * kq;
    if constexpr (kPair) {
        __syncthreads();  // x is no longer read: its place takes the gate halves
        f32x4* ex = reinterpret_cast<f32x4*>(wide_lds);
        constexpr int hw = nw / 2;
        if (wave < hw) {
#pragma unroll
            for (int b = 0; b < MB; ++b) ex[(wave * MB + b) * 64 + lane] = acc[b];
        }
        __syncthreads();
        if (wave >= hw) {
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const int m = 16 * b + r;
                if (m < p.M && n < p.N) {
                    const f32x4 gv = ex[((wave - hw) * MB + b) * 64 + lane];
                    uint16_t o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float g = C::up(C::down(gv[i])), u = C::up(C::down(acc[b][i]));
                        const float act = C::up(C::down(g / (1.f + expf(-g))));
                        o[i] = C::down(act * u);
                    }
                    uint16_t* dst = p.out + (int64_t)m * p.os + n;
                    if (n + 3 < p.N && (p.os % 4) == 0) {
                        u32x2 v2;
                        v2[0] = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
                        v2[1] = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
                        *reinterpret_cast<u32x2*>(dst) = v2;
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if (n + i < p.N) dst[i] = o[i];
                    }
                }
            }
        }
    } else {
        const int prows = ksa_partial_rows(p.M);
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const int m = 16 * b + r;
            if (m < p.M && n < p.N) {
                if (p.ksplit == 1) {
                    uint16_t* dst = p.out + (int64_t)m * p.os + n;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n + i < p.N) dst[i] = C::down(acc[b][i]);
                } else {
                    float* dst = p.part + ((int64_t)blockIdx.y * prows + m) * p.N + n;
                    if (n + 3 < p.N && (p.N % 4) == 0) {
                        *reinterpret_cast<f32x4*>(dst) = acc[b];
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if (n + i < p.N) dst[i] = acc[b][i];
                    }
                }
            }
        }
    }
}

// K splits and chunks per split of the wide kernel for a wanted number of splits (slices are whole
// chunks, none empty)
struct WidePlan {
    int ksplit, chunks_per_split;
};
static WidePlan wide_plan(int K, int want_splits) {
    const int chunks = (K / 32 + kChunkSteps - 1) / kChunkSteps;
    WidePlan pl;
    int sp = want_splits < 1 ? 1 : want_splits;
    if (sp > chunks) sp = chunks;
    pl.chunks_per_split = (chunks + sp - 1) / sp;
    pl.ksplit = (chunks + pl.chunks_per_split - 1) / pl.chunks_per_split;
    return pl;
}

template <typename T, bool kPair>
int launch_wide(const WideParams& p, hipStream_t st) {
    const int mb = (p.M + 15) / 16;
    constexpr int cols = kPair ? 16 * (kWideWaves / 2) : 16 * kWideWaves;
    const dim3 grid((p.N + cols - 1) / cols, p.ksplit), block(64 * kWideWaves);
    size_t lds = (size_t)mb * 16 * kRowB;
    if (kPair && lds < (size_t)(kWideWaves / 2) * mb * 64 * sizeof(f32x4)) lds = (size_t)(kWideWaves / 2) * mb * 64 * sizeof(f32x4);
    if (lds > 160 * 1024) return KSA_ERR_UNSUPPORTED;
    auto go = [&](auto kern) {
        if (lds > 64 * 1024 &&
            hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return (int)KSA_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, block, lds, st, p);
        return ksa_check_launch();
    };
    switch (mb) {
        case 2: return go(ksa_gemm_rows_wide_kernel<T, 2, kPair>);
        case 3: return go(ksa_gemm_rows_wide_kernel<T, 3, kPair>);
        case 4: return go(ksa_gemm_rows_wide_kernel<T, 4, kPair>);
        case 5: return go(ksa_gemm_rows_wide_kernel<T, 5, kPair>);
        case 6: return go(ksa_gemm_rows_wide_kernel<T, 6, kPair>);
        default: return go(ksa_gemm_rows_wide_kernel<T, 8, kPair>);
    }
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
    const KsaWeightLane wl = ksa_weight_lane(p.w, p.ws, p.K, (int64_t)half * p.I + n0, r, kq, (int64_t)(half + 1) * p.I);
    const int xrow = min(r, p.M - 1);

    // eight K steps of weights in flight per wave (32 registers): with at most 64 registers a SIMD
    // holds eight waves, so three workgroups of ten waves per CU and the whole grid of a 4B-shape
    // MLP (608 workgroups) is resident at once
    constexpr int kB = 8;
    u32x4 a[kB];
    auto load_steps = [&](int s0) {
#pragma unroll
        for (int u = 0; u < kB; ++u) a[u] = *reinterpret_cast<const u32x4*>(wl.p + wl.step * min(s0 + u, steps - 1));
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

// The same two questions for a product of M rows (M <= 16: the answers above).  For more rows a slice
// of the partial sums has ksa_partial_rows(M) rows, and K is split as far as the grid (tiles of 128
// columns x splits) stays within about one workgroup per CU - one resident workgroup is all a CU holds
// of this kernel, and a second round costs more than longer slices do (measured at 72 rows on the
// projections of the 4B shape: 6144 x 2560 best at 5 splits, 2560 x 4096 at 8, 2560 x 9728 at 10,
// 19456 x 2560 at 2).
extern "C" int ksa_gemm_rows_splits(int M, int N, int K) {
    if (M <= 16) return ksa_gemm_rows_auto_splits(N, K);
    if (N <= 0 || K <= 0) return 1;
    const int tiles = (N + 127) / 128;
    const int want = (ksa_cu_count_or(256) * 5 / 4) / tiles;
    return wide_plan(K, want).ksplit;
}

extern "C" size_t ksa_gemm_rows_partials_bytes(int M, int N, int ksplit) {
    return ksplit > 1 ? (size_t)ksplit * (size_t)ksa_partial_rows(M) * (size_t)N * sizeof(float) : 0;
}

extern "C" int ksa_gemm_rows(const void* x, const void* w, void* out, int M, int N, int K, long long x_row_stride,
                             long long w_row_stride, long long out_row_stride, int dtype, int ksplit,
                             void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !w) return KSA_ERR_NULL;
    if (!out && ksplit <= 1) return KSA_ERR_NULL;  // out may be null only to leave the partial sums to the caller
    if (M <= 0 || M > kMaxPartialRows || N <= 0 || K <= 0 || K % 32 != 0 || ksplit < 1 || ksplit > 64) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return KSA_ERR_ALIGN;
    if (x_row_stride % 8 || (w_row_stride != kWTiled && w_row_stride % 8)) return KSA_ERR_ALIGN;
    if (M > 16) {
        const WidePlan pl = wide_plan(K, ksplit);
        if (pl.ksplit != ksplit) return KSA_ERR_INVALID;  // not a split count of ksa_gemm_rows_splits: an empty slice
        WideParams wp{};
        wp.x = (const uint16_t*)x, wp.w = (const uint16_t*)w, wp.out = (uint16_t*)out;
        wp.xs = x_row_stride, wp.ws = w_row_stride, wp.os = out_row_stride;
        wp.M = M, wp.N = N, wp.K = K, wp.ksplit = ksplit, wp.chunks_per_split = pl.chunks_per_split;
        if (ksplit > 1) {
            if (!workspace || workspace_bytes < ksa_gemm_rows_partials_bytes(M, N, ksplit)) return KSA_ERR_WORKSPACE;
            if (reinterpret_cast<uintptr_t>(workspace) & 15) return KSA_ERR_ALIGN;  // 16-byte stores of the sums
            wp.part = (float*)workspace;
        }
        const int rc = dtype == KSA_DTYPE_BF16 ? launch_wide<KsaBf16, false>(wp, (hipStream_t)stream)
                                               : launch_wide<KsaF16, false>(wp, (hipStream_t)stream);
        if (rc != KSA_OK || ksplit == 1 || !out) return rc;
        GemmParams rp{};
        rp.out = (uint16_t*)out, rp.part = wp.part, rp.os = out_row_stride;
        rp.M = M, rp.N = N, rp.K = K, rp.ksplit = ksplit;
        const int64_t n = (int64_t)M * N;
        if (dtype == KSA_DTYPE_BF16)
            hipLaunchKernelGGL(ksa_gemm_rows_reduce_kernel<KsaBf16>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                               (hipStream_t)stream, rp);
        else
            hipLaunchKernelGGL(ksa_gemm_rows_reduce_kernel<KsaF16>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                               (hipStream_t)stream, rp);
        return ksa_check_launch();
    }
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
    if (M <= 0 || M > kMaxPartialRows || I <= 0 || K <= 0 || K % 32 != 0) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return KSA_ERR_ALIGN;
    if (x_row_stride % 8 || (w_row_stride != kWTiled && w_row_stride % 8)) return KSA_ERR_ALIGN;
    if (w_row_stride == kWTiled && I % 16 != 0) return KSA_ERR_UNSUPPORTED;  // gate and up rows must start tiles of their own
    if (M > 16) {  // chunks of x through LDS, gate and up waves of a workgroup meet behind the walk
        if (reinterpret_cast<uintptr_t>(out) & 7) return KSA_ERR_ALIGN;  // 8-byte stores of the activation
        WideParams wp{};
        wp.x = (const uint16_t*)x, wp.w = (const uint16_t*)w, wp.out = (uint16_t*)out;
        wp.xs = x_row_stride, wp.ws = w_row_stride, wp.os = out_row_stride;
        wp.M = M, wp.N = I, wp.K = K, wp.ksplit = 1;
        wp.chunks_per_split = (K / 32 + kChunkSteps - 1) / kChunkSteps;
        return dtype == KSA_DTYPE_BF16 ? launch_wide<KsaBf16, true>(wp, (hipStream_t)stream)
                                       : launch_wide<KsaF16, true>(wp, (hipStream_t)stream);
    }
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

// ---- the streaming layout of a weight matrix ----
namespace {
// out [ceil(N / 16)][K / 32][16][32] <- w [N, K] (rows past N: zeros); 16 bytes per thread
__global__ __launch_bounds__(256) void ksa_tile_weights_kernel(const uint16_t* w, uint16_t* out, int N, int K, int64_t ws) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;  // 16-byte piece of the output
    const int steps = K / 32;
    const int64_t total = (int64_t)((N + 15) / 16) * steps * 64;
    if (e >= total) return;
    const int q = (int)(e & 3), r = (int)((e >> 2) & 15);
    const int64_t frag = e >> 6;
    const int s = (int)(frag % steps);
    const int64_t row = (frag / steps) * 16 + r;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < N) v = *reinterpret_cast<const u32x4*>(w + row * ws + 32 * s + 8 * q);
    *reinterpret_cast<u32x4*>(out + 8 * e) = v;
}
}  // namespace

extern "C" size_t ksa_tile_weights_bytes(int N, int K) {
    return N > 0 && K > 0 ? (size_t)((N + 15) / 16 * 16) * (size_t)K * 2 : 0;
}

extern "C" int ksa_tile_weights(const void* w, void* out, int N, int K, long long w_row_stride, void* stream) {
    if (!w || !out) return KSA_ERR_NULL;
    if (N <= 0 || K <= 0 || K % 32 != 0) return KSA_ERR_INVALID;
    if ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(out)) & 15) return KSA_ERR_ALIGN;
    if (w_row_stride % 8) return KSA_ERR_ALIGN;
    const int64_t total = (int64_t)((N + 15) / 16) * (K / 32) * 64;
    hipLaunchKernelGGL(ksa_tile_weights_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t*)w, (uint16_t*)out, N, K, (int64_t)w_row_stride);
    return ksa_check_launch();
}
