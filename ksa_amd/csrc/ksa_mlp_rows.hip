// The MLP of a decoder layer at a decode step as ONE launch (gfx950):
//
//   a  = SiLU(h W_gate^T) * (h W_up^T)       (Qwen3MLP.forward, examples/pretrain/hf_template/modeling_qwen3sa.py:507-514)
//   d  = a W_down^T                          (left as K-split partial sums for the next residual add + norm)
//
// for at most 16 rows h.  As two launches (ksa_gemm_rows_gate_up_silu, ksa_gemm_rows) the second
// one's 50 MB of weights cannot start to move before the first has drained, and each launch pays
// its ramp and tail (about 4.5 us).  Here one grid holds the workgroups of both products: the first
// UB workgroups each make 16 columns of the activation (eight waves, one per gate / up half and
// quarter of K, x whole in LDS, the partial tiles added in LDS); the workgroups behind them each
// own one 512-element chunk of the down projection's K for a group of eight column tiles.  (Eight
// waves, two to a SIMD: three such workgroups fit a CU, 768 in all, so the 608 gate | up workgroups
// of the 4B shape all run from the start; with ten waves a SIMD would have to take three of every
// workgroup and only two workgroups fit.)  Such a workgroup requests its weight fragments
// at once and then waits until the 32 activation tiles of its chunk are there: every gate | up
// workgroup counts itself off on its chunk's word in device memory when its columns are stored.
// Workgroups are started in the order of their numbers, so the ones a waiting workgroup depends
// on have always been started before it; the down workgroups of the first chunks wait next to the
// gate | up workgroups from the beginning, with their weights already in registers, and the rest
// follow as places become free.  No grid-wide barrier, no need for the grid to be resident as a
// whole, and the workgroups stay short-lived (which streams faster here than workgroups that loop).
//
// Optionally the launch begins with the residual add + RMSNorm in front of the MLP (one workgroup per
// row, on the K-split partial sums of the o projection: modeling_qwen3sa.py:944-947), and the
// gate | up workgroups, their first weights requested, wait for its rows the same way - the norm's
// chain of dependent memory trips then runs next to the first weight requests instead of in a
// launch of its own.
//
// The activation, which one workgroup writes and another reads inside the launch, goes through
// agent-scope atomic stores and cache-bypassing loads (the L2 caches of the eight XCDs are not
// coherent with each other for plain accesses); weights, input and output use plain accesses.
// The words only ever count up (so they need no clearing): a chunk's word by its number of tiles
// per launch; a down workgroup takes the number of past launches from a word that the last down
// workgroup of a launch advances.  Every wait is bounded: a workgroup that does not see its tiles
// arrive in time sets a status word and leaves (the output of that launch is then unusable and the
// words must be cleared by the host).
#include <hip/hip_runtime.h>

#include "ksa_api_internal.h"
#include "ksa_cvt.h"
#include "ksa_rows_mfma.h"

namespace {

constexpr int kSlices = 4;        // K slices of the hidden size = waves per gate / up half
constexpr int kTileCols = 16;     // columns of the activation per gate | up workgroup (8: same time, twice the reads of x)
constexpr int kWordStride = 64;   // 64-bit words are 512 bytes apart
// words: [0] launches so far, [1] down workgroups done, [2] status, [3] rows of the norm stages of all past
// launches (a launch may have any number of rows, and one without a norm stage has none: the target of a
// wait is this word plus the rows of the launch itself), [4 .. 11] rows of the norm stage done (eight copies,
// a gate | up workgroup watches copy number % 8: hundreds of workgroups polling one word would queue at it),
// [12 + c] tiles of chunk c stored (the same number in every launch: it depends on I alone)
constexpr int kWordLaunches = 0, kWordDone = 1, kWordStatus = 2, kWordHeadRows = 3, kWordHead0 = 4, kHeadCopies = 8,
              kWordChunk0 = 12;
constexpr int kMaxChunks = 52;    // K of the down projection up to 26624
constexpr int kSyncWords = kWordStride * (kWordChunk0 + kMaxChunks);

struct MlpParams {
    const uint16_t* x;        // h rows [M][H]; null: they come from the norm stage of this launch
    const float* o_part;      // norm stage: [o_ksplit][16][H] partial sums of the o projection
    const uint16_t* res;      // norm stage: residual rows [M][H]
    const uint16_t* norm_w;   // norm stage: weight [H]
    uint16_t* out_sum;        // norm stage: residual + o projection [M][H]
    unsigned long long* hbuf; // norm stage: its rows for the gate | up workgroups, [M][H / 4]
    int64_t res_rs, sum_rs;
    int o_ksplit, head;       // head: workgroups of the norm stage (M, or 0)
    float eps;
    const uint16_t* w_gu;     // [2 I][H]
    const uint16_t* w_dn;     // [H][I]
    float* dn_part;           // [KC][16][H]
    unsigned long long* sync;
    unsigned long long* act;  // [M][I / 4] four 16-bit values per word
    int64_t x_rs, wgu_rs, wdn_rs;
    int M, H, I;
    int UB, GR, KC;           // gate | up workgroups; column-tile groups and K chunks of the down projection
    unsigned spin_limit;
};

__device__ __forceinline__ unsigned long long ld_agent(const unsigned long long* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(unsigned long long* p, unsigned long long v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long add_agent(unsigned long long* p, unsigned long long v) {
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16 bytes written by another workgroup of this launch: a load that is not served from this XCD's
// L2 (the cache-control bit the compiler sets for agent-scope atomic loads; those stop at 8 bytes).
// Assembly with the wait inside the statement: the compiler does not know that the value of a bare
// asm load is still on its way and may copy the register before it has arrived.
__device__ __forceinline__ u32x4 ld_agent_x4_wait(const void* p) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}

template <typename T>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(6, 6))) void ksa_mlp_rows_kernel(const MlpParams p) {
    using C = KsaCvt<T>;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ int s_fail;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: what depends on it stays in scalar registers
    const int r = lane & 15;
    const int kq = lane >> 4;
    const int xrow = min(r, p.M - 1);
    constexpr int kB = 10;  // K steps of weights per request batch (40 registers; six waves per SIMD leave 80)
    u32x4 a[kB];
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};

    if ((int)blockIdx.x < p.head) {
        // ---- norm stage, one workgroup per row: x' = residual + sum of the o_proj partial sums (plain
        // store, for later launches), h = norm(x') w (for the gate | up workgroups of this launch).
        // Arithmetic and summation order of ksa_add_rmsnorm_partials. ----
        const int row = blockIdx.x;
        const int items = p.H / 8;  // at most 512: one per thread
        float* s_ss = reinterpret_cast<float*>(lds);
        float ss = 0.f;
        u32x4 rsum = {0u, 0u, 0u, 0u}, wv = {0u, 0u, 0u, 0u};
        if (tid < items) {
            wv = *reinterpret_cast<const u32x4*>(p.norm_w + 8 * tid);
            const u32x4 q = *reinterpret_cast<const u32x4*>(p.res + (int64_t)row * p.res_rs + 8 * tid);
            float ac[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int sp0 = 0; sp0 < p.o_ksplit; sp0 += 4) {  // (four slices requested at a time: registers)
                f32x4 lo[4], hi[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float* src = p.o_part + ((int64_t)min(sp0 + k, p.o_ksplit - 1) * 16 + row) * p.H + 8 * tid;
                    lo[k] = *reinterpret_cast<const f32x4*>(src);
                    hi[k] = *reinterpret_cast<const f32x4*>(src + 4);
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (sp0 + k < p.o_ksplit) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) ac[i] += lo[k][i], ac[4 + i] += hi[k][i];
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t x = C::down2(ac[2 * i], ac[2 * i + 1]);
                rsum[i] = C::down2(C::lo(x) + C::lo(q[i]), C::hi(x) + C::hi(q[i]));
                const float a_ = C::lo(rsum[i]), b_ = C::hi(rsum[i]);
                ss = fmaf(a_, a_, ss);
                ss = fmaf(b_, b_, ss);
            }
            *reinterpret_cast<u32x4*>(p.out_sum + (int64_t)row * p.sum_rs + 8 * tid) = rsum;
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
        if (lane == 0) s_ss[wave] = ss;
        __syncthreads();
        ss = 0.f;
        for (int w = 0; w < (items + 63) / 64; ++w) ss += s_ss[w];
        const float inv = rsqrtf(ss / (float)p.H + p.eps);
        if (tid < items) {
            uint32_t o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t y = C::down2(C::lo(rsum[i]) * inv, C::hi(rsum[i]) * inv);
                o[i] = C::down2(C::lo(wv[i]) * C::lo(y), C::hi(wv[i]) * C::hi(y));
            }
            unsigned long long* hp = p.hbuf + (int64_t)row * (p.H / 4) + 2 * tid;
            st_agent(hp, (unsigned long long)o[0] | ((unsigned long long)o[1] << 32));
            st_agent(hp + 1, (unsigned long long)o[2] | ((unsigned long long)o[3] << 32));
        }
        // Every thread waits until its own stores have left (they write through to memory), and only then
        // joins the barrier: the barrier itself does not wait for the stores of the other waves.
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid < kHeadCopies) add_agent(p.sync + kWordStride * (kWordHead0 + tid), 1ull);
        return;
    }
    const int bid = blockIdx.x - p.head;  // number among the workgroups of the two products
    if (bid < p.UB) {
        // ---- kTileCols columns of the activation (ksa_gemm_gate_up_silu_kernel's scheme; with fewer than
        // 16 columns the rows of W beyond them are not requested) ----
        const int u = bid;
        const int half = wave / kSlices;  // 0: gate rows of w, 1: up rows
        const int slice = wave - half * kSlices;
        const int sl_steps = p.H / 32 / kSlices;  // K steps of a slice (H is a multiple of 128)
        const int rowb = (p.H + 8) * 2;
        static_assert(kTileCols == 16, "a workgroup's columns are one tile of the streaming weight layout");
        KsaWeightLane wl = ksa_weight_lane(p.w_gu, p.wgu_rs, p.H, (int64_t)half * p.I + kTileCols * u, r, kq,
                                           (int64_t)(half + 1) * p.I);
        wl.p += (int64_t)wl.step * (slice * sl_steps);
        auto load_steps = [&](int s0) {  // (steps beyond the slice repeat its last one and are not multiplied)
            if (r < kTileCols) {
#pragma unroll
                for (int k = 0; k < kB; ++k)
                    a[k] = *reinterpret_cast<const u32x4*>(wl.p + wl.step * min(s0 + k, sl_steps - 1));
            }
        };
        load_steps(0);  // in flight while x is waited for and staged
        if (p.head > 0) {
            // the rows of the norm stage: wait for its count, then fetch them past this XCD's L2
            if (tid == 0) {
                const unsigned long long before = ld_agent(p.sync + kWordStride * kWordHeadRows);
                unsigned long long* word = p.sync + kWordStride * (kWordHead0 + (bid % kHeadCopies));
                unsigned long long* status = p.sync + kWordStride * kWordStatus;
                const unsigned long long want = before + (unsigned long long)p.head;
                unsigned spins = 0;
                int fail = 0;
                while (ld_agent(word) < want) {
                    __builtin_amdgcn_s_sleep(4);
                    if (++spins > p.spin_limit) {
                        st_agent(status, 1ull);
                        fail = 1;
                        break;
                    }
                    if ((spins & 63) == 0 && ld_agent(status) != 0) {
                        fail = 1;
                        break;
                    }
                }
                s_fail = fail;
            }
            __syncthreads();
            if (s_fail) return;
            const int per_row = p.H / 4;  // 8-byte words (agent-scope loads the compiler tracks: several in flight)
            for (int e = tid; e < p.M * per_row; e += blockDim.x) {
                const int m = e / per_row, j = e - m * per_row;
                *reinterpret_cast<unsigned long long*>(lds + m * rowb + 8 * j) = ld_agent(p.hbuf + (int64_t)m * per_row + j);
            }
        } else {
            const int per_row = p.H / 8;
            for (int e = tid; e < p.M * per_row; e += blockDim.x) {
                const int m = e / per_row, j = e - m * per_row;
                *reinterpret_cast<u32x4*>(lds + m * rowb + 16 * j) =
                    *reinterpret_cast<const u32x4*>(p.x + (int64_t)m * p.x_rs + 8 * j);
            }
        }
        __syncthreads();
        for (int s0 = 0; s0 < sl_steps; s0 += kB) {
            if (s0 != 0) load_steps(s0);
            const int nst = min(kB, sl_steps - s0);
            const unsigned char* xb = lds + xrow * rowb + (slice * sl_steps + s0) * 64 + 16 * kq;
#pragma unroll
            for (int k = 0; k < kB; ++k) {
                if (k < nst) acc = mfma16<T>(a[k], *reinterpret_cast<const u32x4*>(xb + 64 * k), acc);
            }
        }
        __syncthreads();  // x is no longer read: its place takes the partial sums
        // C layout of the 16x16 tile: lane holds row of x lane % 16, columns 4 * (lane / 16) + i
        float* red = reinterpret_cast<float*>(lds);  // [2 kSlices][16 rows][17]
#pragma unroll
        for (int i = 0; i < 4; ++i) red[(wave * 16 + r) * 17 + 4 * kq + i] = acc[i];
        __syncthreads();
        if (tid < 64) {  // (row m, four columns): the slices added in order, SiLU, product; one 8-byte store
            constexpr int kQuads = kTileCols / 4;
            const int m = tid / kQuads, c0 = 4 * (tid % kQuads);
            if (m < p.M && m < 16 && kTileCols * u + c0 < p.I) {
                unsigned long long o = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float gs = 0.f, us = 0.f;
                    for (int sl = 0; sl < kSlices; ++sl) {
                        gs += red[(sl * 16 + m) * 17 + c0 + e];
                        us += red[((kSlices + sl) * 16 + m) * 17 + c0 + e];
                    }
                    gs = C::up(C::down(gs));
                    us = C::up(C::down(us));
                    const float sl_ = C::up(C::down(gs / (1.f + expf(-gs))));
                    o |= (unsigned long long)C::down(sl_ * us) << (16 * e);
                }
                st_agent(p.act + (int64_t)m * (p.I / 4) + kQuads * u + (tid % kQuads), o);
            }
            // the stores are complete (this wave made all of them) before the tile is counted off
            __builtin_amdgcn_s_waitcnt(0);
            if (tid == 0) add_agent(p.sync + kWordStride * (kWordChunk0 + u / (kChunkK / kTileCols)), 1ull);
        }
        return;
    }

    // ---- one 512-element chunk kc of the down projection's K for the column tiles of group grp ----
    const int d = bid - p.UB;
    const int kc = d / p.GR, grp = d - kc * p.GR;
    constexpr int W = 2 * kSlices;
    const int CT = p.H / 16;
    const int ct = grp * W + wave;
    const int stepsI = p.I / 32;
    const int s0c = kc * kChunkSteps;
    const int nst = min(kChunkSteps, stepsI - s0c);
    const bool live = ct < CT;
    KsaWeightLane wl = ksa_weight_lane(p.w_dn, p.wdn_rs, p.I, 16 * min(ct, CT - 1), r, kq, p.H);  // (dead behind the requests)
    wl.p += (int64_t)wl.step * s0c;
    // all 16 steps of the chunk are requested at once (steps beyond its end repeat the last one and
    // are not multiplied): nothing but the activation is waited for once the chunk's tiles are there
    u32x4 ad[kChunkSteps];
    if (live) {  // on their way while the activation is waited for
#pragma unroll
        for (int k = 0; k < kChunkSteps; ++k) ad[k] = *reinterpret_cast<const u32x4*>(wl.p + wl.step * min(k, nst - 1));
    }
    unsigned long long launch = 0;  // (thread 0 only) launches before this one
    if (tid == 0) {
        launch = ld_agent(p.sync + kWordStride * kWordLaunches);
        launch = (unsigned long long)__builtin_amdgcn_readfirstlane((unsigned)launch) |  // (kept in scalar registers)
                 ((unsigned long long)__builtin_amdgcn_readfirstlane((unsigned)(launch >> 32)) << 32);
        const int tiles = min(kChunkK / kTileCols, p.UB - (kChunkK / kTileCols) * kc);
        const unsigned long long want = (launch + 1) * (unsigned long long)tiles;
        unsigned long long* word = p.sync + kWordStride * (kWordChunk0 + kc);
        unsigned long long* status = p.sync + kWordStride * kWordStatus;
        unsigned spins = 0;
        int fail = 0;
        while (ld_agent(word) < want) {
            __builtin_amdgcn_s_sleep(2);
            if (++spins > p.spin_limit) {
                st_agent(status, 1ull);
                fail = 1;
                break;
            }
            if ((spins & 63) == 0 && ld_agent(status) != 0) {
                fail = 1;
                break;
            }
        }
        s_fail = fail;
    }
    __syncthreads();
    if (s_fail == 0) {
        // the chunk of the activation: [M][512] through cache-bypassing loads into LDS
        const int per_row = nst * 4;  // 16-byte items
        int t1 = tid;  // (an opaque copy: what is derived from it does not live across the wait above)
        asm volatile("" : "+v"(t1));
        for (int e = t1; e < p.M * per_row; e += (int)blockDim.x) {  // (M = 8: one item per thread)
            const int m = e / per_row, j = e - m * per_row;
            *reinterpret_cast<u32x4*>(lds + m * kRowB + 16 * j) =
                ld_agent_x4_wait(reinterpret_cast<const u32x4*>(p.act + (int64_t)m * (p.I / 4) + s0c * 8) + j);
        }
        __syncthreads();
        if (live) {
            // (lane offsets recomputed from an opaque copy of the thread id: kept across the wait they
            // would hold registers next to the 64 of the weight fragments)
            int t2 = tid;
            asm volatile("" : "+v"(t2));
            const int r2 = t2 & 15, kq2 = (t2 >> 4) & 3;
            const unsigned char* xb = lds + min(r2, p.M - 1) * kRowB + 16 * kq2;
            acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k0 = 0; k0 < kChunkSteps; k0 += 4) {  // (four x operands at a time: registers)
#pragma unroll
                for (int k = k0; k < k0 + 4; ++k) {
                    if (k < nst) acc = mfma16<T>(ad[k], *reinterpret_cast<const u32x4*>(xb + 64 * k), acc);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (r2 < p.M) *reinterpret_cast<f32x4*>(p.dn_part + ((int64_t)kc * 16 + r2) * p.H + 16 * ct + 4 * kq2) = acc;
        }
    }
    // the last down workgroup of the launch advances the launch count (every other one has read it)
    __syncthreads();
    if (tid == 0) {
        const unsigned long long nd = (unsigned long long)p.GR * p.KC;
        if (add_agent(p.sync + kWordStride * kWordDone, 1ull) == (launch + 1) * nd - 1) {
            add_agent(p.sync + kWordStride * kWordLaunches, 1ull);
            if (p.head > 0) add_agent(p.sync + kWordStride * kWordHeadRows, (unsigned long long)p.head);
        }
    }
}

size_t mlp_lds_bytes(int M, int H) {
    const size_t xb = (size_t)M * (H + 8) * 2;
    const size_t red = (size_t)2 * kSlices * 16 * 17 * sizeof(float);
    const size_t xd = (size_t)M * kRowB;
    size_t n = xb > red ? xb : red;
    return n > xd ? n : xd;
}

}  // namespace

// Partial sums that ksa_mlp_rows leaves of the down projection: ceil(I / 512) slices [16][H].
extern "C" int ksa_mlp_rows_down_splits(int H, int I) {
    (void)H;
    return I > 0 ? (I / 32 + kChunkSteps - 1) / kChunkSteps : 0;
}

// Workspace: 32 KiB of counting words (to be zeroed once by the caller, and again after a launch
// left the status word non-zero), then the activation [16][I] and the norm stage's rows [16][H] in 16-bit.
extern "C" size_t ksa_mlp_rows_workspace_bytes(int H, int I) {
    if (H <= 0 || I <= 0) return 0;
    return (size_t)kSyncWords * 8 + (size_t)16 * I * 2 + (size_t)16 * H * 2;
}

namespace {

// x given (head == 0) or made by the norm stage of the launch (x null)
int mlp_rows_launch(const void* x, long long x_row_stride, const float* o_partials, int o_ksplit, const void* residual,
                    const void* norm_weight, void* out_sum, long long residual_row_stride, long long sum_row_stride,
                    float eps, const void* w_gate_up, const void* w_down, float* down_partials, int M, int H, int I,
                    long long w_gate_up_row_stride, long long w_down_row_stride, int dtype, void* workspace,
                    size_t workspace_bytes, void* stream) {
    if (!w_gate_up || !w_down || !down_partials || !workspace) return KSA_ERR_NULL;
    if (M <= 0 || M > 16 || H <= 0 || I <= 0) return KSA_ERR_INVALID;
    if (H % 128 != 0 || I % 32 != 0) return KSA_ERR_UNSUPPORTED;  // four K slices of whole steps; whole steps of the down K
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    const int KC = ksa_mlp_rows_down_splits(H, I);
    if (KC > kMaxChunks) return KSA_ERR_UNSUPPORTED;  // MLP sizes beyond 26624
    if (workspace_bytes < ksa_mlp_rows_workspace_bytes(H, I)) return KSA_ERR_WORKSPACE;
    auto bad = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) != 0; };
    if (bad(w_gate_up) || bad(w_down) || bad(down_partials) || bad(workspace)) return KSA_ERR_ALIGN;
    if ((w_gate_up_row_stride != kWTiled && w_gate_up_row_stride % 8) || (w_down_row_stride != kWTiled && w_down_row_stride % 8))
        return KSA_ERR_ALIGN;
    const size_t lds = mlp_lds_bytes(M, H);
    if (lds > 160 * 1024) return KSA_ERR_UNSUPPORTED;
    auto kern = dtype == KSA_DTYPE_BF16 ? ksa_mlp_rows_kernel<KsaBf16> : ksa_mlp_rows_kernel<KsaF16>;
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
        return KSA_ERR_LAUNCH;
    MlpParams p{};
    p.w_gu = (const uint16_t*)w_gate_up;
    p.w_dn = (const uint16_t*)w_down;
    p.dn_part = down_partials;
    p.sync = (unsigned long long*)workspace;
    p.act = p.sync + kSyncWords;
    p.hbuf = p.act + (size_t)16 * I / 4;
    p.wgu_rs = w_gate_up_row_stride, p.wdn_rs = w_down_row_stride;
    p.M = M, p.H = H, p.I = I;
    p.UB = I / kTileCols;
    p.GR = (H / 16 + 2 * kSlices - 1) / (2 * kSlices);
    p.KC = KC;
    p.spin_limit = 1u << 19;  // polls of a microsecond or two: about a second
    if (x) {
        if (bad(x)) return KSA_ERR_ALIGN;
        if (x_row_stride % 8) return KSA_ERR_ALIGN;
        p.x = (const uint16_t*)x;
        p.x_rs = x_row_stride;
    } else {
        if (!o_partials || !residual || !norm_weight || !out_sum) return KSA_ERR_NULL;
        if (o_ksplit < 1 || o_ksplit > 64) return KSA_ERR_INVALID;
        if (H > 4096) return KSA_ERR_UNSUPPORTED;  // a norm row is one 16-byte item per thread
        if (bad(o_partials) || bad(residual) || bad(norm_weight) || bad(out_sum)) return KSA_ERR_ALIGN;
        if (residual_row_stride % 8 || sum_row_stride % 8) return KSA_ERR_ALIGN;
        p.o_part = o_partials;
        p.o_ksplit = o_ksplit;
        p.res = (const uint16_t*)residual;
        p.norm_w = (const uint16_t*)norm_weight;
        p.out_sum = (uint16_t*)out_sum;
        p.res_rs = residual_row_stride, p.sum_rs = sum_row_stride;
        p.eps = eps;
        p.head = M;
    }
    hipLaunchKernelGGL(kern, dim3(p.head + p.UB + p.GR * p.KC), dim3(128 * kSlices), lds, (hipStream_t)stream, p);
    return ksa_check_launch();
}

}  // namespace

extern "C" int ksa_mlp_rows(const void* x, const void* w_gate_up, const void* w_down, float* down_partials, int M,
                            int H, int I, long long x_row_stride, long long w_gate_up_row_stride,
                            long long w_down_row_stride, int dtype, void* workspace, size_t workspace_bytes,
                            void* stream) {
    if (!x) return KSA_ERR_NULL;
    return mlp_rows_launch(x, x_row_stride, nullptr, 0, nullptr, nullptr, nullptr, 0, 0, 0.f, w_gate_up, w_down,
                           down_partials, M, H, I, w_gate_up_row_stride, w_down_row_stride, dtype, workspace,
                           workspace_bytes, stream);
}

extern "C" int ksa_add_rmsnorm_mlp_rows(const float* o_partials, int o_ksplit, const void* residual,
                                        const void* norm_weight, void* out_sum, const void* w_gate_up,
                                        const void* w_down, float* down_partials, int M, int H, int I,
                                        long long residual_row_stride, long long sum_row_stride,
                                        long long w_gate_up_row_stride, long long w_down_row_stride, int dtype,
                                        float eps, void* workspace, size_t workspace_bytes, void* stream) {
    if (!o_partials) return KSA_ERR_NULL;
    return mlp_rows_launch(nullptr, 0, o_partials, o_ksplit, residual, norm_weight, out_sum, residual_row_stride,
                           sum_row_stride, eps, w_gate_up, w_down, down_partials, M, H, I, w_gate_up_row_stride,
                           w_down_row_stride, dtype, workspace, workspace_bytes, stream);
}

// Status word of the workspace (device memory, 8 bytes at this offset): 0, or 1 after a launch in
// which a workgroup gave up waiting.
extern "C" size_t ksa_mlp_rows_status_offset(void) { return (size_t)kWordStride * kWordStatus * 8; }
