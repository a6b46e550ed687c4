// Block-sparsity index for Summary Attention on gfx950.
//
// Produces the four int32 tensors of the reference's BlockSparsityKernel
//   flash_attn_cute wheel, flash_attn/cute/compute_block_sparsity.py:189-274
// (mask_block_cnt[M], mask_block_idx[M,N], full_block_cnt[M], full_block_idx[M,N];
//  zero padded, ascending n; classification over in-bounds elements only),
// but from the closed-form row counts in ksa_mask.h: one thread owns one
// n-tile of an m-tile and counts, row by row, how many of its columns are
// visible.  One workgroup per m-tile compacts the classes with wave ballots,
// which keeps the lists ascending without atomics.
#include <hip/hip_runtime.h>

#include "ksa_api_internal.h"
#include "ksa_mask.h"

namespace {

constexpr int kIdxThreads = 256;

__global__ __launch_bounds__(kIdxThreads) void ksa_block_index_kernel(
    KsaMask mk, int tile_m, int tile_n, int N, int32_t* __restrict__ mask_cnt,
    int32_t* __restrict__ mask_idx, int32_t* __restrict__ full_cnt,
    int32_t* __restrict__ full_idx) {
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    constexpr int kWaves = kIdxThreads / 64;
    __shared__ int s_part[kWaves], s_full[kWaves];

    const int q0 = m * tile_m;
    const int q1 = min(mk.Sq, q0 + tile_m);
    int32_t* mrow = mask_idx + (size_t)m * N;
    int32_t* frow = full_idx + (size_t)m * N;
    int run_part = 0, run_full = 0;

    for (int base = 0; base < N; base += kIdxThreads) {
        const int n = base + tid;
        int cls = 0;  // 0 empty, 1 partial, 2 full
        if (n < N) {
            const int32_t a = n * tile_n;
            const int32_t b = ksa_imin(mk.Sk, a + tile_n);
            const int32_t width = b - a;
            bool any_vis = false, any_hid = false;
            // every rule is causal in the key's sequence position (column - P): a tile that
            // starts behind the last row of the m-tile is empty, no rows to look at
            const int q_end = a >= mk.P + q1 ? q0 : q1;
            for (int q = q0; q < q_end; ++q) {
                const int32_t cnt = ksa_count_visible(mk, q, a, b);
                any_vis |= cnt > 0;
                any_hid |= cnt < width;
            }
            cls = any_vis ? (any_hid ? 1 : 2) : 0;
        }
        const uint64_t bp = __ballot(cls == 1);
        const uint64_t bf = __ballot(cls == 2);
        if (lane == 0) {
            s_part[wave] = __popcll(bp);
            s_full[wave] = __popcll(bf);
        }
        __syncthreads();
        int off_p = run_part, off_f = run_full, tot_p = 0, tot_f = 0;
        for (int w = 0; w < kWaves; ++w) {
            if (w < wave) {
                off_p += s_part[w];
                off_f += s_full[w];
            }
            tot_p += s_part[w];
            tot_f += s_full[w];
        }
        const uint64_t below = (1ull << lane) - 1ull;
        if (cls == 1) mrow[off_p + __popcll(bp & below)] = n;
        if (cls == 2) frow[off_f + __popcll(bf & below)] = n;
        run_part += tot_p;
        run_full += tot_f;
        __syncthreads();
    }
    // zero the unused tails so callers may hand in uninitialised buffers
    for (int i = run_part + tid; i < N; i += kIdxThreads) mrow[i] = 0;
    for (int i = run_full + tid; i < N; i += kIdxThreads) frow[i] = 0;
    if (tid == 0) {
        mask_cnt[m] = run_part;
        full_cnt[m] = run_full;
    }
}

}  // namespace

extern "C" int ksa_block_index(int Sq, int Sk, int C, int S, int W, int P, int skip_old, int tile_m,
                               int tile_n, int32_t* mask_cnt, int32_t* mask_idx, int32_t* full_cnt,
                               int32_t* full_idx, void* stream) {
    if (Sq <= 0 || Sk < Sq || C <= 0 || S <= 0 || W < 0 || tile_m <= 0 || tile_n <= 0)
        return KSA_ERR_INVALID;
    if (P != Sk - Sq) return KSA_ERR_INVALID;
    if (!mask_cnt || !mask_idx || !full_cnt || !full_idx) return KSA_ERR_NULL;
    const int M = (Sq + tile_m - 1) / tile_m;
    const int N = (Sk + tile_n - 1) / tile_n;
    KsaMask mk{C, S, W, P, skip_old ? 1 : 0, Sq, Sk};
    hipLaunchKernelGGL(ksa_block_index_kernel, dim3(M), dim3(kIdxThreads), 0, (hipStream_t)stream,
                       mk, tile_m, tile_n, N, mask_cnt, mask_idx, full_cnt, full_idx);
    return ksa_check_launch();
}

extern "C" long long ksa_debug_count_visible(long long q, long long a, long long b, int C, int S,
                                             int W, int P, int skip_old, int Sq, int Sk) {
    KsaMask mk{C, S, W, P, skip_old ? 1 : 0, Sq, Sk};
    if (a < 0) a = 0;
    if (b > Sk) b = Sk;
    if (b <= a) return 0;
    return ksa_count_visible(mk, (int)q, (int)a, (int)b);
}
