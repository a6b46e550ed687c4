// Row movers for the ring-buffer KV cache and the summary-prefix gather (gfx950).
//
// The reference moves cache rows with many small Tensor.copy_ calls:
//   examples/pretrain/hf_template/modeling_qwen3sa.py:306-336 (update_text: one row)
//   examples/pretrain/hf_template/modeling_qwen3sa.py:340-398 (update_summary: flush + append)
//   examples/pretrain/hf_template/modeling_qwen3sa.py:209-302 (reorganize_after_prefill: gathers)
// and gathers the summary rows of K/V with boolean indexing
//   summary_attn wheel, summary_attn/interface.py:276-278.
// One kernel covers all of them: it copies `nrows` rows of D 16-bit elements for every
// (sequence, head), source row i being src_index[i] (or src_start + i) and destination row
// dst_start + i, where dst_start may differ per sequence.
#include <hip/hip_runtime.h>

#include "ksa_api_internal.h"
#include "ksa_tile.h"

namespace {

struct CopyParams {
    const uint16_t* src;
    uint16_t* dst;
    const int32_t* src_index;      // [nrows] or null
    const int32_t* dst_start_seq;  // [batch] or null
    int src_start, dst_start, nrows, cpr;  // cpr = 16-byte chunks per row
    int64_t s_bs, s_hs, s_rs;
    int64_t d_bs, d_hs, d_rs;
};

__global__ __launch_bounds__(256) void ksa_copy_rows_kernel(const CopyParams p) {
    const int h = blockIdx.y, b = blockIdx.z;
    const int64_t total = (int64_t)p.nrows * p.cpr;
    const uint16_t* sb = p.src + b * p.s_bs + h * p.s_hs;
    uint16_t* db = p.dst + b * p.d_bs + h * p.d_hs;
    const int d0 = p.dst_start_seq ? p.dst_start_seq[b] : p.dst_start;
    for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < total;
         u += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(u / p.cpr), c = (int)(u % p.cpr);
        const int sr = p.src_index ? p.src_index[i] : p.src_start + i;
        *reinterpret_cast<u32x4*>(db + (int64_t)(d0 + i) * p.d_rs + 8 * c) =
            __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(sb + (int64_t)sr * p.s_rs + 8 * c));
    }
}

// Several independent row moves of one shape (same batch, heads, head_dim) as one launch: the moves of
// a chunk-boundary step (text row, summary rows into the scratch rows; afterwards the flush of the
// chunk into the ring and the append of its summaries, for K and for V) are eight launches otherwise.
constexpr int kMaxMoves = 8;
struct MultiCopyParams {
    CopyParams mv[kMaxMoves];
};

__global__ __launch_bounds__(256) void ksa_copy_rows_multi_kernel(const MultiCopyParams mp, int heads) {
    const int which = blockIdx.y / heads, h = blockIdx.y % heads, b = blockIdx.z;
    const CopyParams& p = mp.mv[which];
    const int64_t total = (int64_t)p.nrows * p.cpr;
    const uint16_t* sb = p.src + b * p.s_bs + h * p.s_hs;
    uint16_t* db = p.dst + b * p.d_bs + h * p.d_hs;
    const int d0 = p.dst_start_seq ? p.dst_start_seq[b] : p.dst_start;
    for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < total;
         u += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(u / p.cpr), c = (int)(u % p.cpr);
        *reinterpret_cast<u32x4*>(db + (int64_t)(d0 + i) * p.d_rs + 8 * c) =
            __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(sb + (int64_t)(p.src_start + i) * p.s_rs + 8 * c));
    }
}

}  // namespace

// n_moves <= 8 moves, move m: dst[m] row (dst_start[m] (+ dst_start_seq[m][sequence] instead, if given) + i)
// <- src[m] row (src_start[m] + i), i < nrows[m], for every (sequence, head).  The moves must not
// depend on each other (no move reads rows that another one writes): they run side by side.
extern "C" int ksa_copy_rows_multi(int n_moves, const void* const* src, void* const* dst,
                                   const int32_t* const* dst_start_seq, const int* src_start, const int* dst_start,
                                   const int* nrows, int batch, int heads, int D, const int64_t* src_strides,
                                   const int64_t* dst_strides, void* stream) {
    if (!src || !dst || !src_start || !dst_start || !nrows || !src_strides || !dst_strides) return KSA_ERR_NULL;
    if (n_moves <= 0 || n_moves > kMaxMoves || batch <= 0 || heads <= 0 || D <= 0 || D % 8 != 0) return KSA_ERR_INVALID;
    MultiCopyParams mp{};
    int64_t most = 0;
    for (int m = 0; m < n_moves; ++m) {
        if (!src[m] || !dst[m]) return KSA_ERR_NULL;
        if (nrows[m] < 0 || src_start[m] < 0 || dst_start[m] < 0) return KSA_ERR_INVALID;
        if ((reinterpret_cast<uintptr_t>(src[m]) | reinterpret_cast<uintptr_t>(dst[m])) & 15) return KSA_ERR_ALIGN;
        for (int i = 0; i < 3; ++i)
            if ((src_strides[3 * m + i] % 8) || (dst_strides[3 * m + i] % 8)) return KSA_ERR_ALIGN;
        CopyParams& p = mp.mv[m];
        p.src = (const uint16_t*)src[m];
        p.dst = (uint16_t*)dst[m];
        p.dst_start_seq = dst_start_seq ? dst_start_seq[m] : nullptr;
        p.src_start = src_start[m], p.dst_start = dst_start[m], p.nrows = nrows[m];
        p.cpr = D / 8;
        p.s_bs = src_strides[3 * m], p.s_hs = src_strides[3 * m + 1], p.s_rs = src_strides[3 * m + 2];
        p.d_bs = dst_strides[3 * m], p.d_hs = dst_strides[3 * m + 1], p.d_rs = dst_strides[3 * m + 2];
        const int64_t total = (int64_t)nrows[m] * p.cpr;
        if (total > most) most = total;
    }
    if (most == 0) return KSA_OK;
    int gx = (int)((most + 255) / 256);
    if (gx > 1024) gx = 1024;
    hipLaunchKernelGGL(ksa_copy_rows_multi_kernel, dim3(gx, heads * n_moves, batch), dim3(256), 0, (hipStream_t)stream,
                       mp, heads);
    return ksa_check_launch();
}

extern "C" int ksa_copy_rows(const void* src, void* dst, const int32_t* src_index,
                             const int32_t* dst_start_seq, int src_start, int dst_start, int nrows,
                             int batch, int heads, int D, const int64_t* src_strides,
                             const int64_t* dst_strides, void* stream) {
    if (!src || !dst || !src_strides || !dst_strides) return KSA_ERR_NULL;
    if (nrows == 0) return KSA_OK;
    if (nrows < 0 || batch <= 0 || heads <= 0 || D <= 0 || D % 8 != 0) return KSA_ERR_INVALID;
    if (src_start < 0 || dst_start < 0) return KSA_ERR_INVALID;
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) return KSA_ERR_ALIGN;
    for (int i = 0; i < 3; ++i)
        if ((src_strides[i] % 8) || (dst_strides[i] % 8)) return KSA_ERR_ALIGN;
    CopyParams p{};
    p.src = (const uint16_t*)src;
    p.dst = (uint16_t*)dst;
    p.src_index = src_index;
    p.dst_start_seq = dst_start_seq;
    p.src_start = src_start;
    p.dst_start = dst_start;
    p.nrows = nrows;
    p.cpr = D / 8;
    p.s_bs = src_strides[0], p.s_hs = src_strides[1], p.s_rs = src_strides[2];
    p.d_bs = dst_strides[0], p.d_hs = dst_strides[1], p.d_rs = dst_strides[2];
    const int64_t total = (int64_t)nrows * p.cpr;
    int gx = (int)((total + 255) / 256);
    if (gx > 1024) gx = 1024;
    hipLaunchKernelGGL(ksa_copy_rows_kernel, dim3(gx, heads, batch), dim3(256), 0,
                       (hipStream_t)stream, p);
    return ksa_check_launch();
}
