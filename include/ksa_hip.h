/* libksa_hip.so — C ABI of the MI355X (gfx950) Summary-Attention kernels.
 *
 * The reference (Kuaishou-OneRec/KSA) has no C/FFI boundary on these paths: its two
 * boundaries are Python call sites.  Each entry point below names the Python-level
 * reference interface it stands behind ("whl-sa" = summary_attn-0.3.0 wheel,
 * "whl-fa" = flash_attn_cute-0.1.0 wheel, "HF" =
 * examples/pretrain/hf_template/modeling_qwen3sa.py).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller unless stated otherwise;
 *     the library never allocates, frees or synchronises, keeps no state between calls (the one
 *     exception, a fixed scratch array, is described at ksa_decode_fwd_noalloc; ksa_mlp_rows keeps
 *     counting words in a workspace that the caller owns and zeroes once) and reads no
 *     environment variable;
 *   - `stream` is a hipStream_t passed as void* (0 = the null stream);
 *   - 16-bit tensors are described by element strides; pointers must be 16-byte
 *     aligned and strides multiples of 8 elements, the innermost (head_dim) stride is 1;
 *   - dtype: 0 = bf16, 1 = fp16; head_dim 64, 128 or 256 for the two attention entry points
 *     (any other multiple of 8 up to 256, which the reference also takes, is zero-padded to the
 *     next of these by the caller: the Python mirrors do), 64 or 128 for ksa_pre_attention;
 *   - return value 0 = launched, negative = rejected before any launch
 *     (see ksa_error_string).
 */
#ifndef KSA_HIP_H
#define KSA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KSA_OK 0
#define KSA_ERR_INVALID (-1)
#define KSA_ERR_NULL (-2)
#define KSA_ERR_UNSUPPORTED (-3)
#define KSA_ERR_WORKSPACE (-4)
#define KSA_ERR_LAUNCH (-5)
#define KSA_ERR_ALIGN (-6)

#define KSA_DTYPE_BF16 0
#define KSA_DTYPE_F16 1

int ksa_version(void);
const char* ksa_error_string(int code);
int ksa_device_cu_count(void);

/* Block-sparsity index.
 * Replaces whl-fa:flash_attn/cute/compute_block_sparsity.py:276-375 (compute_block_sparsity)
 * as called from whl-sa:summary_attn/interface.py:36-68 with (tile_m, tile_n, 1, 1, Sq, Sk)
 * and the predicate of whl-sa:summary_attn/mask.py chosen by (P > 0, skip_old).
 * P must equal Sk - Sq.  Outputs (int32, fully written, zero padded, ascending n):
 *   mask_cnt[M], mask_idx[M*N], full_cnt[M], full_idx[M*N],
 *   M = ceil(Sq/tile_m), N = ceil(Sk/tile_n). */
int ksa_block_index(int Sq, int Sk, int C, int S, int W, int P, int skip_old, int tile_m,
                    int tile_n, int32_t* mask_cnt, int32_t* mask_idx, int32_t* full_cnt,
                    int32_t* full_idx, void* stream);

/* Prefill forward.
 * Replaces whl-sa:summary_attn/interface.py:271-289 (summary_attn_func) ->
 * :70-91 (SummaryAttnFunc.forward) -> whl-fa:flash_attn/cute/interface.py:85-534
 * (_flash_attn_fwd with mask_mod + block_sparse_tensors, tiles 128 x 64).
 *   q   [batch, Sq, Hq, D]        strides {batch, row, head}
 *   k,v [batch, rows, Hkv, D]     one stride triple for both (kv_strides)
 *       phys_prefix == 0: rows = Sq in-line keys; prefix row j (j < P) is read in place
 *           from in-line row (j/S)*(C+S) + C + j%S -- what `k[:, summary_pos]` gathers
 *           when summary_pos is the periodic pattern; nothing is concatenated.
 *       phys_prefix != 0: rows = P + Sq, the layout the reference builds with
 *           torch.cat((k[:, summary_pos], k), dim=1).
 *       rows * row stride * 2 bytes must stay below 4 GiB.
 *   out [batch, Sq, Hq, D]; lse fp32 [batch, Hq, Sq] (natural log) or NULL.
 *   mask_cnt .. full_idx: output of ksa_block_index(Sq, Sq+P, ..., 128, 64), idx_stride = N.
 *   scale: soft-max scale (the reference uses head_dim^-0.5).
 *   shape: workgroup shape, a tuning knob with no effect on the result beyond the tolerance of
 *       the tests.  KSA_PREFILL_SHAPE_AUTO lets the library choose from the launch size and the
 *       device's CU count; the others apply to head_dim 128 with an even Hq / Hkv and fall back
 *       to one head per workgroup elsewhere.
 *   sched: NULL, or 8 int32 of device memory for this call alone (contents irrelevant on entry,
 *       undefined afterwards; calls that may overlap in time need one each).  With it, a long
 *       launch hands out its last, light work items from per-XCD queues (device-scope atomics)
 *       instead of a fixed split, so that XCDs running at slightly different clocks end together;
 *       one small extra kernel in front of the launch clears the counters.  No effect on the
 *       result. */
#define KSA_PREFILL_SHAPE_AUTO 0       /* library's choice */
#define KSA_PREFILL_SHAPE_1HEAD 32     /* one query head on 4 waves, 32 rows per wave */
#define KSA_PREFILL_SHAPE_2HEAD_64 64  /* two heads of a kv group on 4 waves, 64 rows per wave */
#define KSA_PREFILL_SHAPE_2HEAD 2      /* two heads of a kv group on 8 waves, 32 rows per wave */
int ksa_prefill_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int batch,
                    int Sq, int Hq, int Hkv, int D, int dtype, const int64_t* q_strides,
                    const int64_t* kv_strides, const int64_t* out_strides, int C, int S, int W,
                    int P, int skip_old, int phys_prefix, const int32_t* mask_cnt,
                    const int32_t* mask_idx, const int32_t* full_cnt, const int32_t* full_idx,
                    int idx_stride, float scale, int shape, int32_t* sched, void* stream);

/* Decode attention over the ring-buffer slice.
 * Replaces HF:591-612 (_sdpa_attention_forward, incl. repeat_kv :557-566) applied to the
 * slice of HF:402-434 (Qwen3RingBufferCache.get_attention_kv).
 *   q      [batch, Hq, Q, D]      strides {batch, head, query}
 *   kcache [batch, Hkv, rows, D]  strides {batch, head, row}   (same for vcache)
 *   out    [batch, Q, Hq, D]      strides {batch, query, head}
 *   rows attended for sequence b: [start[b], end[b]) if start/end (device int32[batch])
 *   are given, else [start0, end0) for every sequence.  No mask, no causality.
 *   nsplit >= 1 splits of the row range; nsplit > 1 needs a workspace of
 *   ksa_decode_workspace_bytes(...) bytes (fp32 partials). */
size_t ksa_decode_workspace_bytes(int batch, int Hq, int Hkv, int Q, int D, int nsplit);
int ksa_decode_auto_splits(int batch, int Hkv, int max_rows);
int ksa_decode_fwd(const void* q, const void* kcache, const void* vcache, void* out,
                   const int32_t* start, const int32_t* end, int start0, int end0, int batch,
                   int Hq, int Hkv, int Q, int D, int dtype, const int64_t* q_strides,
                   const int64_t* k_strides, const int64_t* v_strides, const int64_t* out_strides,
                   float scale, int nsplit, void* workspace, size_t workspace_bytes, void* stream);

/* Chunk-boundary decode step in one launch (HF:831-876, the two calls of the decode attention
 * function and the torch.cat behind them): query token 0 (the chunk's last text token) attends rows
 * [text_start, text_end), query tokens 1 .. Q - 1 (its summary tokens) attend [sum_start, sum_end),
 * both un-masked; each pair of bounds as device int32[batch] or, when NULL, the scalars behind it.
 * The two groups of columns read their rows separately (the text token's g columns do not ride
 * through the summary tokens' range and vice versa).  Everything else as ksa_decode_fwd; Q >= 2,
 * Hq / Hkv <= 32; workspace ksa_decode_boundary_workspace_bytes(...) bytes when nsplit > 1. */
size_t ksa_decode_boundary_workspace_bytes(int batch, int Hq, int Hkv, int Q, int D, int nsplit);
int ksa_decode_boundary_fwd(const void* q, const void* kcache, const void* vcache, void* out,
                            const int32_t* text_start, const int32_t* text_end, int text_start0, int text_end0,
                            const int32_t* sum_start, const int32_t* sum_end, int sum_start0, int sum_end0,
                            int batch, int Hq, int Hkv, int Q, int D, int dtype, const int64_t* q_strides,
                            const int64_t* k_strides, const int64_t* v_strides, const int64_t* out_strides,
                            float scale, int nsplit, void* workspace, size_t workspace_bytes, void* stream);

/* ksa_decode_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments and results as ksa_decode_fwd without the workspace: the split-K partials go to
 * a fixed array inside the library (KSA_DECODE_NOALLOC_SCRATCH_BYTES = 32 MiB of device memory
 * per GPU the library runs on, held until the process ends).  The call allocates and frees
 * nothing and does not synchronise.  A problem whose ksa_decode_workspace_bytes(...) exceeds
 * ksa_decode_noalloc_max_workspace_bytes() is rejected with KSA_ERR_WORKSPACE before any launch.
 * All calls on one GPU share the array: calls that overlap in time on one GPU (different
 * streams or host threads) race and must be serialised by the caller; back-to-back calls on one
 * stream are safe, nothing has to be cleared between them. */
#define KSA_DECODE_NOALLOC_SCRATCH_BYTES (32u << 20)
size_t ksa_decode_noalloc_max_workspace_bytes(void);
int ksa_decode_fwd_noalloc(const void* q, const void* kcache, const void* vcache, void* out,
                           const int32_t* start, const int32_t* end, int start0, int end0, int batch,
                           int Hq, int Hkv, int Q, int D, int dtype, const int64_t* q_strides,
                           const int64_t* k_strides, const int64_t* v_strides,
                           const int64_t* out_strides, float scale, int nsplit, void* stream);

/* Attention probabilities of a decode step, for callers that ask for them.
 * Replaces the second result of eager_attention_forward (HF:569-588; selected at HF:643-646 when
 * config._attn_implementation == "eager"):
 *   weights = softmax(q K^T * scale (+ mask), fp32).to(dtype)      [batch, Hq, Q, L]
 * over rows [start_b, end_b) of the cache as in ksa_decode_fwd (whose output the same call site
 * takes as attn_output); position j of a row is cache row start_b + j, positions past a sequence's
 * range hold 0, L >= the longest range.  mask: NULL, or additive values of the 16-bit dtype
 * addressed by mask_strides {batch, head, query token, position} in elements (0 = broadcast).
 * workspace: ksa_decode_weights_workspace_bytes(batch, Hq, Q, L) bytes (the fp32 scores), 16-byte
 * aligned.  Two launches; K is read once per kv head. */
size_t ksa_decode_weights_workspace_bytes(int batch, int Hq, int Q, int L);
int ksa_decode_weights(const void* q, const void* kcache, void* weights, const void* mask,
                       const int32_t* start, const int32_t* end, int start0, int end0, int batch, int Hq,
                       int Hkv, int Q, int D, int dtype, int L, const int64_t* q_strides,
                       const int64_t* k_strides, const int64_t* mask_strides, float scale, void* workspace,
                       size_t workspace_bytes, void* stream);

/* Cache row mover.
 * Replaces the Tensor.copy_ sequences of HF:306-336 (update_text), HF:340-398
 * (update_summary), HF:209-302 (reorganize_after_prefill) and the boolean gather of
 * whl-sa:summary_attn/interface.py:276-278.
 * For every (sequence, head): dst row (dst_start + i) <- src row (src_index ? src_index[i]
 * : src_start + i), i < nrows; dst_start_seq (device int32[batch]) overrides dst_start
 * per sequence.  Tensors are [batch, heads, rows, D] by strides {batch, head, row}. */
int ksa_copy_rows(const void* src, void* dst, const int32_t* src_index,
                  const int32_t* dst_start_seq, int src_start, int dst_start, int nrows, int batch,
                  int heads, int D, const int64_t* src_strides, const int64_t* dst_strides,
                  void* stream);

/* Up to 8 independent row moves of one shape (same batch, heads, D) as one launch; move m as
 * ksa_copy_rows without a source index list: dst[m] row (dst_start[m] + i, or dst_start_seq[m][b] + i
 * when that device array is given) <- src[m] row (src_start[m] + i), i < nrows[m].  src_strides /
 * dst_strides hold 3 strides {batch, head, row} per move.  No move may read rows that another one
 * writes.  The moves of a chunk-boundary step (HF:306-336 for its text token, HF:340-398 for the flush
 * and the append, the scratch-row copies of HF:476-497) are two such launches instead of twelve. */
int ksa_copy_rows_multi(int n_moves, const void* const* src, void* const* dst,
                        const int32_t* const* dst_start_seq, const int* src_start, const int* dst_start,
                        const int* nrows, int batch, int heads, int D, const int64_t* src_strides,
                        const int64_t* dst_strides, void* stream);

/* Pre-attention step: per-head RMSNorm of q and k, rotary embedding, layout write of q, k, v.
 * Replaces HF:660-666 (q_norm / k_norm = Qwen3RMSNorm HF:64-79 on head_dim, the three
 * .transpose(1, 2), apply_rotary_pos_emb HF:523-554 in its rotate_half form) and the
 * .transpose(1, 2).contiguous() copies in front of the attention call, with the rounding
 * points of the reference's 16-bit tensor ops.
 *   q [batch, S, Hq, D], k, v [batch, S, Hkv, D]: projection outputs, strides {batch, row, head}
 *   q_weight, k_weight [D]; cos, sin [batch or 1, S, D] with cos_strides {batch, row}
 *   q_out, k_out, v_out: any {batch, row, head} strides -- the [batch, S, H, D] layout of
 *   ksa_prefill_fwd, or rows of a [batch, H, capacity, D] cache tensor (pointer at the
 *   first destination row).  q_out may alias q, k_out k, v_out v (same strides).
 *   kv_out_row_seq: NULL, or int32 [batch] in device memory: sequence b's k and v go
 *   kv_out_row_seq[b] rows (of k_out_strides[1] / v_out_strides[1]) further down - the cache
 *   cursor of update_text (HF:306-336) when only the device knows it (graph replay); the
 *   caller guarantees the rows exist.  With kv_out_row_per_token != 0 the array is int32
 *   [batch][S] and names the destination row of every token's k and v outright, in place of its
 *   position: the text token and the summary tokens of a chunk-boundary step go to different
 *   places of the cache (update_text and the scratch rows of update_summary, HF:306-398). */
int ksa_pre_attention(const void* q, const void* k, const void* v, const void* q_weight,
                      const void* k_weight, const void* cos, const void* sin, void* q_out,
                      void* k_out, void* v_out, int batch, int S, int Hq, int Hkv, int D, int dtype,
                      const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                      const int64_t* q_out_strides, const int64_t* k_out_strides,
                      const int64_t* v_out_strides, const int64_t* cos_strides,
                      const int32_t* kv_out_row_seq, int kv_out_row_per_token, float eps,
                      void* stream);

/* ksa_pre_attention whose q | k | v rows are still the K-split partial sums of the fused qkv
 * projection (fp32 [ksplit][R][(Hq + 2 Hkv) D], R = batch * S rounded up to a multiple of 16, left by
 * ksa_gemm_rows called with out == NULL; row = batch index * S + position): summed in split order and
 * rounded first, so the outputs are bit-identical to the two-kernel form.  batch * S <= 128. */
int ksa_pre_attention_partials(const float* partials, int ksplit, const void* q_weight,
                               const void* k_weight, const void* cos, const void* sin, void* q_out,
                               void* k_out, void* v_out, int batch, int S, int Hq, int Hkv, int D,
                               int dtype, const int64_t* q_out_strides, const int64_t* k_out_strides,
                               const int64_t* v_out_strides, const int64_t* cos_strides,
                               const int32_t* kv_out_row_seq, int kv_out_row_per_token, float eps,
                      void* stream);

/* Residual add + RMSNorm over the hidden size, one pass.
 * Replaces Qwen3RMSNorm.forward (HF:64-79: fp32 normalisation, rounded to the 16-bit type, times
 * the 16-bit weight) together with the residual add in front of it (HF:946, :952).
 *   out_sum  = x + residual   (skipped when residual is null)
 *   out_norm = weight * round(s * rsqrt(mean(s^2) + eps)),  s = out_sum (or x)
 * rows x H elements, row strides in elements (multiples of 8), H a multiple of 8, H <= 8192.
 * out_sum may alias x or residual; out_norm may alias x when residual is null. */
int ksa_add_rmsnorm(const void* x, const void* residual, const void* weight, void* out_norm,
                    void* out_sum, long long rows, int H, long long x_row_stride,
                    long long residual_row_stride, long long norm_row_stride,
                    long long sum_row_stride, int dtype, float eps, void* stream);

/* ksa_add_rmsnorm whose x is not a tensor yet but the K-split partial sums that ksa_gemm_rows
 * leaves in its workspace when called with out == NULL (fp32 [ksplit][R][H], R = rows rounded up to a
 * multiple of 16): x = the sum over
 * the splits in split order, rounded to the 16-bit type.  out_sum is bit-identical to
 * ksa_gemm_rows with an output followed by ksa_add_rmsnorm; out_norm agrees to one unit in the
 * last place (the mean square is summed in a different order).  One launch less per o_proj /
 * down_proj -> residual add + norm (HF:944-952).  rows <= 128, H <= 8192; residual and out_sum
 * are required. */
int ksa_add_rmsnorm_partials(const float* partials, int ksplit, const void* residual,
                             const void* weight, void* out_norm, void* out_sum, int rows, int H,
                             long long residual_row_stride, long long norm_row_stride,
                             long long sum_row_stride, int dtype, float eps, void* stream);

/* out = round(SiLU(gate)) * up, the MLP activation of HF:507-514 (act_fn(gate_proj(x)) *
 * up_proj(x)) in one pass; gate and up may be the two halves of one fused projection output
 * (row strides in elements, multiples of 8; I a multiple of 8; rows < 2^31). */
int ksa_silu_mul(const void* gate, const void* up, void* out, long long rows, int I,
                 long long gate_row_stride, long long up_row_stride, long long out_row_stride,
                 int dtype, void* stream);

/* out[r] = index of the largest value of row r (the lowest such index; a NaN counts as the largest
 * value): the greedy token choice of a generation loop, torch.argmax(logits, dim=-1) of the
 * generate() that drives the reference's model (the reference itself leaves it to transformers),
 * in one small launch instead of the library's general reduction.  x [rows, N] of 16-bit values,
 * row stride in elements (a multiple of 8), out [rows] int64. */
int ksa_argmax_rows(const void* x, long long* out, int rows, int N, long long x_row_stride, int dtype,
                    void* stream);

/* ksa_silu_mul whose gate | up is still the K-split partial sums of the fused gate_up projection
 * (fp32 [ksplit][R][2 I], R = rows rounded up to a multiple of 16, left by ksa_gemm_rows called with
 * out == NULL): both halves are summed in split order and rounded first, so the result is bit-identical
 * to the two-kernel form.  rows <= 128. */
int ksa_silu_mul_partials(const float* partials, int ksplit, void* out, int rows, int I,
                          long long out_row_stride, int dtype, void* stream);

/* y = x W^T for at most 128 rows of x (decode steps), bound by the weight bytes.
 * Replaces torch.nn.functional.linear at the projections of a decode step (HF:628-641 q/k/v and
 * o projections, HF:507-514 MLP, HF:1338 lm_head), bias-free as in the reference's config.
 *   x [M, K], w [N, K], out [M, N], 16-bit, row strides in elements (x, w: multiples of 8);
 *   K a multiple of 32; fp32 accumulation, one rounding at the end.
 * ksplit > 1 splits K over workgroups and needs a device workspace for the partial sums:
 * ksa_gemm_rows_splits(M, N, K) gives the split count to use and ksa_gemm_rows_partials_bytes(M, N,
 * ksplit) the bytes (ksa_gemm_rows_auto_splits(N, K) and ksa_gemm_rows_workspace_bytes(N, ksplit) are
 * the same answers for M <= 16).  For M > 16 (a kernel of its own: every weight fragment meets each
 * 16-row block of x, staged through LDS in chunks of 512 elements of K) only split counts that
 * ksa_gemm_rows_splits can return are taken - slices are whole chunks, none empty - anything else is
 * KSA_ERR_INVALID.  With ksplit > 1 out may be NULL: the partial sums (fp32 [ksplit][R][N], R = M
 * rounded up to a multiple of 16) are then left in the workspace for a consumer that adds them itself
 * (ksa_add_rmsnorm_partials, ksa_silu_mul_partials, ksa_pre_attention_partials).  x and w 16-byte
 * aligned, for M > 16 the workspace as well (KSA_ERR_ALIGN otherwise). */
/* The streaming layout of a weight matrix.  The few-rows kernels read a weight fragment of 16 rows x 32
 * elements of K per wave instruction - in a row-major w [N, K] that is 64 bytes of each of 16 rows K elements
 * apart.  ksa_tile_weights writes the same matrix as [ceil(N / 16)][K / 32][16][32] (rows past N: zeros;
 * ksa_tile_weights_bytes(N, K) bytes, 16-byte aligned), in which a fragment is 1 KB in one piece and a wave's
 * share of the matrix one sequential run; a caller that has the memory keeps this second copy of the
 * projection weights for its decode steps (measured on the 4B-shape projections: q|k|v -7 %, down -15 %,
 * gate|up -10 % of the kernel time).  Such a matrix is passed as `w` with KSA_W_TILED in place of its row
 * stride to ksa_gemm_rows, ksa_gemm_rows_gate_up_silu (I a multiple of 16), ksa_mlp_rows and
 * ksa_add_rmsnorm_mlp_rows; results are bit-identical to the row-major call.  K a multiple of 32. */
#define KSA_W_TILED (-1LL)
size_t ksa_tile_weights_bytes(int N, int K);
int ksa_tile_weights(const void* w, void* out, int N, int K, long long w_row_stride, void* stream);

int ksa_gemm_rows_auto_splits(int N, int K);
size_t ksa_gemm_rows_workspace_bytes(int N, int ksplit);
int ksa_gemm_rows_splits(int M, int N, int K);
size_t ksa_gemm_rows_partials_bytes(int M, int N, int ksplit);
int ksa_gemm_rows(const void* x, const void* w, void* out, int M, int N, int K, long long x_row_stride,
                  long long w_row_stride, long long out_row_stride, int dtype, int ksplit,
                  void* workspace, size_t workspace_bytes, void* stream);

/* The MLP's gate | up projection with its activation folded in, for at most 128 rows of x:
 * out = round(SiLU(round(x w_gate^T))) * round(x w_up^T), one launch, no partial sums in memory.
 * Replaces act_fn(gate_proj(x)) * up_proj(x) of Qwen3MLP.forward (HF:507-514) at a decode step, i.e.
 * ksa_gemm_rows on the fused gate | up matrix followed by ksa_silu_mul (same rounding points; the
 * fp32 sums run over K in one chain instead of split-K order, so the 16-bit results can differ from
 * that pair's in the last place).
 *   x [M, K], w [2 I, K] (gate rows, then up rows), out [M, I]; K a multiple of 32; row strides in
 *   elements (x, w: multiples of 8).  Up to 16 rows x is held in LDS whole: M (K + 8) 2 bytes beyond
 *   160 KiB are KSA_ERR_UNSUPPORTED (use ksa_gemm_rows and ksa_silu_mul then); 17 to 128 rows go
 *   through LDS in chunks (any K), half of a workgroup's waves on gate columns, half on up columns
 *   (out 8-byte aligned then). */
int ksa_gemm_rows_gate_up_silu(const void* x, const void* w, void* out, int M, int I, int K,
                               long long x_row_stride, long long w_row_stride, long long out_row_stride,
                               int dtype, void* stream);

/* The MLP of a decoder layer for at most 16 rows as one launch that holds the workgroups of both
 * products; those of the down projection request their weights and then wait for the tiles of the
 * activation they need, which the gate | up workgroups count off in device memory (Qwen3MLP.forward,
 * HF:507-514):
 *   a = SiLU(x W_gate^T) * (x W_up^T)                        (like ksa_gemm_rows_gate_up_silu)
 *   down_partials[c] = a[:, 512 c : 512 c + 512] W_down[:, same]^T   for c < ksa_mlp_rows_down_splits(H, I)
 *   = ceil(I / 512),
 * i.e. the down projection as K-split partial sums [splits][16][H] fp32 for a consumer that adds
 * them (ksa_add_rmsnorm_partials).  Takes the place of ksa_gemm_rows_gate_up_silu + ksa_gemm_rows:
 * the weights of the down projection move while the activation is still being made, and no launch
 * ramp lies between the two products.
 *   x [M, H]; w_gate_up [2 I, H]; w_down [H, I]; H a multiple of 128 with M (H + 8) 2 bytes within
 *   160 KiB of LDS, I a multiple of 32 up to 26624; row strides in elements, multiples of 8.
 *   workspace: ksa_mlp_rows_workspace_bytes(H, I) bytes, 16-byte aligned, ZEROED ONCE by the caller
 *   before its first use and then left alone (its counting words go up from launch to launch);
 *   it belongs to one device and one pair (H, I), and launches that share it must not overlap.
 *   M may differ from launch to launch on one workspace, and launches with and without the norm
 *   stage of ksa_add_rmsnorm_mlp_rows may be mixed on it.
 *   What the kernel relies on: the workgroups of a launch are STARTED IN THE ORDER OF THEIR NUMBERS
 *   (a waiting workgroup depends only on workgroups with lower numbers, so those have been started
 *   and can finish).  HIP does not promise that order; the hardware dispatcher of gfx950 keeps it
 *   for a one-dimensional grid.  It can also be defeated from outside: a second launch on the same
 *   workspace that runs at the same time (another stream), or a CU mask / a co-tenant that leaves
 *   so few CUs that the launch takes longer than the bound below.  Every wait inside the kernel is
 *   therefore bounded: a workgroup that does not see its tiles arrive within
 *   about a second gives up, every workgroup that waits after it leaves at once, the launch ends
 *   normally, its output is unusable and the 8-byte word at
 *   ksa_mlp_rows_status_offset() of the workspace reads 1.  The caller then waits for the device to
 *   be idle, zeroes the workspace again and repeats the work with the two separate calls
 *   (ksa_gemm_rows_gate_up_silu + ksa_gemm_rows), which depend on no such order.
 *   KSA_ERR_UNSUPPORTED for sizes outside the above: use the two separate calls. */
int ksa_mlp_rows_down_splits(int H, int I);
size_t ksa_mlp_rows_workspace_bytes(int H, int I);
size_t ksa_mlp_rows_status_offset(void);
int ksa_mlp_rows(const void* x, const void* w_gate_up, const void* w_down, float* down_partials, int M, int H,
                 int I, long long x_row_stride, long long w_gate_up_row_stride, long long w_down_row_stride,
                 int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ksa_mlp_rows with the residual add + RMSNorm in front of the MLP in the same launch (HF:944-947):
 *   out_sum = residual + round(sum of the o_proj partial sums),  x = RMSNorm(out_sum) * norm_weight
 * by one workgroup per row at the head of the grid (arithmetic and summation order of
 * ksa_add_rmsnorm_partials; out_sum bit-identical, x to one unit in the last place), for whose rows
 * the gate | up workgroups wait with their first weights already requested.  Takes the place of
 * ksa_add_rmsnorm_partials + ksa_mlp_rows.  o_partials [o_ksplit][16][H] fp32 (ksa_gemm_rows with a
 * null output); residual, out_sum [M, H]; H up to 4096; the rest as ksa_mlp_rows, same workspace. */
int ksa_add_rmsnorm_mlp_rows(const float* o_partials, int o_ksplit, const void* residual, const void* norm_weight,
                             void* out_sum, const void* w_gate_up, const void* w_down, float* down_partials, int M,
                             int H, int I, long long residual_row_stride, long long sum_row_stride,
                             long long w_gate_up_row_stride, long long w_down_row_stride, int dtype, float eps,
                             void* workspace, size_t workspace_bytes, void* stream);

/* Host-side diagnostic: number of key columns in [a, b) visible to query row q under the
 * closed-form rule the kernels use (no GPU involved). */
long long ksa_debug_count_visible(long long q, long long a, long long b, int C, int S, int W,
                                  int P, int skip_old, int Sq, int Sk);

#ifdef __cplusplus
}
#endif
#endif /* KSA_HIP_H */
