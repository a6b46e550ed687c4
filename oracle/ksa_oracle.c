/* CPU oracle in C for the KSA attention hot paths.  TEST INFRASTRUCTURE ONLY:
 * only tests, the smoke check and the benchmark's CPU-baseline leg load this.
 *
 * Restates (does not copy) the reference algorithm:
 *   summary_attention_kernel/summary_attn-0.3.0 wheel, summary_attn/mask.py:5-117
 *       the four visibility predicates (floor division on kv - P < 0)
 *   summary_attention_kernel/flash_attn_cute-0.1.0 wheel,
 *       flash_attn/cute/compute_block_sparsity.py:189-274,312-332
 *       tile classification over in-bounds elements, ascending index lists
 *   examples/pretrain/hf_template/modeling_qwen3sa.py:557-612
 *       decode = un-masked softmax(q k^T / sqrt(D)) v with kv_head = q_head / g
 *
 * Every function here evaluates the predicate element by element; nothing is
 * shared with the closed forms the GPU code uses.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline int64_t fdiv(int64_t a, int64_t b) { /* floor division, b > 0 */
    int64_t q = a / b;
    return (a % b != 0 && a < 0) ? q - 1 : q;
}
static inline int64_t fmod_(int64_t a, int64_t b) { return a - fdiv(a, b) * b; }

int ksa_oracle_visible(int64_t q, int64_t kv, int C, int S, int W, int P, int skip_old) {
    const int64_t B = C + S;
    const int64_t qc = q / B;
    const int is_q_sum = (q % B) >= C;
    if (P > 0) {
        const int64_t kvp = kv - P;
        const int64_t kc = fdiv(kvp, B);
        const int is_sliding = (qc - kc) <= W;
        const int is_kv_sum = fmod_(kvp, B) >= C;
        const int causal = q >= kvp;
        const int v_sum_q = is_q_sum && kc == qc && causal;
        const int v_slide = is_sliding && !is_kv_sum && kv >= P;
        int v_text_q;
        if (skip_old) v_text_q = !is_q_sum && causal && v_slide;
        else {
            const int v_old = (kv / S + W) < qc;
            v_text_q = !is_q_sum && ((causal && v_slide) || v_old);
        }
        return v_sum_q || v_text_q;
    } else {
        const int64_t kc = kv / B;
        const int is_sliding = (qc - kc) <= W;
        const int is_kv_sum = (kv % B) >= C;
        const int causal = q >= kv;
        const int v_sum_q = is_q_sum && kc == qc && causal;
        const int v_slide = is_sliding && !is_kv_sum;
        int v_text_q;
        if (skip_old) v_text_q = !is_q_sum && causal && v_slide;
        else {
            const int v_old = is_kv_sum && (qc - kc) > W;
            v_text_q = !is_q_sum && causal && (v_slide || v_old);
        }
        return v_sum_q || v_text_q;
    }
}

/* Brute-force block index.  Arrays: mask_cnt[M], mask_idx[M*N], full_cnt[M],
 * full_idx[M*N]; all fully written (zero padded).  Returns total visible pairs. */
int64_t ksa_oracle_block_index(int Sq, int Sk, int C, int S, int W, int P, int skip_old,
                               int tile_m, int tile_n, int32_t* mask_cnt, int32_t* mask_idx,
                               int32_t* full_cnt, int32_t* full_idx) {
    const int M = (Sq + tile_m - 1) / tile_m;
    const int N = (Sk + tile_n - 1) / tile_n;
    int64_t pairs = 0;
#pragma omp parallel for schedule(dynamic, 1) reduction(+ : pairs)
    for (int m = 0; m < M; ++m) {
        int nm = 0, nf = 0;
        int32_t* mi = mask_idx + (size_t)m * N;
        int32_t* fi = full_idx + (size_t)m * N;
        memset(mi, 0, sizeof(int32_t) * N);
        memset(fi, 0, sizeof(int32_t) * N);
        const int q0 = m * tile_m, q1 = (q0 + tile_m < Sq) ? q0 + tile_m : Sq;
        for (int n = 0; n < N; ++n) {
            const int k0 = n * tile_n, k1 = (k0 + tile_n < Sk) ? k0 + tile_n : Sk;
            int has_un = 0, has_ma = 0;
            for (int q = q0; q < q1; ++q)
                for (int kv = k0; kv < k1; ++kv) {
                    if (ksa_oracle_visible(q, kv, C, S, W, P, skip_old)) { has_un = 1; ++pairs; }
                    else has_ma = 1;
                }
            if (has_un && has_ma) mi[nm++] = n;
            else if (has_un) fi[nf++] = n;
        }
        mask_cnt[m] = nm;
        full_cnt[m] = nf;
    }
    return pairs;
}

/* Masked attention for selected query rows, fp32 inputs, double accumulation.
 * q [Sq,Hq,D], k/v [Sk,Hkv,D] with the P prefix rows already in place.
 * rows[nrows] = query rows to compute; out [nrows,Hq,D], lse [Hq,nrows]. */
void ksa_oracle_attention_rows(const float* q, const float* k, const float* v, int Sq, int Sk,
                               int Hq, int Hkv, int D, int C, int S, int W, int P, int skip_old,
                               float scale, const int32_t* rows, int nrows, float* out,
                               float* lse) {
    const int g = Hq / Hkv;
#pragma omp parallel for schedule(dynamic, 4) collapse(2)
    for (int r = 0; r < nrows; ++r)
        for (int h = 0; h < Hq; ++h) {
            const int qi = rows[r];
            const float* qv = q + ((size_t)qi * Hq + h) * D;
            const int hk = h / g;
            double m = -INFINITY, l = 0.0;
            double* acc = (double*)calloc(D, sizeof(double));
            for (int kv = 0; kv < Sk; ++kv) {
                if (!ksa_oracle_visible(qi, kv, C, S, W, P, skip_old)) continue;
                const float* kr = k + ((size_t)kv * Hkv + hk) * D;
                const float* vr = v + ((size_t)kv * Hkv + hk) * D;
                double s = 0.0;
                for (int d = 0; d < D; ++d) s += (double)qv[d] * (double)kr[d];
                s *= scale;
                if (s > m) {
                    const double c = exp(m - s);
                    l *= c;
                    for (int d = 0; d < D; ++d) acc[d] *= c;
                    m = s;
                }
                const double p = exp(s - m);
                l += p;
                for (int d = 0; d < D; ++d) acc[d] += p * (double)vr[d];
            }
            float* o = out + ((size_t)r * Hq + h) * D;
            for (int d = 0; d < D; ++d) o[d] = (float)(l > 0 ? acc[d] / l : 0.0);
            lse[(size_t)h * nrows + r] = (float)(l > 0 ? m + log(l) : -INFINITY);
            free(acc);
        }
}

/* Un-masked decode attention.  q [Bz,Hq,Q,D]; k/v rows of sequence b, kv-head h
 * start at k + b*k_bs + h*k_hs (element strides), row stride D.
 * rows [start[b], end[b]) are attended.  out [Bz,Q,Hq,D]. */
void ksa_oracle_decode(const float* q, const float* k, const float* v, int Bz, int Hq, int Hkv,
                       int Q, int D, int64_t k_bs, int64_t k_hs, const int32_t* start,
                       const int32_t* end, float scale, float* out) {
    const int g = Hq / Hkv;
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
    for (int b = 0; b < Bz; ++b)
        for (int h = 0; h < Hq; ++h) {
            const float* kb = k + (size_t)b * k_bs + (size_t)(h / g) * k_hs;
            const float* vb = v + (size_t)b * k_bs + (size_t)(h / g) * k_hs;
            double* acc = (double*)malloc(sizeof(double) * D);
            for (int qi = 0; qi < Q; ++qi) {
                const float* qv = q + (((size_t)b * Hq + h) * Q + qi) * D;
                double m = -INFINITY, l = 0.0;
                for (int d = 0; d < D; ++d) acc[d] = 0.0;
                for (int r = start[b]; r < end[b]; ++r) {
                    const float* kr = kb + (size_t)r * D;
                    const float* vr = vb + (size_t)r * D;
                    double s = 0.0;
                    for (int d = 0; d < D; ++d) s += (double)qv[d] * (double)kr[d];
                    s *= scale;
                    if (s > m) {
                        const double c = exp(m - s);
                        l *= c;
                        for (int d = 0; d < D; ++d) acc[d] *= c;
                        m = s;
                    }
                    const double p = exp(s - m);
                    l += p;
                    for (int d = 0; d < D; ++d) acc[d] += p * (double)vr[d];
                }
                float* o = out + (((size_t)b * Q + qi) * Hq + h) * D;
                for (int d = 0; d < D; ++d) o[d] = (float)(acc[d] / l);
            }
            free(acc);
        }
}
