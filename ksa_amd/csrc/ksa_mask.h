// Summary-Attention visibility rule in closed form (host + device).
//
// The rule is the one of the reference predicates
//   summary_attn wheel, summary_attn/mask.py:5-31   (in-line summaries, P == 0)
//   summary_attn wheel, summary_attn/mask.py:33-59  (prefix summaries,  P  > 0)
//   summary_attn wheel, summary_attn/mask.py:65-117 (skip_old_summary variants)
// restated as a union of intervals per query row instead of a per-element
// predicate, so that a tile can be classified or masked in O(1) per row.
//
// All positions are int32: callers guarantee Sk < 2^30.
// Coordinates: query row q in [0,Sq); key column kv in [0,Sk), Sk = P + Sq.
// With B = C + S, chunk c = q / B, offset o = q % B (summary row iff o >= C):
//   text row:    [0, X)  with X = max(0, c-W)*S                  (old summaries, prefix mode)
//                u  { kv >= max(P + max(0,c-W)*B, X) : kv-P <= q, (kv-P) % B < C }   (window + own chunk text)
//   summary row: [P + c*B, P + q + 1)
// In-line mode (P == 0) replaces [0, X) by the in-line summary rows of chunks < c-W.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define KSA_HD __host__ __device__ __forceinline__
#else
#define KSA_HD static inline
#endif

struct KsaMask {
    int C, S, W, P, skip_old;
    int Sq, Sk;
};

KSA_HD int32_t ksa_imax(int32_t a, int32_t b) { return a > b ? a : b; }
KSA_HD int32_t ksa_imin(int32_t a, int32_t b) { return a < b ? a : b; }

// number of text rows (offset < C) among in-line rows [0, x), x >= 0
KSA_HD int32_t ksa_text_below(int32_t x, int C, int B) {
    const int32_t r = x % B;
    return (x / B) * C + (r < C ? r : C);
}

// number of text rows among in-line rows [lo, hi)
KSA_HD int32_t ksa_text_in(int32_t lo, int32_t hi, int C, int B) {
    if (lo < 0) lo = 0;
    if (hi <= lo) return 0;
    return ksa_text_below(hi, C, B) - ksa_text_below(lo, C, B);
}

// Number of key columns in [a, b) (already clipped to [0, Sk)) visible to row q.
KSA_HD int32_t ksa_count_visible(const KsaMask& mk, int32_t q, int32_t a, int32_t b) {
    const int B = mk.C + mk.S;
    const int32_t c = q / B;
    const int32_t o = q % B;
    const int32_t P = mk.P;
    if (o >= mk.C) {  // summary row: own chunk, causal
        const int32_t lo = ksa_imax(a, P + c * B), hi = ksa_imin(b, P + q + 1);
        return hi > lo ? hi - lo : 0;
    }
    const int32_t w0 = c > mk.W ? c - mk.W : 0;  // first chunk of the text window
    int32_t n = 0;
    if (P > 0) {
        const int32_t X = mk.skip_old ? 0 : w0 * mk.S;
        {   // old summaries: kv in [0, X)
            const int32_t hi = ksa_imin(b, X);
            if (hi > a) n += hi - a;
        }
        // window text + own text, kv >= max(P + w0*B, X)
        const int32_t lo = ksa_imax(ksa_imax(a, P + w0 * B), X) - P;
        const int32_t hi = ksa_imin(b, P + q + 1) - P;
        n += ksa_text_in(lo, hi, mk.C, B);
    } else {
        const int32_t hi_all = ksa_imin(b, q + 1);
        // window text + own text
        n += ksa_text_in(ksa_imax(a, w0 * B), hi_all, mk.C, B);
        if (!mk.skip_old) {  // in-line summary rows of chunks < w0
            const int32_t lo = a, hi = ksa_imin(hi_all, w0 * B);
            if (hi > lo) n += (hi - lo) - ksa_text_in(lo, hi, mk.C, B);
        }
    }
    return n;
}

#if defined(__HIPCC__)
// bits t in [lo, hi) of a 64-bit tile mask
__device__ __forceinline__ uint64_t ksa_range_bits(int lo, int hi) {
    if (lo < 0) lo = 0;
    if (hi > 64) hi = 64;
    if (hi <= lo) return 0ull;
    const uint64_t up = (hi == 64) ? ~0ull : ((1ull << hi) - 1ull);
    return up & ~((1ull << lo) - 1ull);
}

// Per-lane classification of the 64 key columns [n0, n0+64): lane t answers for
// column n0+t.  text = in range and a text row of the in-line sequence that a
// text query may see through the window; valid = column < Sk.
__device__ __forceinline__ void ksa_tile_column_bits(const KsaMask& mk, int n0, int lane,
                                                     uint64_t& text, uint64_t& valid) {
    const int kv = n0 + lane;
    const int B = mk.C + mk.S;
    const bool in = kv < mk.Sk;
    const bool is_text = in && kv >= mk.P && ((kv - mk.P) % B) < mk.C;
    text = __ballot(is_text);
    valid = __ballot(in);
}

// 64-bit visibility mask of row q over columns [n0, n0+64).
__device__ __forceinline__ uint64_t ksa_row_bits(const KsaMask& mk, int q, int n0, uint64_t text,
                                                 uint64_t valid) {
    const int B = mk.C + mk.S;
    const int32_t c = q / B;
    const int32_t o = q % B;
    const int32_t P = mk.P;
    if (o >= mk.C) return ksa_range_bits(P + c * B - n0, P + q + 1 - n0) & valid;
    const int32_t w0 = c > mk.W ? c - mk.W : 0;
    if (P > 0) {
        const int32_t X = mk.skip_old ? 0 : w0 * mk.S;
        const uint64_t old_bits = ksa_range_bits(-n0, X - n0) & valid;
        const int32_t lo = ksa_imax(P + w0 * B, X);
        return old_bits | (ksa_range_bits(lo - n0, P + q + 1 - n0) & text);
    }
    const uint64_t causal = ksa_range_bits(-n0, q + 1 - n0);
    uint64_t vis = ksa_range_bits(w0 * B - n0, 64) & text;
    if (!mk.skip_old) vis |= ksa_range_bits(-n0, w0 * B - n0) & ~text & valid;
    return vis & causal;
}
#endif
