"""CPU oracle for the two KSA attention hot paths.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the algorithm of the reference for
  * the four Summary-Attention mask predicates,
  * the block-sparsity index (partial / full tile lists),
  * masked GQA attention (prefill forward) and its log-sum-exp,
  * un-masked decode attention over a contiguous KV slice,
  * the ring-buffer KV-cache state machine.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may
import it; the product package never does.

Reference files followed ("whl-sa" = summary_attn-0.3.0 wheel, "whl-fa" =
flash_attn_cute-0.1.0 wheel, both under summary_attention_kernel/):
  whl-sa:summary_attn/mask.py:5-117                      predicates
  whl-sa:summary_attn/interface.py:271-289               prefix-summary K/V layout
  whl-fa:flash_attn/cute/compute_block_sparsity.py:189-274,312-332   tile classes
  muse/layers/summary_attention_func.py:506-584          interval form of the mask
  whl-sa:summary_attn/utils.py:80-125                    GQA head order
  examples/pretrain/hf_template/modeling_qwen3sa.py:85-505,557-612   cache + decode

Pinning status of each function (what fixes it besides its own formula) is
listed in tests/test_oracle.py; nothing here is pinned by a reference-held
vector because the reference ships no tests or fixtures.
"""
from __future__ import annotations

import numpy as np


# ----------------------------------------------------------------------------
# Mask predicates  (whl-sa:summary_attn/mask.py)
# numpy's // and % are floor division / non-negative modulo, which is what the
# rule needs for kv - P < 0 (prefix rows).
# ----------------------------------------------------------------------------

def mask_predicate(q, kv, C, S, W, P=0, skip_old=False):
    """Elementwise visibility of key column `kv` for query row `q`.

    P == 0 -> in-line summaries   (mask.py:5-31, skip_old: 65-90)
    P  > 0 -> prefix summaries    (mask.py:33-59, skip_old: 92-117)
    """
    q = np.asarray(q, dtype=np.int64)
    kv = np.asarray(kv, dtype=np.int64)
    B = C + S
    qc = q // B
    is_q_sum = (q % B) >= C
    if P > 0:
        kvp = kv - P
        kc = kvp // B
        is_sliding = (qc - kc) <= W
        is_kv_sum = (kvp % B) >= C
        causal = q >= kvp
        v_sum_q = is_q_sum & (kc == qc) & causal
        v_slide = is_sliding & (~is_kv_sum) & (kv >= P)
        if skip_old:
            v_text_q = (~is_q_sum) & causal & v_slide
        else:
            v_old = ((kv // S) + W) < qc
            v_text_q = (~is_q_sum) & ((causal & v_slide) | v_old)
        return v_sum_q | v_text_q
    kc = kv // B
    is_sliding = (qc - kc) <= W
    is_kv_sum = (kv % B) >= C
    causal = q >= kv
    v_sum_q = is_q_sum & (kc == qc) & causal
    v_slide = is_sliding & (~is_kv_sum)
    if skip_old:
        v_text_q = (~is_q_sum) & causal & v_slide
    else:
        v_old = is_kv_sum & ((qc - kc) > W)
        v_text_q = (~is_q_sum) & causal & (v_slide | v_old)
    return v_sum_q | v_text_q


def dense_mask_predicate(Sq, C, S, W, P=0, skip_old=False):
    """Dense bool [Sq, P+Sq] from the predicate form."""
    q = np.arange(Sq)[:, None]
    kv = np.arange(Sq + P)[None, :]
    return mask_predicate(q, kv, C, S, W, P, skip_old)


def dense_mask_intervals(Sq, C, S, W, skip_old=False):
    """Dense bool [Sq, Sq], in-line layout, built chunk by chunk from index
    sets (muse/layers/summary_attention_func.py:506-584).  Unlike the
    reference builder this accepts a trailing partial chunk of text rows
    (no summaries), which is what HF prefill produces (HF template :1091-1132).
    """
    B = C + S
    n_full = Sq // B
    tail = Sq - n_full * B
    assert tail <= C, "a trailing partial chunk holds text rows only"
    mask = np.zeros((Sq, Sq), dtype=bool)
    text = [np.arange(c * B, c * B + C) for c in range(n_full)]
    summ = [np.arange(c * B + C, (c + 1) * B) for c in range(n_full)]
    if tail:
        text.append(np.arange(n_full * B, Sq))
        summ.append(np.arange(0))
    for c in range(len(text)):
        t, s = text[c], summ[c]
        w0 = max(0, c - W)
        if w0 > 0 and not skip_old:
            old = np.concatenate(summ[:w0])
            mask[np.ix_(t, old)] = True
        if w0 < c:
            prev = np.concatenate(text[w0:c])
            mask[np.ix_(t, prev)] = True
        mask[np.ix_(t, t)] = np.tril(np.ones((len(t), len(t)), dtype=bool))
        if len(s):
            mask[np.ix_(s, t)] = True
            mask[np.ix_(s, s)] = np.tril(np.ones((len(s), len(s)), dtype=bool))
    return mask


def summary_positions(Sq, C, S):
    """summary_pos[i] = row i is a summary row; a trailing partial chunk has none."""
    B = C + S
    i = np.arange(Sq)
    n_full = Sq // B
    return ((i % B) >= C) & (i < n_full * B)


def prefix_to_inline_row(j, C, S):
    """Prefix row j holds the K/V of in-line row (j//S)*B + C + j%S
    (boolean-mask gather keeps order, whl-sa:interface.py:277-278)."""
    j = np.asarray(j)
    return (j // S) * (C + S) + C + (j % S)


def visible_count_text(c, o, C, S, W):
    """Closed form: number of keys a text row (chunk c, offset o) sees."""
    return S * max(0, c - W) + C * min(c, W) + o + 1


def visible_count_summary(k, C):
    """Closed form: keys seen by the k-th summary row of a chunk."""
    return C + k + 1


# ----------------------------------------------------------------------------
# Block-sparsity index (whl-fa:compute_block_sparsity.py:189-274, 312-332)
# ----------------------------------------------------------------------------

def block_index(Sq, Sk, C, S, W, P, skip_old=False, tile_m=128, tile_n=64):
    """Brute-force tile classifier over the predicate, in-bounds elements only.

    Returns (mask_cnt[M], mask_idx[M,N], full_cnt[M], full_idx[M,N]) int32,
    zero padded, indices ascending in n.
    """
    M = -(-Sq // tile_m)
    N = -(-Sk // tile_n)
    mask_cnt = np.zeros(M, np.int32)
    full_cnt = np.zeros(M, np.int32)
    mask_idx = np.zeros((M, N), np.int32)
    full_idx = np.zeros((M, N), np.int32)
    kv = np.arange(Sk)[None, :]
    pad = N * tile_n - Sk
    width = np.full(N, tile_n, np.int64)
    if pad:
        width[-1] = tile_n - pad
    for m in range(M):
        q = np.arange(m * tile_m, min(Sq, (m + 1) * tile_m))[:, None]
        vis = mask_predicate(q, kv, C, S, W, P, skip_old)
        per_col = vis.sum(axis=0)
        if pad:
            per_col = np.concatenate([per_col, np.zeros(pad, per_col.dtype)])
        a = per_col.reshape(N, tile_n).sum(axis=1)
        total = q.shape[0] * width
        partial = np.nonzero((a > 0) & (a < total))[0]
        full = np.nonzero(a == total)[0]
        mask_cnt[m] = len(partial)
        full_cnt[m] = len(full)
        mask_idx[m, : len(partial)] = partial
        full_idx[m, : len(full)] = full
    return mask_cnt, mask_idx, full_cnt, full_idx


# ----------------------------------------------------------------------------
# Masked attention (textbook; GQA head map kv_head = q_head // g)
# ----------------------------------------------------------------------------

def _softmax_rows(s, vis):
    s = np.where(vis, s, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    l = e.sum(axis=-1, keepdims=True)
    return e / l, (m + np.log(l))[..., 0]


def masked_attention(q, k, v, C, S, W, summary_pos=None, skip_old=False,
                     scale=None, dtype=np.float64, rows=None):
    """softmax(q k^T * scale + mask) v for q [Sq,Hq,D], k/v [Sq,Hkv,D].

    summary_pos (bool [Sq]) selects the rows gathered as the K/V prefix
    (whl-sa:interface.py:276-278); None means in-line summaries (P = 0).
    `rows` restricts the computed query rows (array of indices) so that large
    shapes can be spot-checked.  Returns (out [R,Hq,D], lse [Hq,R]) in `dtype`.
    """
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    Sq, Hq, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    if summary_pos is not None:
        sp = np.asarray(summary_pos, dtype=bool)
        k = np.concatenate([k[sp], k], axis=0)
        v = np.concatenate([v[sp], v], axis=0)
    Sk = k.shape[0]
    P = Sk - Sq
    if rows is None:
        rows = np.arange(Sq)
    rows = np.asarray(rows, dtype=np.int64)
    out = np.zeros((len(rows), Hq, D), dtype=dtype)
    lse = np.zeros((Hq, len(rows)), dtype=dtype)
    blk = 256
    kv_all = np.arange(Sk)
    for r0 in range(0, len(rows), blk):
        rr = rows[r0:r0 + blk]
        vis = mask_predicate(rr[:, None], kv_all[None, :], C, S, W, P, skip_old)
        cols = np.nonzero(vis.any(axis=0))[0]
        visc = vis[:, cols]
        for h in range(Hq):
            kh = k[cols, h // g, :]
            vh = v[cols, h // g, :]
            s = (q[rr, h, :] @ kh.T) * scale
            p, l = _softmax_rows(s, visc)
            out[r0:r0 + len(rr), h, :] = p @ vh
            lse[h, r0:r0 + len(rr)] = l
    return out, lse


def decode_attention(q, k, v, start=None, end=None, scale=None, dtype=np.float64):
    """Un-masked attention of q [B,Hq,Q,D] over rows [start_b, end_b) of
    k/v [B,Hkv,L,D]  (HF template :591-612 with repeat_kv :557-566).
    Returns [B,Q,Hq,D]."""
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    Bz, Hq, Q, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    out = np.zeros((Bz, Q, Hq, D), dtype=dtype)
    for b in range(Bz):
        s0 = 0 if start is None else int(np.asarray(start).reshape(-1)[b if np.size(start) > 1 else 0])
        e0 = k.shape[2] if end is None else int(np.asarray(end).reshape(-1)[b if np.size(end) > 1 else 0])
        for h in range(Hq):
            kh = k[b, h // g, s0:e0]
            vh = v[b, h // g, s0:e0]
            s = (q[b, h] @ kh.T) * scale
            m = s.max(axis=-1, keepdims=True)
            e = np.exp(s - m)
            out[b, :, h, :] = (e / e.sum(axis=-1, keepdims=True)) @ vh
    return out


# ----------------------------------------------------------------------------
# Ring-buffer cache state machine (HF template :85-505), one small-window or
# large-window layer, rows tagged by the caller (any array payload).
# ----------------------------------------------------------------------------

class RingBufferModel:
    """Integer model of one cache layer.  `buf` holds one int64 tag per row
    (-1 = never written) so tests can reason about *which* logical rows are
    visible without any floating point."""

    SUMMARY_INIT_CAP = 512
    APPEND_HEADROOM = 1024

    def __init__(self, C, S, scn, large_window=False):
        self.C, self.S, self.scn = C, S, scn
        self.ws = scn * C
        self.large = large_window
        self.buf = None
        self.cap = 0
        self.text_len = 0
        self.ptr = 0
        self.nv = 0
        self.cbl = 0
        self.n_sum = 0

    def reorganize_after_prefill(self, tags, summary_mask):
        """tags: int64 [prefill_len] payload in prefill order (:209-302)."""
        tags = np.asarray(tags, dtype=np.int64)
        sm = np.asarray(summary_mask, dtype=bool)
        text = tags[~sm]
        n_text = len(text)
        C, S, ws = self.C, self.S, self.ws
        if self.large:
            self.cap = n_text + self.APPEND_HEADROOM
            self.buf = np.full(self.cap, -1, np.int64)
            self.buf[:n_text] = text
            self.text_len = n_text
            return
        summ = tags[sm]
        n_sum = len(summ)
        n_complete = n_text // C
        n_partial = n_text % C
        n_win = min(self.scn, n_complete) * C
        self.cap = S + C + ws + n_sum + max(self.SUMMARY_INIT_CAP, n_sum + 256)
        self.buf = np.full(self.cap, -1, np.int64)
        if n_partial:
            self.buf[S + C - n_partial:S + C] = text[n_complete * C:]
        if n_win:
            self.buf[S + C:S + C + n_win] = text[n_complete * C - n_win:n_complete * C]
        self.nv = n_win
        self.ptr = n_win % ws if ws else 0
        self.buf[S + C + ws:S + C + ws + n_sum] = summ
        self.n_sum = n_sum
        self.cbl = n_partial
        self.text_len = 0

    def _grow(self, need):
        while need > self.cap:
            new_cap = max(self.cap + max(self.SUMMARY_INIT_CAP, self.n_sum), self.cap * 2)
            nb = np.full(new_cap, -1, np.int64)
            nb[:self.cap] = self.buf
            self.buf, self.cap = nb, new_cap

    def update_text(self, tag):
        """:306-336"""
        if self.large:
            if self.text_len + 1 > self.cap:
                new_cap = max(self.text_len + 1 + self.APPEND_HEADROOM, self.cap * 2)
                nb = np.full(new_cap, -1, np.int64)
                nb[:self.text_len] = self.buf[:self.text_len]
                self.buf, self.cap = nb, new_cap
            self.buf[self.text_len] = tag
            self.text_len += 1
            return
        dst = self.S + self.C - 1 - self.cbl
        self.buf[dst] = tag
        self.cbl += 1

    def update_summary(self, tags):
        """:340-398"""
        if self.large:
            return
        C, S, ws = self.C, self.S, self.ws
        cbl, ptr = self.cbl, self.ptr
        src = S + C - cbl
        if cbl > 0:
            dst = S + C + ptr
            if ptr + cbl <= ws:
                self.buf[dst:dst + cbl] = self.buf[src:src + cbl].copy()
            else:
                first = ws - ptr
                self.buf[dst:dst + first] = self.buf[src:src + first].copy()
                rest = cbl - first
                self.buf[S + C:S + C + rest] = self.buf[src + first:src + cbl].copy()
        self.ptr = (ptr + cbl) % ws
        if self.nv < ws:
            self.nv = min(ws, self.nv + cbl)
        self.cbl = 0
        n = len(tags)
        if S + C + ws + self.n_sum + n > self.cap:
            self._grow(S + C + ws + self.n_sum + n)
        d = S + C + ws + self.n_sum
        self.buf[d:d + n] = np.asarray(tags, dtype=np.int64)
        self.n_sum += n

    def attention_range(self):
        """(start, end) of get_attention_kv (:402-434)."""
        if self.large:
            return 0, self.text_len
        C, S, ws = self.C, self.S, self.ws
        start = S + C - self.cbl
        if self.nv >= ws:
            skip = min(self.scn * S, self.n_sum)
            end = S + C + ws + (self.n_sum - skip)
        else:
            end = S + C + self.nv
        return start, end

    def summary_attention_range(self, tags):
        """get_summary_attention_kv (:449-474): scratch <- summary tags, rows [0, S+C)."""
        assert not self.large
        self.buf[0:self.S] = np.asarray(tags, dtype=np.int64)
        return 0, self.S + self.C
