"""Pins the CPU oracle.  The reference ships no tests, fixtures or golden vectors, so each
oracle function is fixed by checks that a plausible mistake would fail:

  predicate (4 modes)      two independent statements in the reference must agree by brute
                           force (predicate form vs chunk-by-chunk interval form, prefix column
                           j <-> in-line row (j//S)*B + C + j%S), closed-form row counts,
                           special cases (W >= chunks = causal over text, W = 0, row sees itself)
  block index              known totals for cfg 0 / cfg 1 derived independently (by hand from
                           the rule), format invariants, C vs numpy
  masked attention         torch SDPA with an explicit bool mask (library routine), un-masked
                           and plain-causal special cases, numpy vs C implementations
  decode attention         torch SDPA; partition identity of the split merge
  ring-buffer model        decode == prefill row: the multiset of rows in the attended slice
                           equals the key set the prefill mask allows at that position
"""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle
from oracle import cpu_path
from oracle import ksa_oracle as O

SMALL = [
    # (n_full chunks, tail text rows, C, S)
    (5, 0, 4, 2), (7, 3, 8, 1), (12, 0, 2, 1), (6, 1, 1, 1), (4, 5, 16, 8), (3, 0, 128, 8), (9, 2, 3, 2),
]
WINDOWS = [0, 1, 3, 4, 100]


@pytest.mark.parametrize("shape", SMALL)
@pytest.mark.parametrize("W", WINDOWS)
@pytest.mark.parametrize("skip_old", [False, True])
def test_predicate_forms_agree(shape, W, skip_old):
    n_full, tail, C, S = shape
    B = C + S
    Sq = n_full * B + tail
    interval = O.dense_mask_intervals(Sq, C, S, W, skip_old)          # muse builder form
    inline = O.dense_mask_predicate(Sq, C, S, W, 0, skip_old)          # mask.py in-line form
    assert np.array_equal(interval, inline)
    # prefix form: columns [0,P) are the summary rows, columns [P, P+Sq) the in-line rows
    P = n_full * S
    if P == 0:
        return
    pref = O.dense_mask_predicate(Sq, C, S, W, P, skip_old)
    rows = O.prefix_to_inline_row(np.arange(P), C, S)
    sp = O.summary_positions(Sq, C, S)
    assert np.array_equal(np.nonzero(sp)[0], rows)
    # in-line part of the prefix form: text queries never see in-line summary rows, summary
    # queries see their own chunk exactly as in the in-line form
    is_q_sum = sp[:, None]
    is_kv_sum = sp[None, :]
    expect_inline_part = np.where(is_q_sum, interval, interval & ~is_kv_sum)
    assert np.array_equal(pref[:, P:], expect_inline_part)
    # prefix part: text queries see exactly the old summaries the interval form grants them
    expect_prefix = interval[:, rows] & ~is_q_sum
    assert np.array_equal(pref[:, :P], expect_prefix)


@pytest.mark.parametrize("shape", SMALL)
@pytest.mark.parametrize("W", WINDOWS)
def test_predicate_closed_form_counts(shape, W):
    n_full, tail, C, S = shape
    B = C + S
    Sq = n_full * B + tail
    P = n_full * S
    vis = O.dense_mask_predicate(Sq, C, S, W, P) if P else O.dense_mask_predicate(Sq, C, S, W, 0)
    cnt = vis.sum(axis=1)
    for i in range(Sq):
        c, o = divmod(i, B)
        want = O.visible_count_text(c, o, C, S, W) if o < C else O.visible_count_summary(o - C, C)
        assert cnt[i] == want, (i, cnt[i], want)
        # every row sees itself
        assert vis[i, P + i]


def test_predicate_special_cases():
    C, S, n = 4, 2, 6
    B = C + S
    Sq = n * B
    sp = O.summary_positions(Sq, C, S)
    text = np.nonzero(~sp)[0]
    # W >= chunks: the text part is plain causal attention over text-only positions
    m = O.dense_mask_predicate(Sq, C, S, 50, 0)
    sub = m[np.ix_(text, text)]
    assert np.array_equal(sub, np.tril(np.ones_like(sub)))
    assert not m[np.ix_(text, np.nonzero(sp)[0])].any()
    # W = 0: own chunk + all older summaries
    m0 = O.dense_mask_predicate(Sq, C, S, 0, 0)
    for i in text:
        c = i // B
        want = set(range(c * B, i + 1)) | {j for j in np.nonzero(sp)[0] if j // B < c}
        assert set(np.nonzero(m0[i])[0]) == want
    # skip_old never grants more than the default rule and differs only on summary columns
    ms = O.dense_mask_predicate(Sq, C, S, 1, 0, True)
    m1 = O.dense_mask_predicate(Sq, C, S, 1, 0, False)
    assert not (ms & ~m1).any() and not (m1 & ~ms)[:, ~sp].any()


def test_c_predicate_equals_numpy():
    rng = np.random.default_rng(0)
    L = c_oracle.lib()
    for _ in range(200):
        C, S = int(rng.integers(1, 20)), int(rng.integers(1, 5))
        W = int(rng.integers(0, 6))
        n = int(rng.integers(1, 8))
        Sq = n * (C + S) + int(rng.integers(0, C + 1))
        for P in (0, (Sq // (C + S)) * S):
            skip = bool(rng.integers(0, 2))
            want = O.dense_mask_predicate(Sq, C, S, W, P, skip)
            got = np.array([[L.ksa_oracle_visible(q, kv, C, S, W, P, int(skip)) for kv in range(Sq + P)]
                            for q in range(Sq)], dtype=bool)
            assert np.array_equal(got, want)


@pytest.mark.parametrize("W,want", [(3, (356, 24, 2188416, 13)), (4, (412, 25, 2618496, 15))])
def test_block_index_cfg0_known_answer(W, want):
    mc, mi, fc, fi, pairs = c_oracle.block_index(4352, 4608, 128, 8, W, 256)
    assert (int(mc.sum()), int(fc.sum()), pairs, int((mc + fc).max())) == want
    py = O.block_index(4352, 4608, 128, 8, W, 256)
    for a, b in zip(py, (mc, mi, fc, fi)):
        assert np.array_equal(a, b)
    # format invariants: ascending lists, zero tails, counts bounded
    N = mi.shape[1]
    for m in range(len(mc)):
        assert np.all(np.diff(mi[m, :mc[m]]) > 0) and not mi[m, mc[m]:].any()
        assert np.all(np.diff(fi[m, :fc[m]]) > 0) and not fi[m, fc[m]:].any()
        assert mc[m] + fc[m] <= N
        assert not set(mi[m, :mc[m]]) & set(fi[m, :fc[m]])
    # allowed-pair total is tile independent: compare with the closed-form row counts
    B = 136
    tot = sum(O.visible_count_text(i // B, i % B, 128, 8, W) if i % B < 128
              else O.visible_count_summary(i % B - 128, 128) for i in range(4352))
    assert pairs == tot


@pytest.mark.slow
@pytest.mark.parametrize("W,want", [(3, (6558, 430, 47512576)), (4, (7076, 445, 51383296))])
def test_block_index_cfg1_known_answer(W, want):
    mc, mi, fc, fi, pairs = c_oracle.block_index(34816, 36864, 128, 8, W, 2048)
    assert (int(mc.sum()), int(fc.sum()), pairs) == want


@pytest.mark.parametrize("case", [(999, 16, 2, 3, 110, 128, 64), (513, 8, 1, 2, 57, 64, 32),
                                  (300, 2, 1, 4, 0, 32, 32), (700, 32, 4, 1, 0, 128, 64)])
def test_block_index_c_vs_numpy_odd_shapes(case):
    Sq, C, S, W, P, tm, tn = case
    for skip in (False, True):
        a = O.block_index(Sq, Sq + P, C, S, W, P, skip, tm, tn)
        b = c_oracle.block_index(Sq, Sq + P, C, S, W, P, skip, tm, tn)[:4]
        for x, y in zip(a, b):
            assert np.array_equal(x, y)
        # a tile is listed iff it holds a visible element; full iff all in-bounds are visible
        vis = O.dense_mask_predicate(Sq, C, S, W, P, skip)
        for m in range(len(a[0])):
            for n in range(a[1].shape[1]):
                blk = vis[m * tm:(m + 1) * tm, n * tn:(n + 1) * tn]
                cls = 0 if not blk.any() else (2 if blk.all() else 1)
                listed = 1 if n in a[1][m, :a[0][m]] else (2 if n in a[3][m, :a[2][m]] else 0)
                assert cls == listed


def _rand(shape, seed):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("mode", ["prefix", "inline"])
def test_masked_attention_vs_torch_sdpa(mode):
    Sq, Hq, Hkv, D, C, S, W = 5 * 20 + 7, 4, 2, 32, 16, 4, 2
    q, k, v = _rand((Sq, Hq, D), 0), _rand((Sq, Hkv, D), 1), _rand((Sq, Hkv, D), 2)
    sp = O.summary_positions(Sq, C, S) if mode == "prefix" else None
    out_np, lse_np = O.masked_attention(q.numpy(), k.numpy(), v.numpy(), C, S, W, summary_pos=sp)
    out_c, lse_c = c_oracle.attention_rows(q.numpy(), k.numpy(), v.numpy(), C, S, W, summary_pos=sp)
    # library routine with the interval-form mask on the in-line sequence (both modes must
    # give the same function of the inputs: prefix rows are copies of the in-line summary rows)
    mask = torch.from_numpy(O.dense_mask_intervals(Sq, C, S, W))
    g = Hq // Hkv
    ref = F.scaled_dot_product_attention(
        q.permute(1, 0, 2)[None].double(), k.repeat_interleave(g, 1).permute(1, 0, 2)[None].double(),
        v.repeat_interleave(g, 1).permute(1, 0, 2)[None].double(), attn_mask=mask)[0].permute(1, 0, 2).numpy()
    assert np.abs(out_np - ref).max() < 1e-10
    assert np.abs(out_c - ref).max() < 1e-5
    # lse against a direct log-sum-exp
    s = torch.einsum("qhd,khd->hqk", q.double(), k.repeat_interleave(g, 1).double()) / D ** 0.5
    s = s.masked_fill(~mask[None], float("-inf"))
    want_lse = torch.logsumexp(s, dim=-1).numpy()
    assert np.abs(lse_np - want_lse).max() < 1e-10 and np.abs(lse_c - want_lse).max() < 1e-4
    # restated reference CPU paths agree as well
    assert np.abs(cpu_path.mask_mode(q, k, v, C, S, W).numpy() - ref).max() < 1e-4
    assert np.abs(cpu_path.block_mode_rows(q[20:90], k, v, 20, C, S, W).numpy() - ref[20:90]).max() < 1e-4


def test_masked_attention_special_cases():
    # one chunk, no window needed: text rows are plain causal attention
    C, S = 24, 1
    Sq, H, D = C, 2, 16
    q, k, v = _rand((Sq, H, D), 3), _rand((Sq, H, D), 4), _rand((Sq, H, D), 5)
    out, _ = O.masked_attention(q.numpy(), k.numpy(), v.numpy(), C, S, 3)
    ref = F.scaled_dot_product_attention(q.permute(1, 0, 2)[None].double(), k.permute(1, 0, 2)[None].double(),
                                         v.permute(1, 0, 2)[None].double(), is_causal=True)[0].permute(1, 0, 2)
    assert np.abs(out - ref.numpy()).max() < 1e-10
    # GQA head map is kv_head = q_head // g (repeat_interleave order), not q_head % Hkv
    q4 = _rand((Sq, 4, D), 6)
    out4, _ = O.masked_attention(q4.numpy(), k.numpy(), v.numpy(), C, S, 3)
    for h in range(4):
        single, _ = O.masked_attention(q4[:, h:h + 1].numpy(), k[:, h // 2:h // 2 + 1].numpy(),
                                       v[:, h // 2:h // 2 + 1].numpy(), C, S, 3)
        assert np.abs(out4[:, h] - single[:, 0]).max() < 1e-12


def test_decode_oracle_vs_torch_and_partition_identity():
    Bz, Hq, Hkv, Q, D, L = 3, 8, 2, 2, 32, 97
    q, k, v = _rand((Bz, Hq, Q, D), 7), _rand((Bz, Hkv, L, D), 8), _rand((Bz, Hkv, L, D), 9)
    start = np.array([0, 5, 40], np.int32)
    end = np.array([97, 6, 90], np.int32)
    got_np = O.decode_attention(q.numpy(), k.numpy(), v.numpy(), start, end)
    got_c = c_oracle.decode(q.numpy(), k.numpy(), v.numpy(), start, end)
    for b in range(Bz):
        ref = cpu_path.decode_sdpa(q[b:b + 1].double(), k[b:b + 1, :, start[b]:end[b]].double(),
                                   v[b:b + 1, :, start[b]:end[b]].double(), Hq // Hkv)[0].numpy()
        assert np.abs(got_np[b] - ref).max() < 1e-10
        assert np.abs(got_c[b] - ref).max() < 1e-5
    # merging un-normalised partials over any partition of the rows equals a single pass
    s = (q[0, 0, 0].double() @ k[0, 0].double().T).numpy() / D ** 0.5
    vv = v[0, 0].double().numpy()
    full = (np.exp(s - s.max()) / np.exp(s - s.max()).sum()) @ vv
    parts = [(0, 13), (13, 50), (50, 97)]
    ms = [s[a:b].max() for a, b in parts]
    ls = [np.exp(s[a:b] - m).sum() for (a, b), m in zip(parts, ms)]
    os_ = [np.exp(s[a:b] - m) @ vv[a:b] for (a, b), m in zip(parts, ms)]
    M = max(ms)
    merged = sum(o * np.exp(m - M) for o, m in zip(os_, ms)) / sum(l * np.exp(m - M) for l, m in zip(ls, ms))
    assert np.abs(merged - full).max() < 1e-12


@pytest.mark.parametrize("C,S,scn", [(4, 2, 2), (8, 1, 3), (3, 2, 1)])
@pytest.mark.parametrize("n_prefill", [0, 1, 5, 12, 13, 29, 40])
def test_ring_buffer_decode_equals_prefill_row(C, S, scn, n_prefill):
    """After prefill of n text tokens and t decode steps (with chunk-boundary flushes), the
    rows in the attended slice are exactly the keys the prefill mask grants the text query at
    that logical position (tags = in-line row numbers of the expanded sequence)."""
    B = C + S
    if n_prefill == 0:
        pytest.skip("the reference always prefills at least one token")
    n_full = n_prefill // C
    Sq = n_full * B + n_prefill % C
    sp = O.summary_positions(Sq, C, S)
    ring = O.RingBufferModel(C, S, scn)
    ring.reorganize_after_prefill(np.arange(Sq), sp)
    n_text = n_prefill
    pos = Sq                      # next in-line row number
    if n_text % C == 0 and n_text > 0:
        pass                      # prefill ended on a chunk boundary: summaries already in place
    for step in range(3 * C + 2):
        ring.update_text(pos)
        n_text += 1
        a, b = ring.attention_range()
        got = sorted(ring.buf[a:b].tolist())
        # expected: visible keys of in-line row `pos` in a sequence long enough to hold it
        total = pos + 1
        vis = O.mask_predicate(pos, np.arange(total), C, S, scn, 0)
        want = np.nonzero(vis)[0].tolist()
        assert got == want, (step, got, want)
        pos += 1
        if n_text % C == 0:       # chunk complete: S summary rows follow
            tags = np.arange(pos, pos + S)
            r0, r1 = ring.summary_attention_range(tags)
            # summary queries attend [own summaries | chunk text]
            assert sorted(ring.buf[r0:r1].tolist()) == list(range(pos - C, pos + S))
            ring.update_summary(tags)
            pos += S


def test_ring_buffer_known_answers():
    """Hand-checked values from the formulas of the HF template (:265-266, :285, :330, :421-431)."""
    C, S, scn = 128, 8, 4
    ring = O.RingBufferModel(C, S, scn)
    n_chunks = 1024
    Sq = n_chunks * (C + S)
    ring.reorganize_after_prefill(np.arange(Sq), O.summary_positions(Sq, C, S))
    assert ring.cap == 8 + 128 + 512 + 8192 + 8448 == 17288
    assert (ring.nv, ring.ptr, ring.cbl, ring.n_sum) == (512, 0, 0, 8192)
    ring.update_text(Sq)
    assert ring.buf[8 + 128 - 1] == Sq and ring.cbl == 1
    assert ring.attention_range() == (135, 8808)
    for i in range(1, 57):
        ring.update_text(Sq + i)
    assert ring.attention_range() == (136 - 57, 8 + 128 + 512 + 8160)
    # ring not yet full: no summaries visible
    r2 = O.RingBufferModel(C, S, scn)
    r2.reorganize_after_prefill(np.arange(2 * 136 + 5), O.summary_positions(2 * 136 + 5, C, S))
    assert (r2.nv, r2.ptr, r2.cbl) == (256, 256, 5)
    assert r2.attention_range() == (136 - 5, 136 + 256)


def test_known_answers_fixture():
    """tests/golden/known_answers.json against the oracle: allowed-pair totals of all three
    configurations by the closed-form row counts (no tiles involved), tile totals of cfg 0 by the
    C index builder."""
    import json
    import os
    ka = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")))
    C, S = ka["C"], ka["S"]
    B = C + S
    for name, cfg in ka["configs"].items():
        Sq = cfg["Sq"]
        rows = np.arange(Sq)
        c, o = rows // B, rows % B
        for W in (3, 4):
            text = S * np.maximum(0, c - W) + C * np.minimum(c, W) + o + 1
            summ = C + (o - C) + 1
            pairs = int(np.where(o < C, text, summ).sum())
            assert pairs == cfg[f"W{W}"]["pairs"], (name, W)
            assert cfg["P"] == (Sq // B) * S
    for W in (3, 4):
        mc, mi, fc, fi, pairs = c_oracle.block_index(4352, 4608, C, S, W, 256)
        want = ka["configs"]["cfg0"][f"W{W}"]
        assert (int(mc.sum()), int(fc.sum()), pairs, int((mc + fc).max())) == \
            (want["partial"], want["full"], want["pairs"], want["max_tiles_per_row_tile"])
