"""GPU: the product cache (HIP row mover) + decode kernel reproduce the prefill rule.
For random K/V rows indexed by in-line position, decode output at step t equals the row of
the masked-attention oracle for the text query at that position (decode == prefill row)."""
import types

import numpy as np
import pytest
import torch

from conftest import to_np
from oracle import c_oracle
from oracle import ksa_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("C,S,scn,n_prefill", [(16, 2, 2, 37), (128, 8, 3, 700), (8, 1, 1, 8)])
def test_decode_equals_prefill_row(C, S, scn, n_prefill):
    import ksa_amd
    dev = torch.device("cuda")
    Hq, Hkv, D = 8, 2, 128
    B = C + S
    steps = 2 * C + 3
    # in-line sequence long enough for prefill + decode steps (+ their summaries)
    total_text = n_prefill + steps
    Stot = (total_text // C) * B + total_text % C + B
    g = torch.Generator().manual_seed(0)
    K = torch.randn(Stot, Hkv, D, generator=g).bfloat16()
    V = torch.randn(Stot, Hkv, D, generator=g).bfloat16()
    Q = torch.randn(Stot, Hq, D, generator=g).bfloat16()

    cfg = types.SimpleNamespace(summary_chunk_size=C, summary_token_num=S, num_hidden_layers=2)
    cache = ksa_amd.Qwen3RingBufferCache(cfg, [scn, 10 ** 6])
    n_full = n_prefill // C
    Sq = n_full * B + n_prefill % C
    sp = torch.from_numpy(O.summary_positions(Sq, C, S))[None].to(dev)

    def rows(t, a, b):       # [1, heads, n, D] view as the HF model hands them in
        return t[a:b].permute(1, 0, 2)[None].to(dev)

    for layer in range(2):
        cache.update(rows(K, 0, Sq), rows(V, 0, Sq), layer, {"summary_mask": sp})
    cache.reorganize_after_prefill(sp)

    class M:
        num_key_value_groups = Hq // Hkv

    pos, n_text = Sq, n_prefill
    Kn, Vn, Qn = to_np(K), to_np(V), to_np(Q)
    for _ in range(steps):
        outs = []
        for layer in range(2):
            cache.update_text(rows(K, pos, pos + 1), rows(V, pos, pos + 1), layer)
            kf, vf = cache.get_attention_kv(layer)
            o, _ = ksa_amd.decode_attention_forward(M(), rows(Q, pos, pos + 1), kf, vf, None, scaling=D ** -0.5)
            outs.append(to_np(o)[0, 0])
        n_text += 1
        # small-window layer == Summary-Attention row; large-window layer == causal over text
        want, _ = c_oracle.attention_rows(Qn[:pos + 1], Kn[:pos + 1], Vn[:pos + 1], C, S, scn,
                                          rows=np.array([pos], np.int32))
        assert np.abs(outs[0] - want[0]).max() <= 2e-2, (pos, np.abs(outs[0] - want[0]).max())
        wantl, _ = c_oracle.attention_rows(Qn[:pos + 1], Kn[:pos + 1], Vn[:pos + 1], C, S, 10 ** 6,
                                           rows=np.array([pos], np.int32))
        assert np.abs(outs[1] - wantl[0]).max() <= 2e-2
        pos += 1
        if n_text % C == 0:
            for layer in range(2):
                ks, vs = cache.get_summary_attention_kv(layer, rows(K, pos, pos + S), rows(V, pos, pos + S))
                so, _ = ksa_amd.decode_attention_forward(M(), rows(Q, pos, pos + S), ks, vs, None,
                                                         scaling=D ** -0.5)
                # boundary summary queries attend [own summaries | chunk text] without a mask
                # (HF template :858-870): compare with un-masked attention over those rows
                sel = np.r_[pos:pos + S, pos - C:pos]
                wq = c_oracle.decode(Qn[pos:pos + S].transpose(1, 0, 2)[None],
                                     Kn[sel].transpose(1, 0, 2)[None], Vn[sel].transpose(1, 0, 2)[None],
                                     0, len(sel))
                assert np.abs(to_np(so) - wq).max() <= 2e-2
                cache.update_summary(rows(K, pos, pos + S), rows(V, pos, pos + S), layer)
            pos += S
            cache.reset_chunk_counter()


def test_cache_handoff_at_1024_chunks():
    """The hand-off prefill -> `reorganize_after_prefill` -> decode at the decode benchmark's own size:
    1024 complete chunks (C = 128, S = 8, a ring of 4 chunks, 32 / 8 heads, batch 2 with different rows
    per sequence), a small-window layer next to a large-window one (whose reorganisation gathers the
    131072 text rows out of 139264).  Then C + 3 decode steps across one chunk boundary through
    `update_text`, `get_summary_attention_kv` and `update_summary`.  Every step's output (decode kernel
    over `attention_range` of the whole buffer) is compared with
      (a) the masked-attention oracle's row for that position on the full in-line sequence, and
      (b) the prefill kernel's own row for that position (one prefill launch over the final sequence),
    which is the decode == prefill-row invariant at this size.  The buffer capacity and the attended
    range are the reference's closed forms (modeling_qwen3sa.py:265-266, :421-431): capacity
    S + C + 4 C + 8192 + max(512, 8192 + 256) = 17288, range (136 - rows of the chunk, 8808) until the
    boundary, (…, 8816) after it."""
    import ksa_amd
    dev = torch.device("cuda")
    C, S, scn, Hq, Hkv, D, bsz = 128, 8, 4, 32, 8, 128, 2
    B = C + S
    n_chunks = 1024
    n_prefill = n_chunks * C
    steps = C + 3
    Sq = n_chunks * B
    Stot = Sq + B + 3                      # prefill + one more chunk with its summaries + 3 text rows
    g = torch.Generator().manual_seed(2)
    K = torch.randn(bsz, Stot, Hkv, D, generator=g).bfloat16()
    V = torch.randn(bsz, Stot, Hkv, D, generator=g).bfloat16()
    Q = torch.randn(bsz, Stot, Hq, D, generator=g).bfloat16()
    Kd, Vd, Qd = K.to(dev), V.to(dev), Q.to(dev)

    cfg = types.SimpleNamespace(summary_chunk_size=C, summary_token_num=S, num_hidden_layers=2)
    cache = ksa_amd.Qwen3RingBufferCache(cfg, [scn, 10 ** 6])
    sp = torch.from_numpy(O.summary_positions(Sq, C, S))[None].to(dev)

    def rows(t, a, b):       # [bsz, heads, n, D] view as the HF model hands them in
        return t[:, a:b].permute(0, 2, 1, 3)

    for layer in range(2):
        cache.update(rows(Kd, 0, Sq), rows(Vd, 0, Sq), layer, {"summary_mask": sp})
    cache.reorganize_after_prefill(sp)
    assert cache._capacity[0] == 17288 and cache.key_cache[0].shape == (bsz, Hkv, 17288, D)
    assert cache._text_len[1] == n_prefill and cache.attention_range(1) == (0, n_prefill)
    assert cache.attention_range(0) == (136, 8808)
    # the gather itself, bit for bit: ring rows = text of the last four chunks, summaries in order
    ring = cache.key_cache[0][:, :, S + C:S + C + scn * C]
    want_ring = torch.cat([rows(Kd, c * B, c * B + C) for c in range(n_chunks - scn, n_chunks)], dim=2)
    assert torch.equal(ring, want_ring)
    sums = cache.value_cache[0][:, :, S + C + scn * C:S + C + scn * C + n_chunks * S]
    assert torch.equal(sums, rows(Vd, 0, Sq)[:, :, sp[0]])
    assert torch.equal(cache.key_cache[1][:, :, :n_prefill], rows(Kd, 0, Sq)[:, :, ~sp[0]])

    class M:
        num_key_value_groups = Hq // Hkv

    pos, n_text = Sq, n_prefill
    got = [[], []]
    positions = []
    for step in range(steps):
        for layer in range(2):
            cache.update_text(rows(Kd, pos, pos + 1), rows(Vd, pos, pos + 1), layer)
            a, e = cache.attention_range(layer)
            if layer == 0:
                cbl = cache._chunk_buf_len[0]
                assert (a, e) == (136 - cbl, 8808 if step < C else 8816), (step, a, e)
            o = ksa_amd.ksa_decode(rows(Qd, pos, pos + 1), cache.key_cache[layer], cache.value_cache[layer], a, e)
            if step in (0, C - 1, C):   # the reference's own call form: a slice of the cache
                kf, vf = cache.get_attention_kv(layer)
                o2, _ = ksa_amd.decode_attention_forward(M(), rows(Qd, pos, pos + 1), kf, vf, None, scaling=D ** -0.5)
                assert (o2.float() - o.float()).abs().max().item() <= 1e-2
            got[layer].append(o[:, 0])
        positions.append(pos)
        n_text += 1
        pos += 1
        if n_text % C == 0:
            for layer in range(2):
                ks, vs = cache.get_summary_attention_kv(layer, rows(Kd, pos, pos + S), rows(Vd, pos, pos + S))
                so, _ = ksa_amd.decode_attention_forward(M(), rows(Qd, pos, pos + S), ks, vs, None, scaling=D ** -0.5)
                sel = np.r_[pos:pos + S, pos - C:pos]
                wq = c_oracle.decode(to_np(Q[:, pos:pos + S]).transpose(0, 2, 1, 3),
                                     to_np(K[:, sel]).transpose(0, 2, 1, 3), to_np(V[:, sel]).transpose(0, 2, 1, 3),
                                     0, len(sel))
                assert np.abs(to_np(so) - wq).max() <= 2e-2
                cache.update_summary(rows(Kd, pos, pos + S), rows(Vd, pos, pos + S), layer)
            pos += S
            cache.reset_chunk_counter()
    assert cache._n_summaries[0] == (n_chunks + 1) * S and cache._window_write_ptr[0] == C % (scn * C)
    n_used = pos
    prow = np.array(positions, np.int32)
    spf = torch.from_numpy(O.summary_positions(n_used, C, S)).to(dev)
    for layer, window in ((0, scn), (1, 10 ** 6)):
        dec = torch.stack(got[layer], dim=1)                     # [bsz, steps, Hq, D]
        for b in range(bsz):
            want, _ = c_oracle.attention_rows(to_np(Q[b, :n_used]), to_np(K[b, :n_used]), to_np(V[b, :n_used]),
                                              C, S, window, rows=prow)
            err = np.abs(to_np(dec[b]) - want).max()
            assert err <= 2e-2, (layer, b, err)
            pre, _ = ksa_amd.summary_attn_func(Qd[b:b + 1, :n_used], Kd[b:b + 1, :n_used], Vd[b:b + 1, :n_used],
                                               C, S, window, summary_pos=spf)
            perr = (pre[0, torch.as_tensor(prow, device=dev).long()].float() - dec[b].float()).abs().max().item()
            print(f"layer {layer} seq {b}: decode vs oracle {err:.2e}, decode vs prefill kernel row {perr:.2e}")
            assert perr <= 2e-2, (layer, b, perr)


def test_move_rows_multi_equals_single_moves():
    """Independent moves in one launch (`ksa_copy_rows_multi`) against the same moves one launch each, in
    the two groups a chunk-boundary step makes (first the text row and the summary rows into the
    scratch rows, then the flush of the chunk into the ring and the append of the summaries, for K
    and for V): strided sources (a transposed projection output), a move inside one buffer, scalar
    and per-sequence destinations, a zero-row move dropped."""
    from ksa_amd.cache import _move_rows, _move_rows_multi
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(3)
    b, H, D, S, C = 3, 2, 128, 8, 128
    new = torch.randn(b, 1 + S, H, D, generator=g).bfloat16().to(dev).transpose(1, 2)     # [b, H, 1 + S, D], strided
    bufs = [torch.randn(b, H, 700, D, generator=g).bfloat16().to(dev) for _ in range(2)]
    ref = [x.clone() for x in bufs]
    seq = torch.tensor([200, 328, 456], dtype=torch.int32, device=dev)
    app = torch.tensor([650, 658, 666], dtype=torch.int32, device=dev)
    for group in (lambda x: [(new[:, :, :1], x, 1, 0, 135), (new[:, :, 1:], x, S, 0, 0), (new, x, 0, 0, 5)],
                  lambda x: [(x, x, C, S, seq), (new[:, :, 1:], x, S, 0, app)]):
        _move_rows_multi([m for x in bufs for m in group(x)])
        for x, r in zip(bufs, ref):
            for src, dst, n, s0, d0 in group(r):
                if torch.is_tensor(d0):
                    _move_rows(src, dst, n, s0, 0, dst_start_seq=d0)
                else:
                    _move_rows(src, dst, n, s0, d0)
        torch.cuda.synchronize()
        for x, r in zip(bufs, ref):
            assert torch.equal(x, r)
