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
