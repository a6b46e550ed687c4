"""CPU-side checks of the product's host logic: the C ABI loads and exports everything
include/ksa_hip.h declares, rejects bad arguments before any launch, the closed-form
visibility rule used by the kernels equals the oracle predicate, and the cache class keeps
the reference's bookkeeping (checked against the oracle's integer model with a host row
mover injected by the test — the product itself has none)."""
import ctypes
import os
import re
import types

import numpy as np
import pytest
import torch

from oracle import ksa_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from ksa_amd import _lib
    L = _lib.lib()
    header = open(os.path.join(ROOT, "include", "ksa_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ksa_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    for name in declared:
        assert getattr(L, name) is not None
    assert L.ksa_version() >= 100
    assert b"ok" == L.ksa_error_string(0)


def test_error_codes_before_launch():
    from ksa_amd import _lib
    L = _lib.lib()
    # bad sizes / null pointers are rejected without touching a device
    assert L.ksa_block_index(0, 10, 128, 8, 3, 10, 0, 128, 64, None, None, None, None, None) == -1
    assert L.ksa_block_index(100, 110, 128, 8, 3, 9, 0, 128, 64, None, None, None, None, None) == -1
    assert L.ksa_block_index(100, 110, 128, 8, 3, 10, 0, 128, 64, None, None, None, None, None) == -2
    null3 = ctypes.cast(None, ctypes.POINTER(ctypes.c_int64))
    assert L.ksa_prefill_fwd(None, None, None, None, None, 1, 128, 4, 2, 128, 0, null3, null3, null3,
                             128, 8, 3, 0, 0, 0, None, None, None, None, 2, 1.0, 0, None, None) == -2
    assert L.ksa_decode_fwd(None, None, None, None, None, None, 0, 10, 1, 4, 2, 1, 128, 0, null3, null3,
                            null3, null3, 1.0, 1, None, 0, None) == -2
    assert L.ksa_decode_workspace_bytes(64, 32, 8, 1, 128, 1) == 0
    assert L.ksa_decode_workspace_bytes(64, 32, 8, 1, 128, 2) == 64 * 8 * 2 * 32 * 130 * 4
    assert L.ksa_decode_auto_splits(64, 8, 17288) == 1
    assert L.ksa_decode_auto_splits(8, 8, 17288) == 8
    assert L.ksa_decode_auto_splits(1, 8, 100) == 1
    assert 1 <= L.ksa_decode_auto_splits(1, 8, 100000) <= 64


@pytest.mark.parametrize("P_mode", ["prefix", "inline"])
def test_closed_form_counts_equal_predicate(P_mode):
    """ksa_count_visible (csrc/ksa_mask.h, the rule both the index kernel and the prefill
    mask are built on) against brute force over the oracle predicate."""
    from ksa_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(1)
    for _ in range(60):
        C, S = int(rng.integers(1, 24)), int(rng.integers(1, 6))
        W = int(rng.integers(0, 6))
        n = int(rng.integers(1, 9))
        Sq = n * (C + S) + int(rng.integers(0, C + 1))
        P = (Sq // (C + S)) * S if P_mode == "prefix" else 0
        Sk = Sq + P
        skip = int(rng.integers(0, 2))
        vis = O.dense_mask_predicate(Sq, C, S, W, P, bool(skip))
        cum = np.concatenate([np.zeros((Sq, 1), np.int64), np.cumsum(vis, axis=1)], axis=1)
        for _ in range(40):
            q = int(rng.integers(0, Sq))
            a = int(rng.integers(0, Sk))
            b = int(rng.integers(a, Sk + 1))
            got = L.ksa_debug_count_visible(q, a, b, C, S, W, P, skip, Sq, Sk)
            assert got == cum[q, b] - cum[q, a], (C, S, W, P, skip, q, a, b)


def _host_mover(src, dst, nrows, src_start=0, dst_start=0, src_index=None):
    if nrows <= 0:
        return
    rows = src_index.long() if src_index is not None else torch.arange(src_start, src_start + nrows)
    dst[:, :, dst_start:dst_start + nrows, :] = src[:, :, rows[:nrows], :].clone()


def _make_cache(C, S, scns):
    from ksa_amd.cache import Qwen3RingBufferCache
    cfg = types.SimpleNamespace(summary_chunk_size=C, summary_token_num=S, num_hidden_layers=len(scns))

    class HostCache(Qwen3RingBufferCache):
        _move_rows = staticmethod(_host_mover)
    return HostCache(cfg, scns)


@pytest.mark.parametrize("C,S", [(4, 2), (8, 1)])
@pytest.mark.parametrize("n_prefill", [1, 7, 16, 37])
def test_cache_bookkeeping_matches_model(C, S, n_prefill):
    """Drives the product cache class and the oracle's integer model with the same tagged
    rows through prefill, reorganisation, decode steps and chunk boundaries."""
    scns = [2, 3, 1000]                # last layer is a large-window layer
    cache = _make_cache(C, S, scns)
    assert cache.is_large_window == [False, True, True]
    B = C + S
    n_full = n_prefill // C
    Sq = n_full * B + n_prefill % C
    sp = O.summary_positions(Sq, C, S)
    D, H = 8, 2
    tags = torch.arange(Sq, dtype=torch.float32)
    kv = tags[None, None, :, None].expand(1, H, Sq, D).to(torch.bfloat16).contiguous()
    models = [O.RingBufferModel(C, S, scn, large) for scn, large in zip(scns, cache.is_large_window)]
    spt = torch.from_numpy(sp)[None]
    for layer in range(3):
        k_all, v_all = cache.update(kv, kv, layer, {"summary_mask": spt})
        assert k_all.shape[2] == Sq
    # as in the reference, a small-window layer reports 0 until the cache is reorganised
    assert cache.get_true_token_num() == n_prefill and cache.get_seq_length(0) == 0 and cache.get_seq_length(1) == Sq
    cache.reorganize_after_prefill(spt)
    for m in models:
        m.reorganize_after_prefill(np.arange(Sq), sp)
    pos = Sq
    n_text = n_prefill

    def check():
        for layer, m in enumerate(models):
            a, b = m.attention_range()
            assert cache.attention_range(layer) == (a, b)
            k, v = cache.get_attention_kv(layer)
            assert k.shape[2] == b - a
            assert sorted(k[0, 0, :, 0].float().tolist()) == sorted(m.buf[a:b].tolist())
            assert cache._capacity[layer] == m.cap == cache.key_cache[layer].shape[2]
        assert cache.get_true_token_num() == n_text

    check()
    for _ in range(3 * C + 1):
        row = torch.full((1, H, 1, D), float(pos), dtype=torch.bfloat16)
        for layer, m in enumerate(models):
            cache.update_text(row, row, layer)
            m.update_text(pos)
        n_text += 1
        pos += 1
        check()
        if n_text % C == 0:
            stags = np.arange(pos, pos + S)
            srow = torch.from_numpy(stags.astype(np.float32))[None, None, :, None].expand(1, H, S, D).to(torch.bfloat16)
            for layer, m in enumerate(models):
                ks, vs = cache.get_summary_attention_kv(layer, srow, srow)
                assert sorted(ks[0, 0, :, 0].float().tolist()) == list(range(pos - C, pos + S))
                cache.update_summary(srow, srow, layer)
                m.update_summary(stags)
            pos += S
            assert cache.get_cur_chunk_size() == B
            cache.reset_chunk_counter()
            assert cache.get_cur_chunk_size() == 0
            check()


@pytest.mark.parametrize("C,S,n_prefill", [(4, 2, 7), (8, 1, 16), (4, 2, 1), (2, 1, 3)])
def test_cache_boundary_slots_equal_update_calls(C, S, n_prefill):
    """`boundary_slots` + the caller's own row moves (what the recorded boundary step does)
    against `update_text` + `get_summary_attention_kv` + `update_summary` on a second cache
    driven with the same rows: same counters, same ranges, same buffer contents wherever
    rows are attended, over many boundaries (ring wrap-around, growth of the summary region)."""
    scns = [2, 3, 1000]
    a_cache, b_cache = _make_cache(C, S, scns), _make_cache(C, S, scns)
    for c in (a_cache, b_cache):
        c._SUMMARY_INIT_CAP = 4
        c._APPEND_HEADROOM = 5
    B = C + S
    Sq = (n_prefill // C) * B + n_prefill % C
    sp = torch.from_numpy(O.summary_positions(Sq, C, S))[None]
    D, H = 8, 2
    kv = torch.arange(Sq, dtype=torch.float32)[None, None, :, None].expand(1, H, Sq, D).to(torch.bfloat16).contiguous()
    for c in (a_cache, b_cache):
        for layer in range(3):
            c.update(kv, kv, layer, {"summary_mask": sp})
        c.reorganize_after_prefill(sp)
    pos, n_text, n_boundaries = Sq, n_prefill, 0
    counters = ("_text_len", "_capacity", "_window_write_ptr", "_n_valid_window", "_chunk_buf_len",
                "_n_summaries", "cur_chunk_sizes", "true_tokens", "_total_chunks")
    for _ in range(40 * C):
        row = torch.full((1, H, 1, D), float(pos % 251), dtype=torch.bfloat16)
        boundary = n_text % C == C - 1
        if not boundary:
            for layer in range(3):
                a_cache.update_text(row, row, layer)
                b_cache.update_text(row, row, layer)
            pos += 1
        else:
            srow = (torch.arange(pos + 1, pos + 1 + S) % 251).float()[None, None, :, None].expand(1, H, S, D).to(torch.bfloat16)
            for layer in range(3):
                a_cache.update_text(row, row, layer)
                want_range = a_cache.attention_range(layer)
                ks, _ = a_cache.get_summary_attention_kv(layer, srow, srow)
                want_sum = ks[0, 0, :, 0].float().tolist()
                a_cache.update_summary(srow, srow, layer)
                # the same step from the rows `boundary_slots` names
                assert b_cache.boundary_fits_one_piece(layer)
                sl = b_cache.boundary_slots(layer, S)
                for buf in (b_cache.key_cache[layer], b_cache.value_cache[layer]):
                    _host_mover(row, buf, 1, 0, sl["text"])
                    assert sl["attend"] == want_range
                    if b_cache.is_large_window[layer]:
                        _host_mover(srow, buf, S, 0, sl["spare"])
                        got_sum = buf[0, 0, sl["spare"] - C:sl["spare"] + S, 0].float().tolist()
                    else:
                        _host_mover(srow, buf, S, 0, 0)
                        got_sum = buf[0, 0, :S + C, 0].float().tolist()
                        _host_mover(buf, buf, sl["flush_rows"], sl["flush_src"], sl["flush_dst"])
                        _host_mover(srow, buf, S, 0, sl["append"])
                    assert sorted(got_sum) == sorted(want_sum)
            pos += 1 + S
            n_boundaries += 1
            a_cache.reset_chunk_counter()
            b_cache.reset_chunk_counter()
        n_text += 1
        for name in counters:
            va, vb = getattr(a_cache, name), getattr(b_cache, name)
            if name == "_capacity":   # an append-only buffer also holds the step's spare rows
                assert va[0] == vb[0] and all(x <= y for x, y in zip(va[1:], vb[1:]))
            else:
                assert va == vb, name
        for layer in range(3):
            a, e = a_cache.attention_range(layer)
            assert b_cache.attention_range(layer) == (a, e)
            assert torch.equal(a_cache.key_cache[layer][:, :, a:e], b_cache.key_cache[layer][:, :, a:e])
            assert torch.equal(a_cache.value_cache[layer][:, :, a:e], b_cache.value_cache[layer][:, :, a:e])
    assert n_boundaries >= 30


def test_cache_summary_growth():
    """Summary region overflows its headroom -> buffer grows to the right, rows keep their place."""
    C, S = 2, 1
    cache = _make_cache(C, S, [1])
    cache._SUMMARY_INIT_CAP = 4
    model = O.RingBufferModel(C, S, 1)
    model.SUMMARY_INIT_CAP = 4
    Sq = 3
    sp = O.summary_positions(Sq, C, S)
    kv = torch.arange(Sq, dtype=torch.float32)[None, None, :, None].expand(1, 1, Sq, 8).to(torch.bfloat16).contiguous()
    cache.update(kv, kv, 0, {"summary_mask": torch.from_numpy(sp)[None]})
    cache.reorganize_after_prefill(torch.from_numpy(sp)[None])
    model.reorganize_after_prefill(np.arange(Sq), sp)
    pos = Sq
    for step in range(1200):
        row = torch.full((1, 1, 1, 8), float(pos % 251), dtype=torch.bfloat16)
        cache.update_text(row, row, 0)
        model.update_text(pos % 251)
        pos += 1
        if cache._chunk_buf_len[0] == C:
            srow = torch.full((1, 1, S, 8), float(pos % 251), dtype=torch.bfloat16)
            cache.update_summary(srow, srow, 0)
            model.update_summary([pos % 251])
            pos += 1
    assert cache._capacity[0] == model.cap > 300
    a, b = model.attention_range()
    assert cache.attention_range(0) == (a, b)
    assert cache.key_cache[0][0, 0, a:b, 0].float().tolist() == [float(x) for x in model.buf[a:b]]


def test_split_heuristics_are_host_only_and_bounded():
    """`ksa_gemm_rows_auto_splits` / `ksa_decode_auto_splits` run on the host: the decoder's
    shapes get the split counts the kernels were tuned with, and any shape gets a count the
    kernels accept (at least 1, at most 16, never a slice shorter than one 512-element chunk)."""
    from ksa_amd import _lib
    L = _lib.lib()
    known = {(6144, 2560): 5, (2560, 4096): 8, (19456, 2560): 5, (2560, 9728): 13, (151936, 2560): 1}
    for (N, K), want in known.items():
        assert L.ksa_gemm_rows_auto_splits(N, K) == want, (N, K)
    rng = np.random.default_rng(0)
    for _ in range(200):
        N, K = int(rng.integers(1, 200000)), 32 * int(rng.integers(1, 600))
        sp = L.ksa_gemm_rows_auto_splits(N, K)
        assert 1 <= sp <= 16 and sp <= max(1, K // 512), (N, K, sp)
        assert L.ksa_gemm_rows_workspace_bytes(N, sp) == (0 if sp == 1 else sp * 16 * N * 4)
    for b, h, rows in [(64, 8, 17288), (8, 8, 40000), (1, 1, 100), (1, 8, 1 << 20)]:
        assert 1 <= L.ksa_decode_auto_splits(b, h, rows) <= 64
    assert L.ksa_decode_auto_splits(64, 8, 17288) == 1


def test_summary_pos_analysis_runs_once_for_fresh_views():
    """The HF call site passes `summary_mask.squeeze(0)`, a new tensor object per layer
    (modeling_qwen3sa.py:807-815): the analysis (one host synchronisation) must run once per
    buffer, not once per view, also for masks made under torch.inference_mode(), whose tensors
    have no modification counter."""
    from ksa_amd import prefill
    C, S = 16, 2
    Sq = 5 * (C + S) + 7
    for inference in (False, True):
        prefill.clear_summary_pos_cache()
        ctx = torch.inference_mode() if inference else torch.no_grad()
        with ctx:
            mask = (torch.arange(Sq) % (C + S) >= C)[None].clone()
            mask[0, 5 * (C + S):] = False
            before = prefill._POS_ANALYSES
            res = [prefill._analyse_summary_pos(mask.squeeze(0), Sq, C, S) for _ in range(3)]
        assert prefill._POS_ANALYSES - before == 1, inference
        assert all(r is res[0] for r in res)
        assert res[0][0] == 5 * S and res[0][1] is True and res[0][2] is None
    # an in-place edit of a tracked tensor is seen
    prefill.clear_summary_pos_cache()
    mask = (torch.arange(Sq) % (C + S) >= C).clone()
    mask[5 * (C + S):] = False
    a = prefill._analyse_summary_pos(mask, Sq, C, S)
    mask[3] = True
    b = prefill._analyse_summary_pos(mask, Sq, C, S)
    assert a[1] is True and b[1] is False and b[0] == a[0] + 1
    assert b[2].tolist() == sorted([3] + [i for i in range(5 * (C + S)) if i % (C + S) >= C])
    # a new mask of the same shape that reuses nothing of the old one is analysed on its own
    other = torch.zeros(Sq, dtype=torch.bool)
    assert prefill._analyse_summary_pos(other, Sq, C, S)[0] == 0
    prefill.clear_summary_pos_cache()
