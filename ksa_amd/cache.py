"""Ring-buffer KV cache with summary support — MI355X drop-in for the reference's
`Qwen3RingBufferCache` (examples/pretrain/hf_template/modeling_qwen3sa.py:85-505).

Same constructor, methods, attributes and buffer layout

    small-window layer: [ scratch S | chunk_text C (fills right->left) | ring scn*C |
                          summaries (append ->) | headroom ]
    large-window layer: append-only text rows (summaries are never stored)

so `modeling_qwen3sa.py` can use it unchanged.  Every row movement goes through the
`ksa_copy_rows` HIP kernel of libksa_hip.so (one launch per K and per V instead of the
reference's chains of `Tensor.copy_`); the integer bookkeeping is plain Python as in
the reference.  `attention_range(layer)` additionally exposes the `[start, end)` row
range of `get_attention_kv` so the decode kernel can be handed the whole buffer.
"""
from __future__ import annotations

from typing import Any, Optional

import torch

from . import _lib


def _move_rows(src: torch.Tensor, dst: torch.Tensor, nrows: int, src_start: int = 0,
               dst_start: int = 0, src_index: Optional[torch.Tensor] = None,
               dst_start_seq: Optional[torch.Tensor] = None) -> None:
    """dst[:, :, dst_start + i, :] <- src[:, :, src_index[i] | src_start + i, :] on the GPU.
    src/dst are [bsz, heads, rows, D] with contiguous rows.  `dst_start_seq` (int32 [bsz] on the
    GPU) replaces `dst_start` per sequence with values the kernel reads at run time, so a launch
    recorded in a HIP graph can be replayed with other destination rows."""
    if nrows <= 0:
        return
    bsz, heads, _, D = dst.shape
    assert src.is_cuda and dst.is_cuda, "the cache lives on the GPU"
    assert src.dtype == dst.dtype and src.element_size() == 2, "cache rows are 16-bit floats"
    if src.stride(-1) != 1:
        src = src.contiguous()
    if src.shape[0] != bsz or src.shape[1] != heads:
        src = src.expand(bsz, heads, src.shape[2], D)
    with torch.cuda.device(dst.device):
        rc = _lib.lib().ksa_copy_rows(
            src.data_ptr(), dst.data_ptr(),
            src_index.data_ptr() if src_index is not None else None,
            dst_start_seq.data_ptr() if dst_start_seq is not None else None,
            src_start, dst_start, nrows, bsz, heads, D,
            _lib.strides3(src, (0, 1, 2)), _lib.strides3(dst, (0, 1, 2)),
            _lib.stream_ptr(dst.device))
    _lib.check(rc, "ksa_copy_rows")


def _move_rows_multi(moves) -> None:
    """Up to 8 independent `_move_rows` (without source index lists) as one launch.  Each move is
    (src, dst, nrows, src_start, dst_start) with dst_start an int or an int32 GPU tensor [bsz] (read
    at run time); all tensors [bsz, heads, rows, D] of one shape class.  No move may read rows that
    another one writes."""
    moves = [m for m in moves if m[2] > 0]
    if not moves:
        return
    import ctypes
    bsz, heads, _, D = moves[0][1].shape
    n = len(moves)
    keep = []
    srcs, dsts, seqs = (ctypes.c_void_p * n)(), (ctypes.c_void_p * n)(), (ctypes.c_void_p * n)()
    s0, d0, nr = (ctypes.c_int * n)(), (ctypes.c_int * n)(), (ctypes.c_int * n)()
    sst, dst_ = (ctypes.c_int64 * (3 * n))(), (ctypes.c_int64 * (3 * n))()
    for i, (src, dst, nrows, src_start, dst_start) in enumerate(moves):
        assert src.is_cuda and dst.is_cuda and src.dtype == dst.dtype and src.element_size() == 2
        assert dst.shape[0] == bsz and dst.shape[1] == heads and dst.shape[3] == D
        if src.stride(-1) != 1:
            src = src.contiguous()
        if src.shape[0] != bsz or src.shape[1] != heads:
            src = src.expand(bsz, heads, src.shape[2], D)
        keep.append(src)
        srcs[i], dsts[i] = src.data_ptr(), dst.data_ptr()
        if torch.is_tensor(dst_start):
            assert dst_start.dtype == torch.int32 and dst_start.is_cuda and dst_start.numel() == bsz
            seqs[i], d0[i] = dst_start.data_ptr(), 0
        else:
            seqs[i], d0[i] = None, int(dst_start)
        s0[i], nr[i] = int(src_start), int(nrows)
        for j, dim in enumerate((0, 1, 2)):
            sst[3 * i + j], dst_[3 * i + j] = src.stride(dim), dst.stride(dim)
    dev = moves[0][1].device
    with torch.cuda.device(dev):
        rc = _lib.lib().ksa_copy_rows_multi(n, srcs, dsts, seqs, s0, d0, nr, bsz, heads, D, sst, dst_,
                                            _lib.stream_ptr(dev))
    _lib.check(rc, "ksa_copy_rows_multi")


class Qwen3RingBufferCache:
    is_compileable = False
    _SUMMARY_INIT_CAP = 512
    _APPEND_HEADROOM = 1024

    # row mover; tests without a GPU replace it with a host implementation
    _move_rows = staticmethod(_move_rows)

    def __init__(self, config, sliding_chunk_nums: list):
        self.summary_chunk_size = getattr(config, "summary_chunk_size", 0)
        self.summary_token_num = getattr(config, "summary_token_num", 0)
        n = self.num_hidden_layers = config.num_hidden_layers
        self.sliding_chunk_nums = sliding_chunk_nums
        C = self.summary_chunk_size
        self.window_sizes = [scn * C for scn in sliding_chunk_nums]
        smallest = min(self.window_sizes)
        self.is_large_window = [ws > smallest for ws in self.window_sizes]

        self.key_cache = [None] * n
        self.value_cache = [None] * n
        self._text_len = [0] * n          # append-only length (prefill, large window)
        self._capacity = [0] * n
        self._window_write_ptr = [0] * n  # next ring slot
        self._n_valid_window = [0] * n    # valid ring rows
        self._chunk_buf_len = [0] * n     # rows of the current chunk
        self._n_summaries = [0] * n
        self.cur_chunk_sizes = [0] * n
        self.true_tokens = [0] * n
        self._total_chunks = [0] * n
        self._reorganized = False
        self._reorg_done = set()   # layers already in the ring layout (`reorganize_layer`)
        self._reorg_rows = None    # (text rows, summary rows, counts) of the prefill, made once

    # ---- queries -------------------------------------------------------------------
    def __len__(self):
        return self.num_hidden_layers

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        if layer_idx >= self.num_hidden_layers:
            return 0
        if self.is_large_window[layer_idx]:
            return self._text_len[layer_idx]
        return (self._n_valid_window[layer_idx] + self._chunk_buf_len[layer_idx]
                + self._n_summaries[layer_idx])

    def get_cur_chunk_size(self, layer_idx: Optional[int] = None) -> int:
        return self.cur_chunk_sizes[self.num_hidden_layers - 1 if layer_idx is None else layer_idx]

    def get_true_token_num(self, layer_idx: Optional[int] = None) -> int:
        return self.true_tokens[self.num_hidden_layers - 1 if layer_idx is None else layer_idx]

    # ---- storage helpers -------------------------------------------------------------
    def _alloc(self, like: torch.Tensor, rows: int):
        bsz, heads, _, D = like.shape
        return torch.empty(bsz, heads, rows, D, dtype=like.dtype, device=like.device)

    def _regrow(self, layer: int, new_cap: int, keep_rows: int):
        """Replace the layer's buffers by larger ones, keeping rows [0, keep_rows)."""
        for store in (self.key_cache, self.value_cache):
            old = store[layer]
            new = self._alloc(old, new_cap)
            self._move_rows(old, new, keep_rows)
            store[layer] = new
        self._capacity[layer] = new_cap

    def _append(self, layer: int, k: torch.Tensor, v: torch.Tensor):
        """Append rows at _text_len (prefill before reorganisation, large-window decode)."""
        add = k.shape[-2]
        cur = self._text_len[layer]
        need = cur + add
        if self.key_cache[layer] is None:
            self.key_cache[layer] = self._alloc(k, need + self._APPEND_HEADROOM)
            self.value_cache[layer] = self._alloc(v, need + self._APPEND_HEADROOM)
            self._capacity[layer] = need + self._APPEND_HEADROOM
        elif need > self._capacity[layer]:
            self._regrow(layer, max(need + self._APPEND_HEADROOM, 2 * self._capacity[layer]), cur)
        self._move_rows(k, self.key_cache[layer], add, 0, cur)
        self._move_rows(v, self.value_cache[layer], add, 0, cur)
        self._text_len[layer] = need

    # ---- prefill ---------------------------------------------------------------------
    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict] = None):
        """Append prefill K/V [bsz, heads, n, D]; returns views of everything stored so far."""
        add = key_states.shape[-2]
        self._append(layer_idx, key_states, value_states)
        if self.summary_chunk_size > 0:
            n_text = add
            if cache_kwargs and "summary_mask" in cache_kwargs:
                n_text = add - int(cache_kwargs["summary_mask"][0].sum().item())
            self.cur_chunk_sizes[layer_idx] += add
            self.true_tokens[layer_idx] += n_text
        n = self._text_len[layer_idx]
        return self.key_cache[layer_idx][:, :, :n, :], self.value_cache[layer_idx][:, :, :n, :]

    def prefill_slots(self, layer_idx: int, bsz: int, heads: int, n: int, D: int, dtype, device,
                      n_summary: int = 0):
        """`update` without the copy: reserves `n` rows for prefill K/V and returns the two
        [bsz, n, heads, D] views of them for the producer to write (e.g. the pre-attention
        kernel).  Same counters as `update` with a summary mask holding `n_summary` rows."""
        cur = self._text_len[layer_idx]
        need = cur + n
        if self.key_cache[layer_idx] is None:
            cap = need + self._APPEND_HEADROOM
            self.key_cache[layer_idx] = torch.empty(bsz, heads, cap, D, dtype=dtype, device=device)
            self.value_cache[layer_idx] = torch.empty(bsz, heads, cap, D, dtype=dtype, device=device)
            self._capacity[layer_idx] = cap
        elif need > self._capacity[layer_idx]:
            self._regrow(layer_idx, max(need + self._APPEND_HEADROOM, 2 * self._capacity[layer_idx]), cur)
        self._text_len[layer_idx] = need
        if self.summary_chunk_size > 0:
            self.cur_chunk_sizes[layer_idx] += n
            self.true_tokens[layer_idx] += n - n_summary
        return (self.key_cache[layer_idx][:, :, cur:need, :].transpose(1, 2),
                self.value_cache[layer_idx][:, :, cur:need, :].transpose(1, 2))

    def text_slots(self, layer_idx: int, bsz: int, heads: int, D: int, dtype, device):
        """`update_text` without the copy: returns the [bsz, 1, heads, D] views of the row the
        next text token's K/V belong in and advances the counters."""
        if self.is_large_window[layer_idx]:
            row = self._text_len[layer_idx]
            if self.key_cache[layer_idx] is None:
                cap = row + 1 + self._APPEND_HEADROOM
                self.key_cache[layer_idx] = torch.empty(bsz, heads, cap, D, dtype=dtype, device=device)
                self.value_cache[layer_idx] = torch.empty(bsz, heads, cap, D, dtype=dtype, device=device)
                self._capacity[layer_idx] = cap
            elif row + 1 > self._capacity[layer_idx]:
                self._regrow(layer_idx, max(row + 1 + self._APPEND_HEADROOM, 2 * self._capacity[layer_idx]), row)
            self._text_len[layer_idx] = row + 1
        else:
            cbl = self._chunk_buf_len[layer_idx]
            row = self.summary_token_num + self.summary_chunk_size - 1 - cbl
            self._chunk_buf_len[layer_idx] = cbl + 1
        self.cur_chunk_sizes[layer_idx] += 1
        self.true_tokens[layer_idx] += 1
        return (self.key_cache[layer_idx][:, :, row:row + 1, :].transpose(1, 2),
                self.value_cache[layer_idx][:, :, row:row + 1, :].transpose(1, 2))

    def reorganize_after_prefill(self, summary_mask: torch.Tensor):
        """Prefill order -> ring layout for every layer.  summary_mask: bool [bsz, prefill_len]."""
        if self._reorganized:
            return
        for layer in range(self.num_hidden_layers):
            self.reorganize_layer(layer, summary_mask)
        self._reorganized = True

    def reorganize_layer(self, layer: int, summary_mask: torch.Tensor):
        """`reorganize_after_prefill` for one layer, for a prefill that calls it as soon as the layer's
        attention has run: a small-window layer then gives up all but its window and its summaries at
        once instead of holding the whole prompt's K/V until every layer has run (at the 4B shape 27 of
        36 layers; the reference reorganises all layers at the end, :209-302)."""
        if self._reorganized or layer in self._reorg_done:
            return
        self._reorg_done.add(layer)
        C, S = self.summary_chunk_size, self.summary_token_num
        if self._reorg_rows is None:
            sm = summary_mask[0]
            self._reorg_rows = (torch.nonzero(~sm, as_tuple=False).flatten().to(torch.int32),
                                torch.nonzero(sm, as_tuple=False).flatten().to(torch.int32))
        text_rows, sum_rows = self._reorg_rows
        n_text, n_sum = text_rows.numel(), sum_rows.numel()
        n_complete, n_partial = divmod(n_text, C)

        old_k, old_v = self.key_cache[layer], self.value_cache[layer]
        if self.is_large_window[layer]:
            cap = n_text + self._APPEND_HEADROOM
            new_k, new_v = self._alloc(old_k, cap), self._alloc(old_v, cap)
            self._move_rows(old_k, new_k, n_text, src_index=text_rows)
            self._move_rows(old_v, new_v, n_text, src_index=text_rows)
            self._text_len[layer] = n_text
        else:
            ws, scn = self.window_sizes[layer], self.sliding_chunk_nums[layer]
            n_win = min(scn, n_complete) * C
            cap = S + C + ws + n_sum + max(self._SUMMARY_INIT_CAP, n_sum + 256)
            new_k, new_v = self._alloc(old_k, cap), self._alloc(old_v, cap)
            first_win = n_complete * C - n_win
            for old, new in ((old_k, new_k), (old_v, new_v)):
                # trailing partial chunk, right-aligned in the chunk region
                self._move_rows(old, new, n_partial, dst_start=S + C - n_partial,
                                src_index=text_rows[n_complete * C:])
                # newest complete chunks, chronological, from the ring base
                self._move_rows(old, new, n_win, dst_start=S + C,
                                src_index=text_rows[first_win:n_complete * C])
                self._move_rows(old, new, n_sum, dst_start=S + C + ws, src_index=sum_rows)
            self._n_valid_window[layer] = n_win
            self._window_write_ptr[layer] = n_win % ws
            self._n_summaries[layer] = n_sum
            self._chunk_buf_len[layer] = n_partial
            self._text_len[layer] = 0
        self.key_cache[layer], self.value_cache[layer] = new_k, new_v
        self._capacity[layer] = cap
        self.cur_chunk_sizes[layer] %= C + S
        self._total_chunks[layer] = (self.true_tokens[layer] // C if self.is_large_window[layer]
                                     else self._n_summaries[layer])

    # ---- decode ----------------------------------------------------------------------
    def update_text(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int):
        """Store one text token's K/V [bsz, heads, 1, D]."""
        if self.is_large_window[layer_idx]:
            self._append(layer_idx, key_states, value_states)
        else:
            cbl = self._chunk_buf_len[layer_idx]
            dst = self.summary_token_num + self.summary_chunk_size - 1 - cbl
            self._move_rows(key_states, self.key_cache[layer_idx], 1, 0, dst)
            self._move_rows(value_states, self.value_cache[layer_idx], 1, 0, dst)
            self._chunk_buf_len[layer_idx] = cbl + 1
        self.cur_chunk_sizes[layer_idx] += 1
        self.true_tokens[layer_idx] += 1

    def update_summary(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int):
        """Chunk boundary: flush the chunk region into the ring, append the summary rows."""
        n_new = key_states.shape[2]
        if not self.is_large_window[layer_idx]:
            C, S = self.summary_chunk_size, self.summary_token_num
            ws = self.window_sizes[layer_idx]
            cbl, ptr = self._chunk_buf_len[layer_idx], self._window_write_ptr[layer_idx]
            src = S + C - cbl
            first = min(cbl, ws - ptr)  # rows that fit before the ring wraps
            for buf in (self.key_cache[layer_idx], self.value_cache[layer_idx]):
                self._move_rows(buf, buf, first, src, S + C + ptr)
                self._move_rows(buf, buf, cbl - first, src + first, S + C)
            self._window_write_ptr[layer_idx] = (ptr + cbl) % ws
            self._n_valid_window[layer_idx] = min(ws, self._n_valid_window[layer_idx] + cbl)
            self._chunk_buf_len[layer_idx] = 0

            dst = S + C + ws + self._n_summaries[layer_idx]
            if dst + n_new > self._capacity[layer_idx]:
                self._grow_buffer_right(layer_idx)
            self._move_rows(key_states, self.key_cache[layer_idx], n_new, 0, dst)
            self._move_rows(value_states, self.value_cache[layer_idx], n_new, 0, dst)
            self._n_summaries[layer_idx] += n_new
        self.cur_chunk_sizes[layer_idx] += n_new
        self._total_chunks[layer_idx] += n_new

    def boundary_fits_one_piece(self, layer_idx: int) -> bool:
        """True when the flush of a chunk-boundary step that starts now (the chunk's last text row
        still to come) is one run of rows in the ring, i.e. `boundary_slots` can describe it."""
        if self.is_large_window[layer_idx]:
            return True
        cbl = self._chunk_buf_len[layer_idx] + 1
        return cbl <= self.window_sizes[layer_idx] - self._window_write_ptr[layer_idx]

    def boundary_slots(self, layer_idx: int, n_new: int):
        """`update_text` of a chunk's last text token followed by `update_summary` of its `n_new`
        summary rows, without moving a row: advances the counters (enlarging a buffer that is too
        small) and returns the rows the two calls would have used, for a caller that moves the
        rows itself (a launch sequence replayed with the rows in device memory):

            small window: text (row of the text token), attend (start, end of the text query's
                          range, taken between the two calls as `decode_step` does), flush_src,
                          flush_dst, flush_rows (chunk rows -> ring), append (row of the first
                          new summary)
            large window: text, attend, and spare = the first of `n_new` rows behind the text that
                          the caller may use for the summary rows of the step (they are not kept)

        Requires `boundary_fits_one_piece(layer_idx)`."""
        C, S = self.summary_chunk_size, self.summary_token_num
        if self.is_large_window[layer_idx]:
            row = self._text_len[layer_idx]
            if row + 1 + n_new > self._capacity[layer_idx]:
                self._regrow(layer_idx, max(row + 1 + n_new + self._APPEND_HEADROOM,
                                            2 * self._capacity[layer_idx]), row)
            self._text_len[layer_idx] = row + 1
            out = dict(text=row, attend=(0, row + 1), spare=row + 1)
        else:
            assert self.boundary_fits_one_piece(layer_idx)
            ws = self.window_sizes[layer_idx]
            cbl = self._chunk_buf_len[layer_idx] + 1
            row = S + C - cbl
            self._chunk_buf_len[layer_idx] = cbl
            attend = self.attention_range(layer_idx)
            ptr = self._window_write_ptr[layer_idx]
            self._window_write_ptr[layer_idx] = (ptr + cbl) % ws
            self._n_valid_window[layer_idx] = min(ws, self._n_valid_window[layer_idx] + cbl)
            self._chunk_buf_len[layer_idx] = 0
            dst = S + C + ws + self._n_summaries[layer_idx]
            if dst + n_new > self._capacity[layer_idx]:
                self._grow_buffer_right(layer_idx)
            self._n_summaries[layer_idx] += n_new
            out = dict(text=row, attend=attend, flush_src=row, flush_dst=S + C + ptr, flush_rows=cbl,
                       append=dst)
        self.cur_chunk_sizes[layer_idx] += 1 + n_new
        self.true_tokens[layer_idx] += 1
        self._total_chunks[layer_idx] += n_new
        return out

    def attention_range(self, layer_idx: int):
        """Row range [start, end) a text query attends (the slice of get_attention_kv)."""
        if self.is_large_window[layer_idx]:
            return 0, self._text_len[layer_idx]
        C, S = self.summary_chunk_size, self.summary_token_num
        ws = self.window_sizes[layer_idx]
        start = S + C - self._chunk_buf_len[layer_idx]
        if self._n_valid_window[layer_idx] >= ws:
            # summaries of the chunks still in the ring are not attended
            n_sum = self._n_summaries[layer_idx]
            hidden = min(self.sliding_chunk_nums[layer_idx] * S, n_sum)
            return start, S + C + ws + n_sum - hidden
        return start, S + C + self._n_valid_window[layer_idx]

    def get_attention_kv(self, layer_idx: int):
        a, b = self.attention_range(layer_idx)
        return self.key_cache[layer_idx][:, :, a:b, :], self.value_cache[layer_idx][:, :, a:b, :]

    def get_current_chunk_kv(self, layer_idx: int):
        C = self.summary_chunk_size
        if self.is_large_window[layer_idx]:
            b = self._text_len[layer_idx]
            a = b - C
        else:
            b = self.summary_token_num + C
            a = b - self._chunk_buf_len[layer_idx]
        return self.key_cache[layer_idx][:, :, a:b, :], self.value_cache[layer_idx][:, :, a:b, :]

    def get_summary_attention_kv(self, layer_idx: int, k_summary: torch.Tensor, v_summary: torch.Tensor):
        """K/V the summary queries of a boundary step attend: [own summaries | chunk text]."""
        C, S = self.summary_chunk_size, self.summary_token_num
        if self.is_large_window[layer_idx]:
            tl = self._text_len[layer_idx]
            k_chunk = self.key_cache[layer_idx][:, :, tl - C:tl, :]
            v_chunk = self.value_cache[layer_idx][:, :, tl - C:tl, :]
            return torch.cat([k_chunk, k_summary], dim=2), torch.cat([v_chunk, v_summary], dim=2)
        self._move_rows(k_summary, self.key_cache[layer_idx], S, 0, 0)
        self._move_rows(v_summary, self.value_cache[layer_idx], S, 0, 0)
        return self.key_cache[layer_idx][:, :, :S + C, :], self.value_cache[layer_idx][:, :, :S + C, :]

    def _grow_buffer_right(self, layer_idx: int):
        old_cap = self._capacity[layer_idx]
        extra = max(self._SUMMARY_INIT_CAP, self._n_summaries[layer_idx])
        self._regrow(layer_idx, max(old_cap + extra, 2 * old_cap), old_cap)

    def reset_chunk_counter(self):
        block = self.summary_chunk_size + self.summary_token_num
        for layer in range(self.num_hidden_layers):
            if self.cur_chunk_sizes[layer] >= block:
                self.cur_chunk_sizes[layer] %= block
