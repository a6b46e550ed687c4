"""End-to-end KSA decoder (Qwen3 shape with Summary Attention) on the MI355X kernels.

The caller of both hot paths, restated from the reference's inference model
(examples/pretrain/hf_template/modeling_qwen3sa.py): `Qwen3Model.forward` :1203-1324 (expand the
prompt with summary tokens, run the layers, reorganise the cache after prefill, drop the summary
rows), `_expand_input_with_summary_tokens` :1080-1177, `Qwen3DecoderLayer.forward` :905-953,
`Qwen3SummaryAttention.forward` :741-880 (prefill / one-token decode / chunk-boundary decode),
`Qwen3MLP` :507-514, `Qwen3RMSNorm` :64-79, `Qwen3RotaryEmbedding` :975-1032,
`Qwen3ForCausalLM.forward` :1343-1420 (logits of the last position, truncated to the text
vocabulary) and `prepare_inputs_for_generation` :1432-1560 (what a decode step feeds: the new
token, plus the summary tokens when the chunk completes, and their position ids).

Differences from the reference, on purpose:
* any batch size (the reference refuses batch > 1 at :753; its cache tensors and counters are
  already batch-shaped, all sequences of a batch have the same length);
* weights are plain tensors (fused q|k|v and gate|up matrices), not nn.Modules; the GEMMs are
  torch matmuls (hipBLASLt) except for the few rows of a decode step (`ksa_gemm_rows`);
  everything else (pre-attention, attention, cache rows, residual add + RMSNorm, SiLU-mul) is
  this package's kernels;
* a "full attention" layer is, as in the reference's inference model, a Summary layer whose
  window is larger than any sequence (append-only text cache, :114-115, :232-242);
* `summary_independent_parameters` (:756-789): for mix_coeff 1 (the reference's default) the
  summary rows take their q, k, v from their own projection, for mix_coeff 0 that projection is
  unused, and in between the two are blended.  The reference blends the normalised q and k (and
  the plain v) before the rotary embedding; the rotation is linear, so the blend is done here on
  the outputs of the fused pre-attention step instead.

The attention-side and element-wise operators come from an `ops` object; the default binds the
HIP kernels of this package and needs a GPU.  Tests pass a CPU fp32 implementation of the same
operators to obtain the reference run of this very module.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Tuple, Union

import torch
import torch.nn.functional as F


@dataclass
class KsaQwen3Config:
    """Field names follow the reference's config.json (examples/pretrain/hf_template/config.json)."""
    hidden_size: int = 2560
    num_hidden_layers: int = 36
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 9728
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1e6
    vocab_size: int = 151936
    initializer_range: float = 0.02
    tie_word_embeddings: bool = True
    summary_chunk_size: int = 128
    summary_token_num: int = 8
    summary_token_begin: int = 151936          # ids of the summary tokens: begin .. begin + num - 1
    # per layer; the reference writes this as a pattern string such as "([4]*3+[1024]*1)*9".
    # As in the reference's cache (:114-115) there are two kinds of layers: those with the
    # smallest window, and "large window" layers (anything larger), which keep every text row
    # and no summaries during decoding.
    summary_sliding_chunk_num: Union[int, List[int]] = field(
        default_factory=lambda: ([4] * 3 + [1 << 20]) * 9)
    summary_chunk_position_ids_type: str = "origin"
    summary_token_position_ids_type: str = "last_chunk_slice_right"
    summary_independent_parameters: bool = False
    mix_coeff: float = 1.0

    def sliding_chunk_nums(self) -> List[int]:
        v = self.summary_sliding_chunk_num
        if isinstance(v, int):
            return [v] * self.num_hidden_layers
        v = [int(x) for x in v]
        if len(v) != self.num_hidden_layers:
            raise ValueError(f"summary_sliding_chunk_num has {len(v)} entries for "
                             f"{self.num_hidden_layers} layers")
        return v

    def embedding_rows(self) -> int:
        return max(self.vocab_size, self.summary_token_begin + self.summary_token_num)


def init_weights(config: KsaQwen3Config, device, dtype=torch.bfloat16, seed: int = 0) -> dict:
    """Random weights as the reference initialises them (normal, std = initializer_range, for
    every Linear and Embedding; RMSNorm weights 1), drawn on `device` tensor by tensor and rounded
    to `dtype`."""
    g = torch.Generator(device=device).manual_seed(seed)
    std = config.initializer_range
    H, D = config.hidden_size, config.head_dim
    nq, nkv, I = config.num_attention_heads * D, config.num_key_value_heads * D, config.intermediate_size

    def normal(*shape):
        return (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * std).to(dtype)

    def ones(n):
        return torch.ones(n, device=device, dtype=dtype)

    layers = []
    for _ in range(config.num_hidden_layers):
        lw = {
            "input_layernorm": ones(H), "post_attention_layernorm": ones(H),
            "qkv_proj": normal(nq + 2 * nkv, H),        # rows: q | k | v
            "q_norm": ones(D), "k_norm": ones(D),
            "o_proj": normal(H, nq),
            "gate_up_proj": normal(2 * I, H),           # rows: gate | up
            "down_proj": normal(H, I),
        }
        if config.summary_independent_parameters:
            lw["qkv_proj_summary"] = normal(nq + 2 * nkv, H)
        layers.append(lw)
    w = {"embed_tokens": normal(config.embedding_rows(), H), "layers": layers, "norm": ones(H)}
    if not config.tie_word_embeddings:
        w["lm_head"] = normal(config.vocab_size, H)
    return w


def convert_weights(weights: dict, device, dtype) -> dict:
    """The same weights on another device / in another dtype (e.g. the fp32 CPU copy of a bf16 set)."""
    def conv(x):
        if isinstance(x, torch.Tensor):
            return x.to(device=device, dtype=dtype)
        if isinstance(x, dict):
            return {k: conv(v) for k, v in x.items()}
        if isinstance(x, list):
            return [conv(v) for v in x]
        return x
    return conv(weights)


class HipOps:
    """The attention-side operators of the model, bound to this package's HIP kernels."""

    def __init__(self):
        from . import cache, decode, elementwise, gemm, pre, prefill
        self.cache_cls = cache.Qwen3RingBufferCache
        self.pre_attention = pre.pre_attention
        self.pre_attention_partials = pre.pre_attention_partials
        self.summary_attn_func = prefill.summary_attn_func
        self.add_rmsnorm = elementwise.add_rmsnorm
        self.silu_mul = elementwise.silu_mul
        self._decode = decode.ksa_decode
        self.decode_boundary = decode.ksa_decode_boundary   # text token + summary tokens of a boundary step, one launch
        self.move_rows_multi = cache._move_rows_multi        # the step's row moves, one launch for up to eight
        self._linear_rows = gemm.linear_rows
        self._gate_up_silu_rows = gemm.gate_up_silu_rows
        self._argmax_rows = elementwise.argmax_rows
        self._max_rows = gemm.MAX_ROWS
        self._gemm = gemm
        self.timeout_error = gemm.MlpRowsTimeout
        self._mlp_ws = {}   # (device, H, I) -> MlpRowsWorkspace, see `mlp_rows`
        # False: the MLP of a decode step runs as separate launches (set after a one-launch MLP timed out)
        self.mlp_one_launch = True
        # True: the few-rows kernels of the decode steps read a second copy of every projection matrix in
        # their streaming layout (`gemm.TiledWeight`: + the size of those matrices in device memory, made the
        # first time a matrix is used at a decode step; q|k|v -7 %, down -15 %, gate|up -10 % of the kernel time)
        self.tile_weights = True
        self._tiled = {}    # (address, shape, row stride) -> (the matrix, its TiledWeight)

    def _streaming(self, weight, multiple=16):
        """`weight` in the streaming layout (kept with the matrix it was made from, so that the key stays
        unique for as long as the copy exists); the matrix itself where that layout does not apply."""
        if not self.tile_weights or not torch.is_tensor(weight) or weight.dim() != 2 or weight.stride(1) != 1 \
                or weight.shape[1] % 32 or weight.shape[0] % multiple or weight.stride(0) % 8:
            return weight
        key = (weight.data_ptr(), tuple(weight.shape), weight.stride(0))
        hit = self._tiled.get(key)
        if hit is None:
            hit = self._tiled[key] = (weight, self._gemm.TiledWeight(weight))
        return hit[1]

    def decode(self, q, kbuf, vbuf, start, end, scale):
        return self._decode(q, kbuf, vbuf, start, end, scale=scale)

    def argmax(self, logits):
        """Greedy token choice over the last dimension (lowest index among equal values)."""
        if (logits.dtype in (torch.bfloat16, torch.float16) and logits.stride(-1) == 1 and logits.dim() == 2
                and logits.stride(0) % 8 == 0 and logits.data_ptr() % 16 == 0):
            return self._argmax_rows(logits)
        return logits.argmax(-1)

    def prepare_mlp_rows(self, H, I, device):
        """Makes the workspace of `mlp_rows` for this MLP shape ahead of time (it has to exist, zeroed,
        before a step that uses it is recorded into a graph)."""
        key = (str(device), H, I)
        if key not in self._mlp_ws:
            self._mlp_ws[key] = self._gemm.MlpRowsWorkspace(H, I, device)
        return self._mlp_ws[key]

    def mlp_rows(self, x, w_gate_up, w_down):
        """down(SiLU(gate(x)) * up(x)) for the few rows of a decode step in one launch, as the K-split
        partial sums of the down projection; None when the shape is outside what that kernel takes."""
        rows = x.numel() // x.shape[-1]
        H, I = x.shape[-1], w_down.shape[1]
        if not self.mlp_one_launch or not self._gemm.mlp_rows_supported(rows, H, I):
            return None
        return self._gemm.mlp_rows(x, self._streaming(w_gate_up, 32), self._streaming(w_down),
                                   self.prepare_mlp_rows(H, I, x.device))

    def add_norm_mlp_rows(self, o_partials, residual, norm_weight, eps, w_gate_up, w_down):
        """(residual + o_proj output, down(SiLU(gate(h)) * up(h)) for h = norm of that sum) in one launch,
        from the K-split partial sums of the o projection; None when the shapes are outside what the
        kernel takes."""
        if not self.mlp_one_launch or not isinstance(o_partials, self._gemm.SplitKPartials):
            return None
        H, I = residual.shape[-1], w_down.shape[1]
        if not self._gemm.mlp_rows_supported(o_partials.rows, H, I) or H > 4096:
            return None
        return self._gemm.add_rmsnorm_mlp_rows(o_partials, residual, norm_weight, eps, self._streaming(w_gate_up, 32),
                                               self._streaming(w_down), self.prepare_mlp_rows(H, I, residual.device))

    def mlp_rows_failed(self):
        """True if a `mlp_rows` launch gave up waiting since the last call (waits for the device; every
        workspace is looked at and, where needed, cleared: see `MlpRowsWorkspace.failed`)."""
        return any([ws.failed() for ws in self._mlp_ws.values()])

    def check_mlp_rows(self):
        """Raises `MlpRowsTimeout` if a one-launch MLP gave up waiting since the last check, and from
        then on runs the MLP of a decode step as separate launches, which depend on nothing but the
        order of launches on a stream."""
        if self.mlp_one_launch and self.mlp_rows_failed():
            self.mlp_one_launch = False
            raise self._gemm.MlpRowsTimeout(
                "ksa_mlp_rows: a workgroup gave up waiting for the tiles it depends on; the steps since the "
                "last check are not valid.  The one-launch MLP is switched off for this operator set.")

    def gate_up_act(self, x, weight):
        """SiLU(x W_gate^T) * (x W_up^T) for the fused gate | up matrix: one kernel for the few rows of
        a decode step, the library GEMM and the activation kernel otherwise."""
        rows = x.numel() // x.shape[-1]
        k = x.shape[-1]
        if rows <= self._max_rows and k % 32 == 0 and (rows > 16 or rows * (k + 8) * 2 <= 160 * 1024):
            return self._gate_up_silu_rows(x, self._streaming(weight, 32))
        if rows <= self._max_rows:
            return self.silu_mul(self._linear_rows(x, self._streaming(weight), defer=True))
        return self.silu_mul(F.linear(x, weight))

    def linear(self, x, weight, defer=False):
        """x W^T: the weight-streaming kernel for the few rows of a decode step, the library
        GEMM otherwise.  `defer`: the caller hands the result to `add_rmsnorm` as it is, so a
        product split over K may come back as its partial sums (one launch less)."""
        rows = x.numel() // x.shape[-1]
        if rows <= self._max_rows and x.shape[-1] % 32 == 0:
            return self._linear_rows(x, self._streaming(weight), defer=defer)
        return F.linear(x, weight)


def expand_with_summary_tokens(input_ids: torch.Tensor, config: KsaQwen3Config):
    """Prompt -> (ids with `summary_token_num` summary ids after every complete chunk, position
    ids [1, L], summary mask [L]).  Text keeps its original positions ('origin'); summary token k
    (1-based, 'last_chunk_slice_right') of chunk i sits at i*C + (k*C)//S - 1, token k-1 of
    'last_chunk_slice_left' at max(i*C, i*C + ((k-1)*C)//S - 1); 'zeros' and 'inner_chunk' as in
    the reference (:1134-1175)."""
    C, S = config.summary_chunk_size, config.summary_token_num
    bsz, n = input_ids.shape
    dev = input_ids.device
    n_full, rem = divmod(n, C)
    blk = C + S
    L = n_full * blk + rem
    slot = torch.arange(L, device=dev)
    chunk, off = slot // blk, slot % blk
    is_sum = off >= C
    text_src = chunk * C + torch.clamp(off, max=C - 1)
    ids = input_ids[:, text_src]
    sum_ids = (config.summary_token_begin + (off - C)).to(input_ids.dtype)
    ids = torch.where(is_sum[None], sum_ids[None].expand(bsz, -1), ids)

    if config.summary_chunk_position_ids_type == "origin":
        text_pos = text_src
    elif config.summary_chunk_position_ids_type == "inner_chunk":
        text_pos = torch.clamp(off, max=C - 1)
    else:
        raise ValueError(f"summary_chunk_position_ids_type {config.summary_chunk_position_ids_type!r}")
    kind = config.summary_token_position_ids_type
    if kind == "zeros":
        sum_pos = torch.zeros_like(slot)
    elif kind in ("last_chunk_slice_left", "last_chunk_slice_right"):
        k = (off - C) + (1 if kind == "last_chunk_slice_right" else 0)
        sum_pos = torch.maximum(chunk * C + (k * C) // S - 1, chunk * C)
    else:
        raise ValueError(f"summary_token_position_ids_type {kind!r}")
    pos = torch.where(is_sum, sum_pos, text_pos)
    return ids, pos[None], is_sum


def boundary_position_ids(true_tokens: int, config: KsaQwen3Config, device) -> torch.Tensor:
    """Position ids [1, 1 + S] of a chunk-boundary decode step: the text token at its index in
    the text, the summary tokens by the same slice rule as in prefill (:1497-1531)."""
    C, S = config.summary_chunk_size, config.summary_token_num
    kind = config.summary_token_position_ids_type
    if config.summary_chunk_position_ids_type == "origin":
        text = true_tokens
    elif config.summary_chunk_position_ids_type == "inner_chunk":
        text = C - 1
    else:
        raise ValueError(f"summary_chunk_position_ids_type {config.summary_chunk_position_ids_type!r}")
    prev_end = true_tokens + 1 - C
    if kind == "zeros":
        sp = torch.zeros(S, dtype=torch.long, device=device)
    elif kind in ("last_chunk_slice_left", "last_chunk_slice_right"):
        k = torch.arange(S, device=device, dtype=torch.long) + (1 if kind == "last_chunk_slice_right" else 0)
        sp = torch.clamp(prev_end + (k * C) // S - 1, min=prev_end)
    else:
        raise ValueError(f"summary_token_position_ids_type {kind!r}")
    return torch.cat([torch.tensor([text], dtype=torch.long, device=device), sp])[None]


class KsaQwen3ForCausalLM:
    """Inference-only decoder: `forward` for one prefill or one decode step, `generate` for a
    greedy loop.  All sequences of a batch have the same length."""

    # `decode_step_graph` runs this many chunk-boundary steps of a cache eagerly before it records
    # them: a replayed boundary step saves about 1 ms against an eager one (6.2 against 7.2 ms at the
    # 4B shape, batch 8), its recording costs about 17 ms more than an eager step (an eager run outside
    # the capture first, then the capture), i.e. sixteen boundaries' worth: so a short generation never
    # pays for a recording it does not use, and a long one pays at most twice the best possible.
    BOUNDARY_GRAPH_AFTER = 16

    def __init__(self, config: KsaQwen3Config, weights: dict, ops=None):
        self.config = config
        self.w = weights
        self.ops = ops if ops is not None else HipOps()
        if config.summary_independent_parameters and not 0.0 <= float(config.mix_coeff) <= 1.0:
            raise ValueError("mix_coeff must lie in [0, 1]")
        self.scns = config.sliding_chunk_nums()
        D = config.head_dim
        self.inv_freq = 1.0 / (config.rope_theta ** (torch.arange(0, D, 2, dtype=torch.int64).float() / D))
        self.scaling = D ** -0.5
        emb = weights["embed_tokens"]
        self.dtype, self.device = emb.dtype, emb.device
        self.inv_freq_dev = self.inv_freq.to(self.device)
        self.lm_head = emb[: config.vocab_size] if config.tie_word_embeddings else weights["lm_head"]
        if hasattr(self.ops, "prepare_mlp_rows") and self.device.type == "cuda":
            self.ops.prepare_mlp_rows(config.hidden_size, config.intermediate_size, self.device)

    # ---- pieces ----------------------------------------------------------------------
    def _add_norm(self, delta, x, w):
        """(x + delta, w * rmsnorm(x + delta)); delta None: (x, w * rmsnorm(x))."""
        if delta is None:
            return self.ops.add_rmsnorm(x, None, w, self.config.rms_norm_eps)
        return self.ops.add_rmsnorm(delta, x, w, self.config.rms_norm_eps)

    def _boundary_rows_in_cache(self):
        """Whether a boundary step may write the new K/V rows straight to their cache rows (a row per token,
        `pre_attention(..., kv_out_row=[b, 1 + S])`): the fused operators, and no second set of summary
        projections whose rows are blended in after the pre-attention step."""
        return (hasattr(self.ops, "decode_boundary") and hasattr(self.ops, "pre_attention_partials")
                and not self.config.summary_independent_parameters)

    def _boundary_row_table(self, text, base, b):
        """int32 [b, 1 + S] on the device: the cache row of every token of a boundary step - the text token's
        row `text`, summary token i at `base + i`; `text` / `base` ints or int32 device tensors [b]."""
        S = self.config.summary_token_num
        if not torch.is_tensor(text) and not torch.is_tensor(base):
            row = [int(text)] + [int(base) + i for i in range(S)]
            return torch.tensor([row] * b, dtype=torch.int32).to(self.device)
        # (no host-to-device copies: this runs inside a recording)
        some = text if torch.is_tensor(text) else base
        as_rows = lambda v: v.to(torch.int32).expand(b) if torch.is_tensor(v) else torch.full_like(some, int(v), dtype=torch.int32).expand(b)
        ar = torch.arange(S, dtype=torch.int32, device=self.device)
        return torch.cat([as_rows(text)[:, None], as_rows(base)[:, None] + ar[None]], dim=1).contiguous()

    def _boundary_qkv(self, lw, h, sum_rows, cos, sin, slots=None):
        """q, k, v [b, 1 + S, H, D] (normalised, rotated) of a chunk-boundary step's rows.  With one
        set of projection weights the product may stay the K-split partial sums of the few-rows GEMM,
        which the pre-attention kernel adds itself (one launch less).  `slots` = (key cache, value cache,
        row table of `_boundary_row_table`): k and v go straight to those cache rows and are not returned."""
        cfg, ops = self.config, self.ops
        out = {}
        if slots is not None:
            kc, vc, table = slots
            n = table.shape[1]
            out = dict(k_out=kc[:, :, :n].transpose(1, 2), v_out=vc[:, :, :n].transpose(1, 2), kv_out_row=table)
        qkv = None
        if not cfg.summary_independent_parameters and hasattr(ops, "pre_attention_partials"):
            qkv = ops.linear(h, lw["qkv_proj"], defer=True)
        if qkv is not None and not torch.is_tensor(qkv):
            q, k, v = ops.pre_attention_partials(qkv, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                                                 lw["q_norm"], lw["k_norm"], cos, sin, cfg.rms_norm_eps, **out)
            return (q, None, None) if slots is not None else (q, k, v)
        q, k, v = self._split_qkv(qkv) if qkv is not None else self._qkv(lw, h, sum_rows)
        q, k, v = ops.pre_attention(q, k, v, lw["q_norm"], lw["k_norm"], cos, sin, cfg.rms_norm_eps, **out)
        if slots is not None:
            return q, None, None
        self._blend_summary(lw, h, sum_rows, cos, sin, q, k, v)
        return q, k, v

    def _boundary_logits(self, x, delta):
        """Logits of the text rows (row 0 of every sequence) behind the last layer of a boundary step."""
        if torch.is_tensor(delta):
            return self._logits(x[:, :1], delta[:, :1])
        # (the last MLP's partial sums cover all rows: final norm over all of them, logits of the text rows)
        _, h = self._add_norm(delta, x, self.w["norm"])
        return self.ops.linear(h[:, :1], self.lm_head)[..., : self.config.vocab_size]

    def _boundary_attention(self, qh, kh, vh, kc, vc, large, rows):
        """Attention and cache update of one layer at a chunk-boundary step with the fused operators
        (`ops.decode_boundary`, `ops.move_rows_multi`): three launches (+ the merge) in place of the
        reference's sequence (:831-876, :306-398, :476-497: update_text, attention of the text token,
        summaries into the scratch rows, attention of the summary tokens, flush, append) of twelve.
        qh [b, Hq, 1 + S, D], kh, vh [b, Hkv, 1 + S, D]; `rows` names the cache rows as
        `Qwen3RingBufferCache.boundary_slots` does, every value an int or an int32 device tensor [b]:
        small window: text, start, end, flush_src, flush_dst, flush_rows, append; large window: text,
        start, end, spare, sum_start, sum_end (= spare - C, spare + S).  Returns [b, 1 + S, Hq, D].
        kh, vh None: the pre-attention step has already written the step's K/V rows to the cache (text
        row, scratch rows of a small window / spare rows of a large one), which leaves two launches
        (+ the merge)."""
        ops = self.ops
        C, S = self.config.summary_chunk_size, self.config.summary_token_num
        in_cache = kh is None
        if not in_cache:
            kt, vt, ks, vs = kh[:, :, :1], vh[:, :, :1], kh[:, :, 1:], vh[:, :, 1:]
        if large:
            # the summary rows sit in spare rows behind the text for the length of the step, so that
            # [chunk text | own summaries] is one row range
            sp = rows["spare"]
            if not in_cache:
                ops.move_rows_multi([(kt, kc, 1, 0, rows["text"]), (vt, vc, 1, 0, rows["text"]),
                                     (ks, kc, S, 0, sp), (vs, vc, S, 0, sp)])
            return ops.decode_boundary(qh, kc, vc, rows["start"], rows["end"], rows["sum_start"], rows["sum_end"],
                                       self.scaling)
        if not in_cache:
            ops.move_rows_multi([(kt, kc, 1, 0, rows["text"]), (vt, vc, 1, 0, rows["text"]),
                                 (ks, kc, S, 0, 0), (vs, vc, S, 0, 0)])
        attn = ops.decode_boundary(qh, kc, vc, rows["start"], rows["end"], 0, S + C, self.scaling)
        # (the summaries are appended from the scratch rows when they did not come as tensors)
        ops.move_rows_multi([(kc, kc, rows["flush_rows"], rows["flush_src"], rows["flush_dst"]),
                             (vc, vc, rows["flush_rows"], rows["flush_src"], rows["flush_dst"]),
                             (kc if in_cache else ks, kc, S, 0, rows["append"]),
                             (vc if in_cache else vs, vc, S, 0, rows["append"])])
        return attn

    def _post_attention(self, lw, attn, x):
        """The second half of a layer at a decode step, from the attention output: (x', delta) with
        x' = x + o_proj(attn) and delta = mlp(post_attention_layernorm(x')) (deferred sums)."""
        o = self.ops.linear(attn, lw["o_proj"], defer=True)
        if hasattr(self.ops, "add_norm_mlp_rows"):
            out = self.ops.add_norm_mlp_rows(o, x, lw["post_attention_layernorm"], self.config.rms_norm_eps,
                                             lw["gate_up_proj"], lw["down_proj"])
            if out is not None:
                return out
        x, h = self._add_norm(o, x, lw["post_attention_layernorm"])
        return x, self._mlp(lw, h, defer=True)

    def _rope_tables(self, position_ids):
        """cos, sin [1, L, D] in the model dtype from position ids [1, L] (computed in fp32)."""
        freqs = position_ids[0].to(self.device).float()[:, None] * self.inv_freq_dev[None, :]
        emb = torch.cat((freqs, freqs), dim=-1)
        return emb.cos().to(self.dtype)[None], emb.sin().to(self.dtype)[None]

    def _qkv(self, lw, h, summary_rows):
        """Projection outputs as strided views q [b, L, Hq, D], k, v [b, L, Hkv, D]."""
        cfg = self.config
        D, Hq, Hkv = cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads
        qkv = self.ops.linear(h, lw["qkv_proj"])
        if (cfg.summary_independent_parameters and cfg.mix_coeff == 1 and summary_rows is not None
                and summary_rows.numel() > 0):
            qkv[:, summary_rows] = self.ops.linear(h[:, summary_rows], lw["qkv_proj_summary"])
        return self._split_qkv(qkv)

    def _blend_summary(self, lw, h, summary_rows, cos, sin, q, k, v):
        """mix_coeff strictly between 0 and 1 (:776-788): the summary rows of q, k, v (already
        normalised and rotated, from the shared projection) become
        mix * (the same from the summary projection) + (1 - mix) * themselves, in place."""
        cfg = self.config
        m = float(cfg.mix_coeff)
        if (not cfg.summary_independent_parameters or m in (0.0, 1.0) or summary_rows is None
                or summary_rows.numel() == 0):
            return
        qs, ks, vs = self._split_qkv(self.ops.linear(h[:, summary_rows], lw["qkv_proj_summary"]))
        qs, ks, vs = self.ops.pre_attention(qs, ks, vs, lw["q_norm"], lw["k_norm"], cos[:, summary_rows],
                                            sin[:, summary_rows], cfg.rms_norm_eps)
        for dst, src in ((q, qs), (k, ks), (v, vs)):
            dst[:, summary_rows] = (m * src + (1.0 - m) * dst[:, summary_rows]).to(dst.dtype)

    def _split_qkv(self, qkv):
        cfg = self.config
        D, Hq, Hkv = cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads
        b, L, _ = qkv.shape
        q = qkv[..., : Hq * D].view(b, L, Hq, D)
        k = qkv[..., Hq * D: (Hq + Hkv) * D].view(b, L, Hkv, D)
        v = qkv[..., (Hq + Hkv) * D:].view(b, L, Hkv, D)
        return q, k, v

    # A prefill whose gate | up activation would be larger than this runs its MLP over slices of the batch
    # (at the 4B shape a 32k prompt at batch 8 has 10.8 GB and is not sliced; at batch 64 it would be 86 GB).
    MLP_SLICE_BYTES = 16 << 30

    def _mlp(self, lw, x, defer=False):
        """`defer`: the result only goes to `_add_norm` (see `HipOps.linear`)."""
        if not defer and x.dim() == 3 and x.shape[0] > 1:
            per_seq = x.shape[1] * lw["gate_up_proj"].shape[0] * x.element_size()
            if per_seq * x.shape[0] > self.MLP_SLICE_BYTES:
                n = max(1, int(self.MLP_SLICE_BYTES // per_seq))
                out = torch.empty_like(x)
                for i in range(0, x.shape[0], n):
                    out[i:i + n] = self._mlp(lw, x[i:i + n])
                return out
        if defer and hasattr(self.ops, "mlp_rows"):
            out = self.ops.mlp_rows(x, lw["gate_up_proj"], lw["down_proj"])
            if out is not None:
                return out
        if hasattr(self.ops, "gate_up_act"):
            act = self.ops.gate_up_act(x, lw["gate_up_proj"])
        else:
            act = self.ops.silu_mul(self.ops.linear(x, lw["gate_up_proj"], defer=defer))
        return self.ops.linear(act, lw["down_proj"], defer=defer)

    def _logits(self, x_last, delta_last):
        _, h = self._add_norm(delta_last, x_last, self.w["norm"])
        return self.ops.linear(h, self.lm_head)[..., : self.config.vocab_size]

    # ---- prefill ---------------------------------------------------------------------
    @torch.no_grad()
    def prefill(self, input_ids: torch.Tensor):
        """input_ids [b, n] -> (logits [b, 1, vocab] of the last prompt token, cache)."""
        cfg, ops = self.config, self.ops
        C, S = cfg.summary_chunk_size, cfg.summary_token_num
        ids, pos, is_sum = expand_with_summary_tokens(input_ids.to(self.device), cfg)
        b, L = ids.shape
        n_sum = int(is_sum.sum().item())
        sum_rows = torch.nonzero(is_sum).flatten()
        cos, sin = self._rope_tables(pos)
        cache = ops.cache_cls(cfg, self.scns)
        x = self.w["embed_tokens"][ids]
        delta = None     # output of the previous MLP, added to the residual stream by the next norm
        Hkv, D = cfg.num_key_value_heads, cfg.head_dim
        for li, lw in enumerate(self.w["layers"]):
            x, h = self._add_norm(delta, x, lw["input_layernorm"])
            q, k, v = self._qkv(lw, h, sum_rows)
            k_slot, v_slot = cache.prefill_slots(li, b, Hkv, L, D, self.dtype, self.device, n_sum)
            q, k, v = ops.pre_attention(q, k, v, lw["q_norm"], lw["k_norm"], cos, sin, cfg.rms_norm_eps,
                                        k_out=k_slot, v_out=v_slot)
            self._blend_summary(lw, h, sum_rows, cos, sin, q, k, v)
            attn, _ = ops.summary_attn_func(q, k, v, C, S, self.scns[li], summary_pos=is_sum)
            del q, k, v, k_slot, v_slot
            if hasattr(cache, "reorganize_layer"):   # the layer's K/V in prompt order are not needed any more
                cache.reorganize_layer(li, is_sum[None])
            x, h = self._add_norm(ops.linear(attn.reshape(b, L, -1), lw["o_proj"]), x, lw["post_attention_layernorm"])
            delta = self._mlp(lw, h)
        cache.reorganize_after_prefill(is_sum[None])
        last_text = L - 1 if (L % (C + S)) != 0 else L - 1 - S   # the last prompt token's slot
        return self._logits(x[:, last_text:last_text + 1], delta[:, last_text:last_text + 1]), cache

    # ---- decode ----------------------------------------------------------------------
    def check_steps(self, cache=None):
        """Raises (`ops.timeout_error`) if a launch of the decode steps since the last check reported
        that it could not finish its work (the one-launch MLP's bounded waits); the operator set then
        uses the separate launches from there on, and the recordings of `cache` that hold the
        one-launch form are dropped.  Waits for the device.  `decode_step` and `decode_step_graph`
        call this at every chunk boundary, `generate` also at its end, and repeats the call."""
        chk = getattr(self.ops, "check_mlp_rows", None)
        if chk is None:
            return
        try:
            chk()
        except getattr(self.ops, "timeout_error", ()):
            st = getattr(cache, "_ksa_graph_state", None)
            if st is not None:
                st["graphs"].clear()
            self._graph_warm = set()   # the other path's launches get their eager run before a recording
            raise

    @torch.no_grad()
    def decode_step(self, token_ids: torch.Tensor, cache):
        """token_ids [b, 1] (the newest text token) -> logits [b, 1, vocab].  When the token
        completes a chunk the step also runs the chunk's summary tokens and stores their K/V."""
        cfg, ops = self.config, self.ops
        C, S = cfg.summary_chunk_size, cfg.summary_token_num
        Hkv, D = cfg.num_key_value_heads, cfg.head_dim
        b = token_ids.shape[0]
        true_tokens = cache.get_true_token_num()
        boundary = cache.get_cur_chunk_size() == C - 1
        if boundary:
            self.check_steps(cache)   # before the step that cannot be undone (it flushes the chunk)
        ids = token_ids.to(self.device)
        if boundary:
            sids = torch.arange(S, device=self.device, dtype=ids.dtype) + cfg.summary_token_begin
            ids = torch.cat([ids, sids[None].expand(b, -1)], dim=1)
            pos = boundary_position_ids(true_tokens, cfg, self.device)
            sum_rows = torch.arange(1, 1 + S, device=self.device)
        else:
            p = true_tokens if cfg.summary_chunk_position_ids_type == "origin" else cache.get_cur_chunk_size()
            pos = torch.tensor([[p]], dtype=torch.long, device=self.device)
            sum_rows = None
        cos, sin = self._rope_tables(pos)
        x = self.w["embed_tokens"][ids]
        delta = None
        tables = {}   # boundary step: (text row, first summary row) -> row table on the device
        for li, lw in enumerate(self.w["layers"]):
            x, h = self._add_norm(delta, x, lw["input_layernorm"])
            if not boundary:
                k_slot, v_slot = cache.text_slots(li, b, Hkv, D, self.dtype, self.device)
                qkv = ops.linear(h, lw["qkv_proj"], defer=True)
                if torch.is_tensor(qkv):
                    q, k, v = self._split_qkv(qkv)
                    q, _, _ = ops.pre_attention(q, k, v, lw["q_norm"], lw["k_norm"], cos, sin, cfg.rms_norm_eps,
                                                k_out=k_slot, v_out=v_slot)
                else:  # still the K-split partial sums of the projection: added inside the kernel
                    q, _, _ = ops.pre_attention_partials(qkv, cfg.num_attention_heads, Hkv, D, lw["q_norm"],
                                                         lw["k_norm"], cos, sin, cfg.rms_norm_eps,
                                                         k_out=k_slot, v_out=v_slot)
                a, e = cache.attention_range(li)
                attn = ops.decode(q.transpose(1, 2), cache.key_cache[li], cache.value_cache[li], a, e,
                                  self.scaling)
            else:
                fused = hasattr(ops, "decode_boundary") and cache.boundary_fits_one_piece(li)
                if fused:
                    # fused operators: the cache only does the bookkeeping and names the rows
                    sl = cache.boundary_slots(li, S)
                    rows = dict(text=sl["text"], start=sl["attend"][0], end=sl["attend"][1])
                    if cache.is_large_window[li]:
                        rows.update(spare=sl["spare"], sum_start=sl["spare"] - C, sum_end=sl["spare"] + S)
                    else:
                        rows.update(flush_src=sl["flush_src"], flush_dst=sl["flush_dst"],
                                    flush_rows=sl["flush_rows"], append=sl["append"])
                slots = None
                if fused and self._boundary_rows_in_cache():
                    key = (rows["text"], rows["spare"] if cache.is_large_window[li] else 0)
                    if key not in tables:  # the same for every layer of a kind: two small copies per step
                        tables[key] = self._boundary_row_table(key[0], key[1], b)
                    slots = (cache.key_cache[li], cache.value_cache[li], tables[key])
                q, k, v = self._boundary_qkv(lw, h, sum_rows, cos, sin, slots)
                qh = q.transpose(1, 2)
                kh, vh = (None, None) if k is None else (k.transpose(1, 2), v.transpose(1, 2))
                if fused:
                    attn = self._boundary_attention(qh, kh, vh, cache.key_cache[li], cache.value_cache[li],
                                                    cache.is_large_window[li], rows)
                else:   # the reference's own sequence of cache calls
                    cache.update_text(kh[:, :, :1], vh[:, :, :1], li)
                    a, e = cache.attention_range(li)
                    text_out = ops.decode(qh[:, :, :1], cache.key_cache[li], cache.value_cache[li], a, e,
                                          self.scaling)
                    k_cs, v_cs = cache.get_summary_attention_kv(li, kh[:, :, 1:], vh[:, :, 1:])
                    sum_out = ops.decode(qh[:, :, 1:], k_cs, v_cs, 0, k_cs.shape[2], self.scaling)
                    cache.update_summary(kh[:, :, 1:], vh[:, :, 1:], li)
                    attn = torch.cat([text_out, sum_out], dim=1)
            if boundary:
                x, h = self._add_norm(ops.linear(attn.reshape(b, ids.shape[1], -1), lw["o_proj"], defer=True), x,
                                      lw["post_attention_layernorm"])
                delta = self._mlp(lw, h, defer=True)
            else:
                x, delta = self._post_attention(lw, attn.reshape(b, ids.shape[1], -1), x)
        cache.reset_chunk_counter()
        if not boundary:
            return self._logits(x, delta)
        return self._boundary_logits(x, delta)

    # ---- decode through a HIP graph ----------------------------------------------------
    def _text_step_body(self, st, cache):
        """One non-boundary decode step in a form that can be recorded once and replayed: every
        per-step quantity (token ids, position, the cache row the new K/V go to, the attended row
        range) is read from device tensors of `st`, never baked into a launch."""
        cfg, ops = self.config, self.ops
        rope = st["rope_tab"].index_select(0, st["rope_rel"])   # [1, 2, D]: this step's cos and sin rows
        cos, sin = rope[:, 0][None], rope[:, 1][None]
        x = self.w["embed_tokens"][st["tok"]]
        b = x.shape[0]
        delta = None
        for li, lw in enumerate(self.w["layers"]):
            kind = 1 if cache.is_large_window[li] else 0
            x, h = self._add_norm(delta, x, lw["input_layernorm"])
            # k and v go straight to the cache row the device-side cursor names
            slots = dict(k_out=cache.key_cache[li][:, :, :1].transpose(1, 2),
                         v_out=cache.value_cache[li][:, :, :1].transpose(1, 2), kv_out_row=st["cur"][kind, 0])
            qkv = ops.linear(h, lw["qkv_proj"], defer=True)
            if torch.is_tensor(qkv):
                q, k, v = self._split_qkv(qkv)
                q, _, _ = ops.pre_attention(q, k, v, lw["q_norm"], lw["k_norm"], cos, sin, cfg.rms_norm_eps, **slots)
            else:  # still the K-split partial sums of the projection: added inside the kernel
                q, _, _ = ops.pre_attention_partials(qkv, cfg.num_attention_heads, cfg.num_key_value_heads,
                                                     cfg.head_dim, lw["q_norm"], lw["k_norm"], cos, sin,
                                                     cfg.rms_norm_eps, **slots)
            attn = ops.decode(q.transpose(1, 2), cache.key_cache[li], cache.value_cache[li],
                              st["cur"][kind, 1], st["cur"][kind, 2], self.scaling)
            x, delta = self._post_attention(lw, attn.reshape(b, 1, -1), x)
        return self._logits(x, delta)

    def _boundary_step_body(self, st, cache):
        """One chunk-boundary decode step in the recordable form of `_text_step_body`: the text
        token and the chunk's S summary tokens run together, and every row that `decode_step` takes
        from the cache's counters (where the text row goes, the text query's range, where the chunk
        is flushed to in the ring, where the new summaries are appended) is read from `st["bcur"]`:

            [0: small window][text row, range start, range end, flush destination, append row, -]
            [1: large window][text row, range start, range end, first spare row behind the text,
                              start and end of [chunk text | spare rows]]

        In a large-window layer the summary rows' K/V sit in spare rows behind the text for the
        length of the step (the next text token overwrites them), which gives the summary queries
        the [chunk | own summaries] rows of `get_summary_attention_kv` as one row range."""
        cfg, ops = self.config, self.ops
        C, S = cfg.summary_chunk_size, cfg.summary_token_num
        ids, bc = st["btok"], st["bcur"]
        b = ids.shape[0]
        sum_rows = st["bsum_rows"]
        cos, sin = self._rope_tables(st["bpos"])
        x = self.w["embed_tokens"][ids]
        delta = None
        tables = None
        if self._boundary_rows_in_cache():  # where the step's K/V rows go: small window, large window
            tables = (self._boundary_row_table(bc[0, 0], 0, b), self._boundary_row_table(bc[1, 0], bc[1, 3], b))
        for li, lw in enumerate(self.w["layers"]):
            kind = 1 if cache.is_large_window[li] else 0
            kc, vc, mv = cache.key_cache[li], cache.value_cache[li], cache._move_rows
            x, h = self._add_norm(delta, x, lw["input_layernorm"])
            q, k, v = self._boundary_qkv(lw, h, sum_rows, cos, sin, None if tables is None else (kc, vc, tables[kind]))
            qh = q.transpose(1, 2)
            kh, vh = (None, None) if k is None else (k.transpose(1, 2), v.transpose(1, 2))
            if hasattr(ops, "decode_boundary"):
                rows = dict(text=bc[kind, 0], start=bc[kind, 1], end=bc[kind, 2])
                if kind:
                    rows.update(spare=bc[1, 3], sum_start=bc[1, 4], sum_end=bc[1, 5])
                else:
                    rows.update(flush_src=S, flush_rows=C, flush_dst=bc[0, 3], append=bc[0, 4])
                attn = self._boundary_attention(qh, kh, vh, kc, vc, bool(kind), rows)
            else:
                mv(kh[:, :, :1], kc, 1, dst_start_seq=bc[kind, 0])
                mv(vh[:, :, :1], vc, 1, dst_start_seq=bc[kind, 0])
                text_out = ops.decode(qh[:, :, :1], kc, vc, bc[kind, 1], bc[kind, 2], self.scaling)
                if kind == 0:
                    mv(kh[:, :, 1:], kc, S, 0, 0)
                    mv(vh[:, :, 1:], vc, S, 0, 0)
                    sum_out = ops.decode(qh[:, :, 1:], kc[:, :, :S + C], vc[:, :, :S + C], 0, S + C, self.scaling)
                    for buf, new in ((kc, kh), (vc, vh)):
                        mv(buf, buf, C, S, dst_start_seq=bc[0, 3])            # chunk rows -> ring
                        mv(new[:, :, 1:], buf, S, dst_start_seq=bc[0, 4])     # the chunk's summaries
                else:
                    mv(kh[:, :, 1:], kc, S, dst_start_seq=bc[1, 3])
                    mv(vh[:, :, 1:], vc, S, dst_start_seq=bc[1, 3])
                    sum_out = ops.decode(qh[:, :, 1:], kc, vc, bc[1, 4], bc[1, 5], self.scaling)
                attn = torch.cat([text_out, sum_out], dim=1)
            x, h = self._add_norm(ops.linear(attn.reshape(b, 1 + S, -1), lw["o_proj"], defer=True), x,
                                  lw["post_attention_layernorm"])
            delta = self._mlp(lw, h, defer=True)
        return self._boundary_logits(x, delta)

    def _stage_ints(self, st, key, vals):
        """Host integers `vals` (a flat list) -> the int32 device tensor st[key], through a ring of
        pinned host slots: a copy from pageable memory would hold the host until the GPU has reached
        it, i.e. until the previous step has ended, and the GPU would then idle while the host
        prepares the next replay.  A slot is written again only after the copy that read it has run
        (its event), so the host may be up to a ring's length of steps ahead of the GPU."""
        ring = st["rings"].get(key)
        if ring is None:
            ring = st["rings"][key] = {"slots": torch.empty(16, len(vals), dtype=torch.int32, pin_memory=True),
                                       "events": [None] * 16, "next": 0}
        slot = ring["next"]
        ring["next"] = (slot + 1) % 16
        if ring["events"][slot] is not None:
            ring["events"][slot].synchronize()
        ring["slots"][slot].copy_(torch.tensor(vals, dtype=torch.int32))
        st[key].view(-1).copy_(ring["slots"][slot], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(self.device))
        ring["events"][slot] = ev

    def _warm_up(self, st, which, body, cache):
        """Runs `body` once, launched eagerly on a side stream, the first time a recording of this
        kind is needed for a batch size, so that everything that happens lazily (kernel modules,
        GEMM handles, workspaces) happens outside the capture.  Returns whether it ran."""
        warm = getattr(self, "_graph_warm", None)
        if warm is None:
            warm = self._graph_warm = set()
        if (which, st["batch"]) in warm:
            return False
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            body(st, cache)
        torch.cuda.current_stream(self.device).wait_stream(side)
        warm.add((which, st["batch"]))
        return True

    def _replay(self, st, which, body, cache):
        """Replays the recording `which` of `body`, recording it first when there is none for the
        cache buffers as they are now (the launches bake in addresses, strides and capacity)."""
        ptrs = tuple((t.data_ptr(), tuple(t.shape), t.stride()) for t in cache.key_cache + cache.value_cache)
        rec = st["graphs"].get(which)
        if rec is None or rec["ptrs"] != ptrs:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                logits = body(st, cache)
            rec = st["graphs"][which] = {"graph": g, "ptrs": ptrs, "logits": logits}
        rec["graph"].replay()
        return rec["logits"]

    @torch.no_grad()
    def decode_step_graph(self, token_ids: torch.Tensor, cache):
        """`decode_step` with the launches of a step replayed from a HIP graph (about 400 launches
        per step otherwise cost more host time than GPU time): one recording for the steps inside a
        chunk, one for the chunk-boundary steps.  The recordings belong to the cache object they
        were made for (they are kept on it) and are made again when a cache buffer was reallocated
        or changed its shape.  The returned logits live in a buffer that a later call overwrites."""
        cfg = self.config
        C, S = cfg.summary_chunk_size, cfg.summary_token_num
        b = token_ids.shape[0]
        Hkv, D = cfg.num_key_value_heads, cfg.head_dim
        nl = cfg.num_hidden_layers
        st = getattr(cache, "_ksa_graph_state", None)
        if st is None or st["batch"] != b or st["owner"] is not self:
            sids = torch.arange(S, device=self.device, dtype=torch.long) + cfg.summary_token_begin
            st = {"batch": b, "owner": self, "graphs": {}, "rings": {},
                  "tok": torch.zeros(b, 1, dtype=torch.long, device=self.device),
                  # [kind: small / large window][destination row, range start, range end][sequence]
                  "cur": torch.zeros(2, 3, b, dtype=torch.int32, device=self.device),
                  # the same for a boundary step (see `_boundary_step_body`), its ids and positions
                  "bcur": torch.zeros(2, 6, b, dtype=torch.int32, device=self.device),
                  "btok": torch.cat([torch.zeros(b, 1, dtype=torch.long, device=self.device),
                                     sids[None].expand(b, -1)], dim=1).contiguous(),
                  "bpos": torch.zeros(1, 1 + S, dtype=torch.int32, device=self.device),
                  "bsum_rows": torch.arange(1, 1 + S, device=self.device)}
            cache._ksa_graph_state = st
        kinds = [1 if cache.is_large_window[li] else 0 for li in range(nl)]
        if cache.get_cur_chunk_size() == C - 1:
            self.check_steps(cache)
            # recorded: a boundary step whose flush is one whole chunk in one piece (every boundary of
            # a cache filled by `prefill`), once the cache has seen enough of them; else eagerly
            st["boundaries"] = st.get("boundaries", 0) + 1
            if st["boundaries"] <= self.BOUNDARY_GRAPH_AFTER or not all(
                    cache.boundary_fits_one_piece(li) and (kinds[li] or cache._chunk_buf_len[li] == C - 1)
                    for li in range(nl)):
                return self.decode_step(token_ids, cache)
            pos = boundary_position_ids(cache.get_true_token_num(), cfg, "cpu")[0].tolist()
            vals = [[0, 0, 1, 0, 0, 0], [0, 0, 1, 0, 0, 1]]
            seen = [None, None]
            for li in range(nl):
                sl = cache.boundary_slots(li, S)
                a, e = sl["attend"]
                if kinds[li]:
                    row = [sl["text"], a, e, sl["spare"], sl["spare"] - C, sl["spare"] + S]
                else:
                    assert sl["flush_src"] == S and sl["flush_rows"] == C
                    row = [sl["text"], a, e, sl["flush_dst"], sl["append"], 0]
                assert seen[kinds[li]] in (None, row), "layers of one kind must move in step"
                seen[kinds[li]] = vals[kinds[li]] = row
            self._stage_ints(st, "bpos", pos)
            st["btok"][:, :1].copy_(token_ids.to(self.device))
            # A boundary step is not idempotent (its flush overwrites ring rows that its text query
            # still attends), so the warm-up run flushes the chunk onto itself and appends the
            # summaries onto the scratch rows that already hold them.
            if ("boundary", b) not in getattr(self, "_graph_warm", ()):
                harmless = [vals[0][:3] + [S, 0, 0], vals[1]]
                self._stage_ints(st, "bcur", [v for kind in harmless for x in kind for v in [x] * b])
                self._warm_up(st, "boundary", self._boundary_step_body, cache)
            self._stage_ints(st, "bcur", [v for kind in vals for x in kind for v in [x] * b])
            logits = self._replay(st, "boundary", self._boundary_step_body, cache)
            cache.reset_chunk_counter()
            return logits
        p = cache.get_true_token_num() if cfg.summary_chunk_position_ids_type == "origin" \
            else cache.get_cur_chunk_size()
        # host bookkeeping of the step (may enlarge an append-only buffer), then this step's rows
        rows = [None, None]
        for li in range(nl):
            if rows[kinds[li]] is None:
                rows[kinds[li]] = cache._text_len[li] if kinds[li] else S + C - 1 - cache._chunk_buf_len[li]
            cache.text_slots(li, b, Hkv, D, self.dtype, self.device)
        vals = [[0, 0, 1], [0, 0, 1]]
        for li in range(nl):
            if rows[kinds[li]] is not None:
                a, e = cache.attention_range(li)
                vals[kinds[li]] = [rows[kinds[li]], a, e]
                rows[kinds[li]] = None
        self._stage_ints(st, "cur", [v for kind in vals for x in kind for v in [x] * b])
        st["tok"].copy_(token_ids.to(self.device))
        # rotary rows of a window of positions, made with the prefill's own tensor ops (so a step's
        # cos / sin are the values `_rope_tables` gives) and refilled in place when p leaves it; the
        # recorded step only picks a row
        if st.get("rope_p0") is None or not (st["rope_p0"] <= p < st["rope_p0"] + st["rope_tab"].shape[0]):
            n = 1024
            c, s_ = self._rope_tables(torch.arange(p, p + n, device=self.device)[None])
            tab = torch.stack((c[0], s_[0]), dim=1)
            if "rope_tab" in st:
                st["rope_tab"].copy_(tab)
            else:
                st["rope_tab"] = tab.contiguous()
                st["rope_rel"] = torch.zeros(1, dtype=torch.long, device=self.device)
            st["rope_p0"] = p
        st["rope_rel"].fill_(p - st["rope_p0"])
        self._warm_up(st, "text", self._text_step_body, cache)   # a step inside a chunk is idempotent
        logits = self._replay(st, "text", self._text_step_body, cache)
        cache.reset_chunk_counter()
        return logits

    # ---- driver ----------------------------------------------------------------------
    def forward(self, input_ids: torch.Tensor, cache=None):
        """Prefill when there is no (or an empty) cache, one decode step otherwise."""
        if cache is None or cache.get_seq_length() == 0:
            return self.prefill(input_ids)
        return self.decode_step(input_ids[:, -1:], cache), cache

    @torch.no_grad()
    def generate(self, input_ids: torch.Tensor, max_new_tokens: int, forced: Optional[torch.Tensor] = None,
                 return_logits: bool = False, use_graph: bool = False):
        """Greedy decoding.  Returns ids [b, n + max_new_tokens] (and the logits of every step,
        [b, max_new_tokens, vocab], on request).  `forced` [b, max_new_tokens] replaces the
        arg-max token fed back at every step (teacher forcing, for comparing two runs).
        `use_graph` replays the decode steps from HIP graphs (`decode_step_graph`).
        If a launch reports that it could not finish (`check_steps`), the whole call is repeated
        once on the separate-launch path, which `check_steps` has switched to."""
        try:
            return self._generate(input_ids, max_new_tokens, forced, return_logits, use_graph)
        except getattr(self.ops, "timeout_error", ()):
            return self._generate(input_ids, max_new_tokens, forced, return_logits, use_graph)

    def _generate(self, input_ids, max_new_tokens, forced, return_logits, use_graph):
        logits, cache = self.prefill(input_ids)
        out, steps = [], []
        for t in range(max_new_tokens):
            if return_logits:
                steps.append(logits[:, 0].float())
            last = logits[:, 0]
            nxt = (self.ops.argmax(last) if hasattr(self.ops, "argmax") else last.argmax(-1))[:, None]
            out.append(nxt)
            if t + 1 < max_new_tokens:
                feed = nxt if forced is None else forced[:, t:t + 1].to(self.device)
                logits = self.decode_step_graph(feed, cache) if use_graph else self.decode_step(feed, cache)
        ids = torch.cat([input_ids.to(self.device)] + out, dim=1)
        self.check_steps(cache)
        return (ids, torch.stack(steps, dim=1)) if return_logits else ids
