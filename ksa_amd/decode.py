"""Decode attention over the contiguous ring-buffer KV slice on MI355X.

`decode_attention_forward` has the signature of the reference's `_decode_attn_fn`
(examples/pretrain/hf_template/modeling_qwen3sa.py:591-612 `_sdpa_attention_forward`,
selected at :643-646 and called at :820-830, :844-870): un-masked, non-causal
soft-max attention of `query [b, Hq, q_len, D]` over `key/value [b, Hkv, L, D]`
(strided views of the cache), GQA by `module.num_key_value_groups`, returning
`(attn_output [b, q_len, Hq, D], None)`.  `ksa_decode` is the lower-level form that
takes the whole cache tensor and per-sequence row ranges, which the reference cannot
express (its cache counters are shared by the batch, :753-754).
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib

_DTYPES = {torch.bfloat16: 0, torch.float16: 1}


@torch.library.custom_op("ksa_amd::decode_fwd", mutates_args=())
def _decode_fwd(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                start: Optional[torch.Tensor], end: Optional[torch.Tensor], start0: int, end0: int,
                scale: float, nsplit: int) -> torch.Tensor:
    b, Hq, Q, D = q.shape
    Hkv = kcache.shape[1]
    lib = _lib.lib()
    out = torch.empty((b, Q, Hq, D), dtype=q.dtype, device=q.device)
    ws = None
    ws_bytes = 0
    if nsplit > 1:
        ws_bytes = lib.ksa_decode_workspace_bytes(b, Hq, Hkv, Q, D, nsplit)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        rc = lib.ksa_decode_fwd(
            q.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), out.data_ptr(),
            start.data_ptr() if start is not None else None,
            end.data_ptr() if end is not None else None, start0, end0,
            b, Hq, Hkv, Q, D, _DTYPES[q.dtype],
            _lib.strides3(q, (0, 1, 2)), _lib.strides3(kcache, (0, 1, 2)),
            _lib.strides3(vcache, (0, 1, 2)), _lib.strides3(out, (0, 1, 2)),
            float(scale), nsplit, ws.data_ptr() if ws is not None else None, ws_bytes,
            _lib.stream_ptr(q.device))
    _lib.check(rc, "ksa_decode_fwd")
    return out


@_decode_fwd.register_fake
def _(q, kcache, vcache, start, end, start0, end0, scale, nsplit):
    b, Hq, Q, D = q.shape
    return q.new_empty((b, Q, Hq, D))


def ksa_decode(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
               start=None, end=None, scale: Optional[float] = None,
               nsplit: Optional[int] = None) -> torch.Tensor:
    """q [b, Hq, Q, D]; kcache/vcache [b, Hkv, rows, D] (any batch/head/row strides);
    rows [start, end) are attended: ints for every sequence, or int32 device tensors [b]
    per sequence; default is the whole row axis.  Returns [b, Q, Hq, D]."""
    assert q.is_cuda and kcache.is_cuda and vcache.is_cuda, "inputs must be on a GPU"
    assert q.dtype in _DTYPES and q.dtype == kcache.dtype == vcache.dtype, "inputs must share a 16-bit float dtype"
    assert q.dim() == 4 and kcache.dim() == 4 and kcache.shape == vcache.shape
    b, Hq, Q, D = q.shape
    assert kcache.shape[0] == b and kcache.shape[3] == D and Hq % kcache.shape[1] == 0
    if q.stride(-1) != 1:
        q = q.contiguous()
    assert kcache.stride(-1) == 1 and vcache.stride(-1) == 1, "cache rows must be contiguous"
    rows = kcache.shape[2]
    t_start = t_end = None
    s0, e0 = 0, rows
    if isinstance(start, torch.Tensor) or isinstance(end, torch.Tensor):
        t_start = torch.as_tensor(start if start is not None else 0, device=q.device).to(torch.int32).expand(b).contiguous()
        t_end = torch.as_tensor(end if end is not None else rows, device=q.device).to(torch.int32).expand(b).contiguous()
        max_rows = rows
    else:
        s0 = 0 if start is None else int(start)
        e0 = rows if end is None else int(end)
        assert 0 <= s0 < e0 <= rows, "row range out of bounds"
        max_rows = e0 - s0
    if scale is None:
        scale = float(D) ** -0.5
    if nsplit is None:
        nsplit = _lib.lib().ksa_decode_auto_splits(b, kcache.shape[1], max_rows)
    from .prefill import kernel_head_dim, pad_head_dim
    Dk = kernel_head_dim(D)
    if Dk != D:
        # A head dimension without a kernel of its own (the kernels are built for 64 / 128 / 256): the
        # attended rows are copied into zero-padded buffers for this call.  Correct, but it moves the
        # rows twice; a cache that stores its rows at a kernel size avoids it.
        assert D % 8 == 0, "head dimension must be a multiple of 8"
        if t_start is not None:
            lo, hi = int(t_start.min().item()), int(t_end.max().item())
            t_start, t_end = t_start - lo, t_end - lo
        else:
            lo, hi, s0, e0 = s0, e0, 0, e0 - s0
        kcache, vcache = pad_head_dim(kcache[:, :, lo:hi], Dk), pad_head_dim(vcache[:, :, lo:hi], Dk)
        out = torch.ops.ksa_amd.decode_fwd(pad_head_dim(q, Dk), kcache, vcache, t_start, t_end, s0, e0,
                                           float(scale), int(nsplit))
        return out[..., :D].contiguous()
    return torch.ops.ksa_amd.decode_fwd(q, kcache, vcache, t_start, t_end, s0, e0, float(scale), int(nsplit))


def ksa_decode_boundary(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, text_start, text_end,
                        sum_start, sum_end, scale: Optional[float] = None,
                        nsplit: Optional[int] = None) -> torch.Tensor:
    """The attention of a chunk-boundary step in one launch (modeling_qwen3sa.py:831-876: two calls of
    the decode attention function and a `torch.cat`): q [b, Hq, 1 + S, D]; query token 0 attends the
    cache rows [text_start, text_end), the S summary tokens attend [sum_start, sum_end); each bound
    an int or an int32 GPU tensor [b].  Returns [b, 1 + S, Hq, D]."""
    assert q.is_cuda and q.dtype in _DTYPES and q.dtype == kcache.dtype == vcache.dtype
    b, Hq, Q, D = q.shape
    Hkv, rows = kcache.shape[1], kcache.shape[2]
    assert Q >= 2 and kcache.shape == vcache.shape and kcache.shape[0] == b and kcache.shape[3] == D and Hq % Hkv == 0
    assert D in (64, 128, 256), "the boundary form has no padded path: head_dim 64, 128 or 256"
    if q.stride(-1) != 1:
        q = q.contiguous()
    assert kcache.stride(-1) == 1 and vcache.stride(-1) == 1, "cache rows must be contiguous"

    def pair(lo, hi):
        if torch.is_tensor(lo) or torch.is_tensor(hi):
            tl = torch.as_tensor(lo, device=q.device).to(torch.int32).expand(b).contiguous()
            th = torch.as_tensor(hi, device=q.device).to(torch.int32).expand(b).contiguous()
            return tl, th, 0, 1
        assert 0 <= int(lo) < int(hi) <= rows, "row range out of bounds"
        return None, None, int(lo), int(hi)
    ts, te, ts0, te0 = pair(text_start, text_end)
    ss, se, ss0, se0 = pair(sum_start, sum_end)
    if scale is None:
        scale = float(D) ** -0.5
    lib = _lib.lib()
    if nsplit is None:
        nsplit = lib.ksa_decode_auto_splits(b, Hkv, rows if ts is not None else te0 - ts0)
    out = torch.empty((b, Q, Hq, D), dtype=q.dtype, device=q.device)
    ws, ws_bytes = None, 0
    if nsplit > 1:
        ws_bytes = lib.ksa_decode_boundary_workspace_bytes(b, Hq, Hkv, Q, D, nsplit)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    ptr = lambda t: t.data_ptr() if t is not None else None
    with torch.cuda.device(q.device):
        rc = lib.ksa_decode_boundary_fwd(
            q.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), out.data_ptr(), ptr(ts), ptr(te), ts0, te0,
            ptr(ss), ptr(se), ss0, se0, b, Hq, Hkv, Q, D, _DTYPES[q.dtype], _lib.strides3(q, (0, 1, 2)),
            _lib.strides3(kcache, (0, 1, 2)), _lib.strides3(vcache, (0, 1, 2)), _lib.strides3(out, (0, 1, 2)),
            float(scale), int(nsplit), ptr(ws), ws_bytes, _lib.stream_ptr(q.device))
    _lib.check(rc, "ksa_decode_boundary_fwd")
    return out


def ksa_decode_weights(q: torch.Tensor, kcache: torch.Tensor, start=None, end=None,
                       scale: Optional[float] = None, mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The attention probabilities of `ksa_decode`: softmax(q K^T * scale (+ mask)) over the rows
    [start, end) of every sequence, computed in fp32 and rounded to q's dtype, [b, Hq, Q, L] with
    L = the longest range; positions past a shorter sequence's range hold 0.  `mask`, if given, is
    additive, of q's dtype and broadcastable to [b, Hq, Q, L] (the `attention_mask` of the
    reference's eager_attention_forward, modeling_qwen3sa.py:569-588)."""
    assert q.is_cuda and kcache.is_cuda and q.dtype in _DTYPES and q.dtype == kcache.dtype
    assert q.dim() == 4 and kcache.dim() == 4
    b, Hq, Q, D = q.shape
    Hkv, rows = kcache.shape[1], kcache.shape[2]
    assert kcache.shape[0] == b and kcache.shape[3] == D and Hq % Hkv == 0
    if q.stride(-1) != 1:
        q = q.contiguous()
    assert kcache.stride(-1) == 1, "cache rows must be contiguous"
    t_start = t_end = None
    s0, e0 = 0, rows
    if isinstance(start, torch.Tensor) or isinstance(end, torch.Tensor):
        t_start = torch.as_tensor(start if start is not None else 0, device=q.device).to(torch.int32).expand(b).contiguous()
        t_end = torch.as_tensor(end if end is not None else rows, device=q.device).to(torch.int32).expand(b).contiguous()
        L = int((t_end - t_start).max().item())
    else:
        s0 = 0 if start is None else int(start)
        e0 = rows if end is None else int(end)
        assert 0 <= s0 < e0 <= rows, "row range out of bounds"
        L = e0 - s0
    assert L > 0
    from .prefill import kernel_head_dim, pad_head_dim
    Dk = kernel_head_dim(D)
    if scale is None:
        scale = float(D) ** -0.5
    if Dk != D:   # zero-padded copies of the attended rows, as in `ksa_decode`
        assert D % 8 == 0, "head dimension must be a multiple of 8"
        if t_start is not None:
            lo, hi = int(t_start.min().item()), int(t_end.max().item())
            t_start, t_end = t_start - lo, t_end - lo
        else:
            lo, hi, s0, e0 = s0, e0, 0, e0 - s0
        q, kcache = pad_head_dim(q, Dk), pad_head_dim(kcache[:, :, lo:hi], Dk)
    m_strides = None
    if mask is not None:
        assert mask.dtype == q.dtype and mask.is_cuda
        mask = mask.expand(b, Hq, Q, L)
        m_strides = (ctypes.c_int64 * 4)(*mask.stride())
    lib = _lib.lib()
    out = torch.empty((b, Hq, Q, L), dtype=q.dtype, device=q.device)
    ws_bytes = lib.ksa_decode_weights_workspace_bytes(b, Hq, Q, L)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        rc = lib.ksa_decode_weights(
            q.data_ptr(), kcache.data_ptr(), out.data_ptr(), mask.data_ptr() if mask is not None else None,
            t_start.data_ptr() if t_start is not None else None, t_end.data_ptr() if t_end is not None else None,
            s0, e0, b, Hq, Hkv, Q, Dk, _DTYPES[q.dtype], L, _lib.strides3(q, (0, 1, 2)),
            _lib.strides3(kcache, (0, 1, 2)), m_strides, float(scale), ws.data_ptr(), ws_bytes,
            _lib.stream_ptr(q.device))
    _lib.check(rc, "ksa_decode_weights")
    return out


def eager_attention_forward(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                            attention_mask: Optional[torch.Tensor] = None, scaling: Optional[float] = None,
                            dropout: float = 0.0, **kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
    """Drop-in for the reference's `eager_attention_forward` (modeling_qwen3sa.py:569-588), the decode
    attention function it selects when `config._attn_implementation == "eager"` (:643-646): returns
    `(attn_output [b, q_len, Hq, D], attn_weights [b, Hq, q_len, L])`.  The output comes from the
    decode kernel, the probabilities from `ksa_decode_weights` (a second pass over K).  The cache
    call sites pass no mask (:820-870); one is refused here, because the output kernel has no masked
    form."""
    if dropout:
        raise NotImplementedError("decode attention is inference-only (dropout must be 0)")
    if attention_mask is not None:
        raise NotImplementedError("the decode kernels take no attention mask (the reference's cache call sites pass None)")
    g = query.shape[1] // key.shape[1]
    assert getattr(module, "num_key_value_groups", g) == g, "module.num_key_value_groups does not match the tensor shapes"
    return ksa_decode(query, key, value, scale=scaling), ksa_decode_weights(query, key, scale=scaling)


def decode_attention_forward(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                             attention_mask: Optional[torch.Tensor] = None,
                             scaling: Optional[float] = None, dropout: float = 0.0,
                             **kwargs) -> Tuple[torch.Tensor, None]:
    """Drop-in for `Qwen3Attention._decode_attn_fn`.  `attention_mask` is ignored exactly
    as the reference's SDPA variant ignores it (it passes attn_mask=None); dropout must be 0."""
    if dropout:
        raise NotImplementedError("decode attention is inference-only (dropout must be 0)")
    g = query.shape[1] // key.shape[1]
    mg = getattr(module, "num_key_value_groups", g)
    assert mg == g, "module.num_key_value_groups does not match the tensor shapes"
    return ksa_decode(query, key, value, scale=scaling), None
