"""Pre-attention step of a Qwen3 / KSA attention layer as one HIP kernel.

Mirrors what `Qwen3Attention.forward` does between the projections and the attention call
(examples/pretrain/hf_template/modeling_qwen3sa.py:660-666: q_norm / k_norm on head_dim,
apply_rotary_pos_emb in the rotate_half form :523-554) and writes q, k, v directly in the
layout the attention kernels or the KV cache want, so the `.transpose(1, 2).contiguous()`
copies of the reference disappear.  There is no fallback: without libksa_hip.so it raises.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib

_DT = {torch.bfloat16: 0, torch.float16: 1}


def _bsh(t):  # element strides of a [batch, rows, heads, D] view
    return _lib.strides3(t, (0, 1, 2))


def pre_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_norm_weight: torch.Tensor,
                  k_norm_weight: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, eps: float = 1e-6,
                  q_out: Optional[torch.Tensor] = None, k_out: Optional[torch.Tensor] = None,
                  v_out: Optional[torch.Tensor] = None,
                  kv_out_row: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """q [b, S, Hq, D], k, v [b, S, Hkv, D] (views of the projection outputs, head_dim contiguous);
    cos, sin [b or 1, S, D] as returned by the rotary embedding module, in the dtype of q.

    Returns (q', k', v) with q' = rope(q_norm(q)), k' = rope(k_norm(k)) in [b, S, H, D].  `*_out`
    may be given as [b, S, H, D]-shaped views with arbitrary batch/row/head strides, e.g.
    `cache_k[:, :, start:start + S].transpose(1, 2)` to write the keys straight into a
    [b, Hkv, capacity, D] cache tensor; they may alias the inputs.  `kv_out_row` (int32 [b] on
    the GPU) moves sequence b's k and v `kv_out_row[b]` rows further down their outputs: the
    cache cursor when only the device knows it (a recorded step that is replayed).  As int32
    [b, S] it names the output row of every token's k and v outright (k_out / v_out then only give
    the base address and the strides: pass the view that starts at row 0).
    """
    assert q.dtype in _DT and k.dtype == q.dtype and v.dtype == q.dtype, "q, k, v must share bf16 or fp16"
    assert q.is_cuda and k.is_cuda and v.is_cuda, "inputs must be on a GPU"
    b, S, Hq, D = q.shape
    Hkv = k.shape[2]
    assert k.shape == (b, S, Hkv, D) and v.shape == (b, S, Hkv, D), "k, v must be [b, S, Hkv, D]"
    assert q.stride(3) == 1 and k.stride(3) == 1 and v.stride(3) == 1, "head_dim must be contiguous"
    if cos.dim() == 2:
        cos, sin = cos[None], sin[None]
    assert cos.shape[-2:] == (S, D) and sin.shape == cos.shape and cos.shape[0] in (1, b)
    cos = cos.to(q.dtype).contiguous()
    sin = sin.to(q.dtype).contiguous()
    qw = q_norm_weight.to(q.dtype).contiguous()
    kw = k_norm_weight.to(q.dtype).contiguous()
    assert qw.shape == (D,) and kw.shape == (D,)
    outs = []
    for given, like in ((q_out, q), (k_out, k), (v_out, v)):
        if given is None:
            given = torch.empty(like.shape, dtype=like.dtype, device=like.device)
        assert given.shape == like.shape and given.dtype == like.dtype and given.stride(3) == 1
        outs.append(given)
    qo, ko, vo = outs
    if kv_out_row is not None:
        assert kv_out_row.is_cuda and kv_out_row.dtype == torch.int32 and tuple(kv_out_row.shape) in ((b,), (b, S)) \
            and kv_out_row.is_contiguous(), "kv_out_row must be a contiguous int32 [b] or [b, S] GPU tensor"
        assert k_out is not None and v_out is not None, "kv_out_row needs k_out and v_out"
    per_token = int(kv_out_row is not None and kv_out_row.dim() == 2)
    cstr = (ctypes.c_int64 * 3)(cos.stride(0) if cos.shape[0] > 1 else 0, cos.stride(1), 0)
    L = _lib.lib()
    with torch.cuda.device(q.device):
        rc = L.ksa_pre_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), qw.data_ptr(), kw.data_ptr(),
                                 cos.data_ptr(), sin.data_ptr(), qo.data_ptr(), ko.data_ptr(), vo.data_ptr(),
                                 b, S, Hq, Hkv, D, _DT[q.dtype], _bsh(q), _bsh(k), _bsh(v), _bsh(qo),
                                 _bsh(ko), _bsh(vo), cstr, None if kv_out_row is None else kv_out_row.data_ptr(),
                                 per_token, float(eps), _lib.stream_ptr(q.device))
    _lib.check(rc, "ksa_pre_attention")
    return qo, ko, vo


def pre_attention_partials(qkv, Hq: int, Hkv: int, D: int, q_norm_weight: torch.Tensor,
                           k_norm_weight: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, eps: float = 1e-6,
                           q_out: Optional[torch.Tensor] = None, k_out: Optional[torch.Tensor] = None,
                           v_out: Optional[torch.Tensor] = None,
                           kv_out_row: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """`pre_attention` on a fused q | k | v projection [b, S, (Hq + 2 Hkv) D] that is still the
    `SplitKPartials` of a deferred `linear_rows` (at most 128 rows): the partial sums are added
    inside the kernel, with the outputs of the two-kernel form."""
    from .gemm import SplitKPartials
    assert isinstance(qkv, SplitKPartials) and len(qkv.shape) == 3 and qkv.shape[-1] == (Hq + 2 * Hkv) * D
    b, S = qkv.shape[0], qkv.shape[1]
    dev, dtype = qkv.device, qkv.dtype
    if cos.dim() == 2:
        cos, sin = cos[None], sin[None]
    assert cos.shape[-2:] == (S, D) and sin.shape == cos.shape and cos.shape[0] in (1, b)
    cos = cos.to(dtype).contiguous()
    sin = sin.to(dtype).contiguous()
    qw = q_norm_weight.to(dtype).contiguous()
    kw = k_norm_weight.to(dtype).contiguous()
    assert qw.shape == (D,) and kw.shape == (D,)
    outs = []
    for given, H in ((q_out, Hq), (k_out, Hkv), (v_out, Hkv)):
        if given is None:
            given = torch.empty(b, S, H, D, dtype=dtype, device=dev)
        assert given.shape == (b, S, H, D) and given.dtype == dtype and given.stride(3) == 1
        outs.append(given)
    qo, ko, vo = outs
    if kv_out_row is not None:
        assert kv_out_row.is_cuda and kv_out_row.dtype == torch.int32 and tuple(kv_out_row.shape) in ((b,), (b, S)) \
            and kv_out_row.is_contiguous(), "kv_out_row must be a contiguous int32 [b] or [b, S] GPU tensor"
        assert k_out is not None and v_out is not None, "kv_out_row needs k_out and v_out"
    per_token = int(kv_out_row is not None and kv_out_row.dim() == 2)
    cstr = (ctypes.c_int64 * 3)(cos.stride(0) if cos.shape[0] > 1 else 0, cos.stride(1), 0)
    L = _lib.lib()
    with torch.cuda.device(dev):
        rc = L.ksa_pre_attention_partials(qkv.workspace.data_ptr(), qkv.ksplit, qw.data_ptr(), kw.data_ptr(),
                                          cos.data_ptr(), sin.data_ptr(), qo.data_ptr(), ko.data_ptr(),
                                          vo.data_ptr(), b, S, Hq, Hkv, D, _DT[dtype], _bsh(qo), _bsh(ko),
                                          _bsh(vo), cstr, None if kv_out_row is None else kv_out_row.data_ptr(),
                                          per_token, float(eps), _lib.stream_ptr(dev))
    _lib.check(rc, "ksa_pre_attention_partials")
    return qo, ko, vo
