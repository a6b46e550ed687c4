"""The reference's PyTorch CPU paths, restated for timing beside the GPU numbers.
TEST / BENCHMARK INFRASTRUCTURE ONLY (the benchmark's `cpu_baseline` leg and tests).

Follows
  muse/layers/summary_attention_func.py:327-457  block mode: query blocks of 4096 rows,
      gathered key set + compact bool mask per block, F.scaled_dot_product_attention,
      K/V already expanded to the query head count
  muse/layers/summary_attention_func.py:142-191  mask mode (dense [s, s] bool mask)
  examples/pretrain/hf_template/modeling_qwen3sa.py:557-566,591-612  decode:
      repeat_kv + F.scaled_dot_product_attention(attn_mask=None, is_causal=False)
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

from . import ksa_oracle as O

BLOCK_ROWS = 4096


def block_mode_rows(q_blk, k, v, q0, C, S, W):
    """Attention output of query rows [q0, q0+n) of an in-line sequence.
    q_blk [n, Hq, D]; k, v [Sq, Hkv, D] fp32.  Returns [n, Hq, D]."""
    n, Hq, D = q_blk.shape
    Sq, Hkv, _ = k.shape
    g = Hq // Hkv
    rows = np.arange(q0, q0 + n)
    hi = q0 + n  # causal: nothing beyond the block's last row is visible
    vis = O.mask_predicate(rows[:, None], np.arange(hi)[None, :], C, S, W, 0)
    k_pos = np.nonzero(vis.any(axis=0))[0]
    mask = torch.from_numpy(vis[:, k_pos])
    kp = torch.from_numpy(k_pos)
    kb = k[kp].repeat_interleave(g, dim=1).permute(1, 0, 2)[None]   # [1, Hq, k_len, D]
    vb = v[kp].repeat_interleave(g, dim=1).permute(1, 0, 2)[None]
    qb = q_blk.permute(1, 0, 2)[None]
    out = F.scaled_dot_product_attention(qb, kb, vb, attn_mask=mask, dropout_p=0.0, is_causal=False)
    return out[0].permute(1, 0, 2)


def mask_mode(q, k, v, C, S, W):
    """Dense-mask path for small sequences.  q [Sq, Hq, D], k/v [Sq, Hkv, D] -> [Sq, Hq, D]."""
    Sq, Hq, D = q.shape
    g = Hq // k.shape[1]
    mask = torch.from_numpy(O.dense_mask_intervals(Sq, C, S, W))
    kb = k.repeat_interleave(g, dim=1).permute(1, 0, 2)[None]
    vb = v.repeat_interleave(g, dim=1).permute(1, 0, 2)[None]
    out = F.scaled_dot_product_attention(q.permute(1, 0, 2)[None], kb, vb, attn_mask=mask)
    return out[0].permute(1, 0, 2)


def decode_sdpa(q, k, v, g):
    """q [b, Hq, Q, D], k/v [b, Hkv, L, D] -> [b, Q, Hq, D]"""
    b, Hkv, L, D = k.shape
    ke = k[:, :, None].expand(b, Hkv, g, L, D).reshape(b, Hkv * g, L, D)
    ve = v[:, :, None].expand(b, Hkv, g, L, D).reshape(b, Hkv * g, L, D)
    out = F.scaled_dot_product_attention(q, ke, ve, attn_mask=None, dropout_p=0.0, is_causal=False)
    return out.transpose(1, 2).contiguous()


def pre_attention(q, k, v, q_weight, k_weight, cos, sin, eps=1e-6):
    """The reference's pre-attention sequence restated with torch CPU tensor ops in the input
    dtype (examples/pretrain/hf_template/modeling_qwen3sa.py:64-79 Qwen3RMSNorm.forward,
    :516-554 rotate_half / apply_rotary_pos_emb, :660-666 call site), for [b, S, H, D] inputs
    (the reference holds them as [b, H, S, D]; every op here is element-wise over (b, S, H)).
    Returns (q', k', v)."""
    def rms(x, w):
        dt = x.dtype
        xf = x.to(torch.float32)
        var = xf.pow(2).mean(-1, keepdim=True)
        xf = xf * torch.rsqrt(var + eps)
        return w * xf.to(dt)

    def rot(x):
        h = x.shape[-1] // 2
        return torch.cat((-x[..., h:], x[..., :h]), dim=-1)

    c = cos.unsqueeze(2)  # broadcast over heads
    s = sin.unsqueeze(2)
    qn, kn = rms(q, q_weight), rms(k, k_weight)
    return qn * c + rot(qn) * s, kn * c + rot(kn) * s, v


def add_rmsnorm(x, residual, weight, eps=1e-6):
    """Residual add followed by Qwen3RMSNorm.forward, with torch CPU tensor ops in the input
    dtype (examples/pretrain/hf_template/modeling_qwen3sa.py:64-79 and the adds at :946, :952).
    Returns (x + residual, weight * norm(x + residual))."""
    s = x if residual is None else x + residual
    sf = s.to(torch.float32)
    sf = sf * torch.rsqrt(sf.pow(2).mean(-1, keepdim=True) + eps)
    return s, weight * sf.to(s.dtype)


def silu_mul(gate, up):
    """act_fn(gate) * up of Qwen3MLP.forward (:507-514) in the input dtype."""
    return F.silu(gate) * up
