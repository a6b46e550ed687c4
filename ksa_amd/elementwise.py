"""Element-wise steps of a decoder layer around the attention path, one HIP kernel each.

`add_rmsnorm` is the reference's `Qwen3RMSNorm.forward`
(examples/pretrain/hf_template/modeling_qwen3sa.py:64-79) fused with the residual add in front of
it (`Qwen3DecoderLayer.forward` :946, :952); `silu_mul` is the activation of `Qwen3MLP.forward`
(:507-514).  Both keep the rounding points of the reference's 16-bit tensor ops.  No fallback:
without libksa_hip.so they raise.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from .gemm import SplitKPartials

_DT = {torch.bfloat16: 0, torch.float16: 1}


def _rows2d(t: torch.Tensor) -> torch.Tensor:
    """[..., H] -> [rows, H] view with a contiguous last dim (copies only if it must)."""
    if t.stride(-1) != 1:
        t = t.contiguous()
    try:
        return t.view(-1, t.shape[-1])
    except RuntimeError:
        return t.reshape(-1, t.shape[-1])


def _add_rmsnorm_partials(x: SplitKPartials, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    assert residual is not None and residual.is_cuda and residual.dtype == x.dtype and tuple(residual.shape) == x.shape
    H = x.shape[-1]
    r2 = _rows2d(residual)
    assert r2.shape[0] == x.rows
    w = weight.to(x.dtype).contiguous()
    assert w.shape == (H,)
    out = torch.empty(r2.shape, dtype=x.dtype, device=x.device)
    s = torch.empty(r2.shape, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ksa_add_rmsnorm_partials(x.workspace.data_ptr(), x.ksplit, r2.data_ptr(), w.data_ptr(),
                                                 out.data_ptr(), s.data_ptr(), x.rows, H, r2.stride(0),
                                                 out.stride(0), s.stride(0), _DT[x.dtype], float(eps),
                                                 _lib.stream_ptr(x.device))
    _lib.check(rc, "ksa_add_rmsnorm_partials")
    return s.view(x.shape), out.view(x.shape)


def add_rmsnorm(x: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor,
                eps: float = 1e-6) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (s, weight * rmsnorm(s)) with s = x + residual (s is x itself when residual is None).
    x may be the `SplitKPartials` of a deferred `linear_rows` (then residual is required): the
    partial sums are added here, with the same result as the reduced product would give."""
    if isinstance(x, SplitKPartials):
        return _add_rmsnorm_partials(x, residual, weight, eps)
    assert x.is_cuda and x.dtype in _DT, "x must be a bf16/fp16 GPU tensor"
    H = x.shape[-1]
    x2 = _rows2d(x)
    w = weight.to(x.dtype).contiguous()
    assert w.shape == (H,)
    out = torch.empty(x2.shape, dtype=x.dtype, device=x.device)
    L = _lib.lib()
    if residual is not None:
        assert residual.shape == x.shape and residual.dtype == x.dtype
        r2 = _rows2d(residual)
        s = torch.empty(x2.shape, dtype=x.dtype, device=x.device)
        args = (r2.data_ptr(), w.data_ptr(), out.data_ptr(), s.data_ptr(), x2.shape[0], H, x2.stride(0),
                r2.stride(0), out.stride(0), s.stride(0))
    else:
        s = x2
        args = (None, w.data_ptr(), out.data_ptr(), None, x2.shape[0], H, x2.stride(0), 0, out.stride(0), 0)
    with torch.cuda.device(x.device):
        rc = L.ksa_add_rmsnorm(x2.data_ptr(), *args, _DT[x.dtype], float(eps), _lib.stream_ptr(x.device))
    _lib.check(rc, "ksa_add_rmsnorm")
    return s.view(x.shape), out.view(x.shape)


def silu_mul(gate, up: Optional[torch.Tensor] = None) -> torch.Tensor:
    """round(silu(gate)) * up; gate and up may be strided views (halves of one GEMM output).
    With `up` left out, `gate` is the whole gate | up projection [..., 2 I]: a tensor, or the
    `SplitKPartials` of a deferred `linear_rows`, whose partial sums are then added here."""
    if isinstance(gate, SplitKPartials):
        assert up is None
        x = gate
        I = x.shape[-1] // 2
        out = torch.empty(x.rows, I, dtype=x.dtype, device=x.device)
        with torch.cuda.device(x.device):
            rc = _lib.lib().ksa_silu_mul_partials(x.workspace.data_ptr(), x.ksplit, out.data_ptr(), x.rows, I,
                                                  out.stride(0), _DT[x.dtype], _lib.stream_ptr(x.device))
        _lib.check(rc, "ksa_silu_mul_partials")
        return out.view(*x.shape[:-1], I)
    if up is None:
        I = gate.shape[-1] // 2
        gate, up = gate[..., :I], gate[..., I:]
    assert gate.is_cuda and gate.dtype in _DT and up.dtype == gate.dtype and gate.shape == up.shape
    I = gate.shape[-1]
    g2, u2 = _rows2d(gate), _rows2d(up)
    out = torch.empty(g2.shape, dtype=gate.dtype, device=gate.device)
    with torch.cuda.device(gate.device):
        rc = _lib.lib().ksa_silu_mul(g2.data_ptr(), u2.data_ptr(), out.data_ptr(), g2.shape[0], I, g2.stride(0),
                                     u2.stride(0), out.stride(0), _DT[gate.dtype], _lib.stream_ptr(gate.device))
    _lib.check(rc, "ksa_silu_mul")
    return out.view(gate.shape)


def argmax_rows(x: torch.Tensor) -> torch.Tensor:
    """Index of the largest value along the last dimension (lowest index among equals), int64:
    `torch.argmax(x, dim=-1)` for 16-bit logits in one small launch (`ksa_argmax_rows`)."""
    assert x.is_cuda and x.dtype in _DT
    x2 = _rows2d(x)
    out = torch.empty(x2.shape[0], dtype=torch.long, device=x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ksa_argmax_rows(x2.data_ptr(), out.data_ptr(), x2.shape[0], x2.shape[1], x2.stride(0),
                                        _DT[x.dtype], _lib.stream_ptr(x.device))
    _lib.check(rc, "ksa_argmax_rows")
    return out.view(x.shape[:-1])
