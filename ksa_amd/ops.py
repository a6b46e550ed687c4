"""The helper operators around the two attention paths as `torch.library.custom_op`s with fake
(shape-only) kernels, so that a caller may trace or `torch.compile` code that contains them:
`torch.ops.ksa_amd.{pre_attention, rmsnorm, add_rmsnorm, add_rmsnorm_partials, silu_mul, linear_rows,
gate_up_silu_rows, mlp_rows, argmax_rows}`.  (`summary_attn_fwd` and `decode_fwd` are registered where
they are defined, `prefill.py` and `decode.py`.)

They take and return plain tensors and allocate their outputs; the forms that write into a caller's
buffers or pass un-reduced partial sums between launches as Python objects (`pre.pre_attention(...,
k_out=cache view)`, `gemm.linear_rows(..., defer=True)`) stay plain functions, for the decoder module
that records them into HIP graphs itself.  The package-level `ksa_amd.pre_attention`, `add_rmsnorm`,
`silu_mul` and `linear_rows` go through these operators while a compiler is tracing and call the
kernels directly otherwise (an operator call costs some tens of microseconds of host time, as much as
a decode step's launch takes on the GPU).

Reference call sites: examples/pretrain/hf_template/modeling_qwen3sa.py:660-666 (q/k norm + rotary),
:64-79 with :946, :952 (residual add + RMSNorm), :507-514 (MLP), :628-641, :879, :1338 (projections).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib, elementwise, gemm, pre


@torch.library.custom_op("ksa_amd::pre_attention", mutates_args=())
def pre_attention_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_norm_weight: torch.Tensor,
                     k_norm_weight: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                     eps: float) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return pre.pre_attention(q, k, v, q_norm_weight, k_norm_weight, cos, sin, eps)


@pre_attention_op.register_fake
def _(q, k, v, q_norm_weight, k_norm_weight, cos, sin, eps):
    return q.new_empty(q.shape), k.new_empty(k.shape), v.new_empty(v.shape)


@torch.library.custom_op("ksa_amd::rmsnorm", mutates_args=())
def rmsnorm_op(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return elementwise.add_rmsnorm(x, None, weight, eps)[1]


@rmsnorm_op.register_fake
def _(x, weight, eps):
    return x.new_empty(x.shape)


@torch.library.custom_op("ksa_amd::add_rmsnorm", mutates_args=())
def add_rmsnorm_op(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                   eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    return elementwise.add_rmsnorm(x, residual, weight, eps)


@add_rmsnorm_op.register_fake
def _(x, residual, weight, eps):
    return x.new_empty(x.shape), x.new_empty(x.shape)


@torch.library.custom_op("ksa_amd::add_rmsnorm_partials", mutates_args=())
def add_rmsnorm_partials_op(partials: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                            eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """partials: fp32 [ksplit, 16, H], the un-reduced product of `mlp_rows` (rows = those of residual)."""
    ks, _, H = partials.shape
    rows = residual.numel() // H
    sk = gemm.SplitKPartials(partials.view(torch.uint8), ks, rows, residual.shape, residual.dtype)
    return elementwise.add_rmsnorm(sk, residual, weight, eps)


@add_rmsnorm_partials_op.register_fake
def _(partials, residual, weight, eps):
    return residual.new_empty(residual.shape), residual.new_empty(residual.shape)


@torch.library.custom_op("ksa_amd::silu_mul", mutates_args=())
def silu_mul_op(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return elementwise.silu_mul(gate, up)


@silu_mul_op.register_fake
def _(gate, up):
    return gate.new_empty(gate.shape)


@torch.library.custom_op("ksa_amd::linear_rows", mutates_args=())
def linear_rows_op(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    return gemm.linear_rows(x, weight)


@linear_rows_op.register_fake
def _(x, weight):
    return x.new_empty((*x.shape[:-1], weight.shape[0]))


@torch.library.custom_op("ksa_amd::gate_up_silu_rows", mutates_args=())
def gate_up_silu_rows_op(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    return gemm.gate_up_silu_rows(x, weight)


@gate_up_silu_rows_op.register_fake
def _(x, weight):
    return x.new_empty((*x.shape[:-1], weight.shape[0] // 2))


def mlp_rows_workspace(H: int, I: int, device) -> torch.Tensor:
    """Zeroed workspace tensor for `torch.ops.ksa_amd.mlp_rows` at one (hidden size, MLP size): make it
    once and pass it to every call on one stream."""
    return torch.zeros(_lib.lib().ksa_mlp_rows_workspace_bytes(H, I), dtype=torch.uint8, device=device)


def mlp_rows_down_splits(H: int, I: int) -> int:
    return int(_lib.lib().ksa_mlp_rows_down_splits(H, I))


class _WorkspaceView:
    """What `gemm.mlp_rows` needs of a `gemm.MlpRowsWorkspace`, around a caller's tensor."""

    def __init__(self, buf: torch.Tensor, H: int, I: int):
        self.buf, self.H, self.I = buf, H, I


@torch.library.custom_op("ksa_amd::mlp_rows", mutates_args=("workspace",))
def mlp_rows_op(x: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor,
                workspace: torch.Tensor) -> torch.Tensor:
    """down(SiLU(gate(x)) * up(x)) for at most 16 rows in one launch; returns the product's fp32 partial
    sums [ksplit, 16, H] for `add_rmsnorm_partials` (the next layer's residual add + norm adds them)."""
    H, I = x.shape[-1], w_gate_up.shape[0] // 2
    assert workspace.dtype == torch.uint8 and workspace.is_contiguous()
    assert gemm.mlp_rows_supported(x.numel() // H, H, I), "mlp_rows: shape not supported by the one-launch kernel"
    sk = gemm.mlp_rows(x, w_gate_up, w_down, _WorkspaceView(workspace, H, I))
    return sk.workspace.view(torch.float32).view(sk.ksplit, 16, H)


@mlp_rows_op.register_fake
def _(x, w_gate_up, w_down, workspace):
    H, I = x.shape[-1], w_gate_up.shape[0] // 2
    return x.new_empty((mlp_rows_down_splits(H, I), 16, H), dtype=torch.float32)


@torch.library.custom_op("ksa_amd::argmax_rows", mutates_args=())
def argmax_rows_op(x: torch.Tensor) -> torch.Tensor:
    return elementwise.argmax_rows(x)


@argmax_rows_op.register_fake
def _(x):
    return x.new_empty(x.shape[:-1], dtype=torch.long)


OPERATORS = ("pre_attention", "rmsnorm", "add_rmsnorm", "add_rmsnorm_partials", "silu_mul", "linear_rows",
             "gate_up_silu_rows", "mlp_rows", "argmax_rows")


def _tracing() -> bool:
    return torch.compiler.is_compiling()


# ---- the package-level functions: operators while a compiler traces, direct calls otherwise ----

def pre_attention(q, k, v, q_norm_weight, k_norm_weight, cos, sin, eps: float = 1e-6, q_out=None, k_out=None,
                  v_out=None, kv_out_row=None):
    if _tracing() and q_out is None and k_out is None and v_out is None and kv_out_row is None:
        return pre_attention_op(q, k, v, q_norm_weight, k_norm_weight, cos, sin, float(eps))
    return pre.pre_attention(q, k, v, q_norm_weight, k_norm_weight, cos, sin, eps, q_out, k_out, v_out, kv_out_row)


pre_attention.__doc__ = pre.pre_attention.__doc__


def add_rmsnorm(x, residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float = 1e-6):
    if _tracing() and isinstance(x, torch.Tensor):
        if residual is None:
            return x, rmsnorm_op(x, weight, float(eps))
        return add_rmsnorm_op(x, residual, weight, float(eps))
    return elementwise.add_rmsnorm(x, residual, weight, eps)


add_rmsnorm.__doc__ = elementwise.add_rmsnorm.__doc__


def silu_mul(gate, up: Optional[torch.Tensor] = None):
    if _tracing() and isinstance(gate, torch.Tensor):
        if up is None:
            I = gate.shape[-1] // 2
            gate, up = gate[..., :I], gate[..., I:]
        return silu_mul_op(gate, up)
    return elementwise.silu_mul(gate, up)


silu_mul.__doc__ = elementwise.silu_mul.__doc__


def linear_rows(x: torch.Tensor, weight: torch.Tensor, defer: bool = False):
    if _tracing() and not defer:
        return linear_rows_op(x, weight)
    return gemm.linear_rows(x, weight, defer)


linear_rows.__doc__ = gemm.linear_rows.__doc__
