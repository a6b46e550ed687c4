"""y = x W^T for the few rows of a decode step, as one weight-streaming HIP kernel.

Stands in for `torch.nn.functional.linear` (bias-free, as the reference's projections are:
examples/pretrain/hf_template/modeling_qwen3sa.py:628-641, :507-514, :1338) when x has at most
16 rows; anything larger should stay a library GEMM.  fp32 accumulation, one rounding at the
end.  No fallback: without libksa_hip.so it raises.
"""
from __future__ import annotations

import torch

from . import _lib

_DT = {torch.bfloat16: 0, torch.float16: 1}
MAX_ROWS = 16


def linear_rows(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x [..., K] with at most 16 rows in all, weight [N, K] -> [..., N]."""
    assert x.is_cuda and x.dtype in _DT and weight.dtype == x.dtype, "bf16/fp16 GPU tensors"
    K = x.shape[-1]
    N = weight.shape[0]
    assert weight.shape == (N, K) and weight.stride(1) == 1
    x2 = x.reshape(-1, K)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    assert 1 <= M <= MAX_ROWS, "linear_rows is for at most 16 rows"
    L = _lib.lib()
    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    ks = L.ksa_gemm_rows_auto_splits(N, K)
    ws = None
    ws_bytes = 0
    if ks > 1:
        ws_bytes = L.ksa_gemm_rows_workspace_bytes(N, ks)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = L.ksa_gemm_rows(x2.data_ptr(), weight.data_ptr(), out.data_ptr(), M, N, K, x2.stride(0),
                             weight.stride(0), out.stride(0), _DT[x.dtype], ks,
                             ws.data_ptr() if ws is not None else None, ws_bytes, _lib.stream_ptr(x.device))
    _lib.check(rc, "ksa_gemm_rows")
    return out.view(*x.shape[:-1], N)
