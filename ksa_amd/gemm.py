"""y = x W^T for the few rows of a decode step, as one weight-streaming HIP kernel.

Stands in for `torch.nn.functional.linear` (bias-free, as the reference's projections are:
examples/pretrain/hf_template/modeling_qwen3sa.py:628-641, :507-514, :1338) when x has at most
128 rows (up to 16: one MFMA operand; 17 to 128, a larger batch or the 9 tokens per sequence of a
chunk-boundary step: the kernel's wide form); anything larger should stay a library GEMM.  fp32
accumulation, one rounding at the end.  No fallback: without libksa_hip.so it raises.
"""
from __future__ import annotations

import torch

from . import _lib

_DT = {torch.bfloat16: 0, torch.float16: 1}
MAX_ROWS = 128       # rows of x the GEMM kernels take
MLP_MAX_ROWS = 16    # rows the one-launch MLP takes (x whole in LDS)


W_TILED = -1   # row stride that names the streaming layout (include/ksa_hip.h, KSA_W_TILED)


class TiledWeight:
    """A weight matrix [N, K] in the streaming layout of the few-rows kernels, [ceil(N / 16)][K / 32][16][32]
    (`ksa_tile_weights`): what a wave reads of it is one sequential run instead of 64-byte pieces of rows K
    elements apart.  A second copy of the matrix for the decode steps; `linear_rows`, `gate_up_silu_rows`,
    `mlp_rows` and `add_rmsnorm_mlp_rows` take it in place of the tensor, with bit-identical results."""

    def __init__(self, weight: torch.Tensor):
        assert weight.is_cuda and weight.dtype in _DT and weight.dim() == 2 and weight.stride(1) == 1
        N, K = weight.shape
        assert K % 32 == 0, "K must be a multiple of 32"
        L = _lib.lib()
        self.shape, self.dtype, self.device = (N, K), weight.dtype, weight.device
        self.data = torch.empty(L.ksa_tile_weights_bytes(N, K) // 2, dtype=weight.dtype, device=weight.device)
        with torch.cuda.device(weight.device):
            rc = L.ksa_tile_weights(weight.data_ptr(), self.data.data_ptr(), N, K, weight.stride(0),
                                    _lib.stream_ptr(weight.device))
        _lib.check(rc, "ksa_tile_weights")

    def stride(self, dim):
        return W_TILED if dim == 0 else 1

    def data_ptr(self):
        return self.data.data_ptr()


def _weight_ok(weight, N, K, dtype):
    """Shape / dtype / layout check of a weight operand (a tensor with contiguous rows, or a `TiledWeight`)."""
    return tuple(weight.shape) == (N, K) and weight.dtype == dtype and weight.stride(1) == 1


class SplitKPartials:
    """Output of `linear_rows(..., defer=True)` when K was split over workgroups: the fp32 partial
    sums [ksplit, rows rounded up to whole 16-row blocks, N] as the kernel left them, for a consumer that adds them itself
    (`ksa_amd.add_rmsnorm`).  `shape` / `dtype` are those of the tensor it stands for."""

    def __init__(self, workspace: torch.Tensor, ksplit: int, rows: int, shape, dtype):
        self.workspace, self.ksplit, self.rows, self.shape, self.dtype = workspace, ksplit, rows, tuple(shape), dtype

    @property
    def device(self):
        return self.workspace.device


def linear_rows(x: torch.Tensor, weight: torch.Tensor, defer: bool = False):
    """x [..., K] with at most 128 rows in all, weight [N, K] -> [..., N].  With `defer`, a product
    whose K is split over workgroups comes back as `SplitKPartials` (no reduction launch)."""
    assert x.is_cuda and x.dtype in _DT and weight.dtype == x.dtype, "bf16/fp16 GPU tensors"
    K = x.shape[-1]
    N = weight.shape[0]
    assert _weight_ok(weight, N, K, x.dtype)
    x2 = x.reshape(-1, K)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    assert 1 <= M <= MAX_ROWS, "linear_rows is for at most 128 rows"
    L = _lib.lib()
    with torch.cuda.device(x.device):
        ks = L.ksa_gemm_rows_splits(M, N, K)
    defer = defer and ks > 1
    out = None if defer else torch.empty(M, N, dtype=x.dtype, device=x.device)
    ws = None
    ws_bytes = 0
    if ks > 1:
        ws_bytes = L.ksa_gemm_rows_partials_bytes(M, N, ks)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = L.ksa_gemm_rows(x2.data_ptr(), weight.data_ptr(), None if defer else out.data_ptr(), M, N, K,
                             x2.stride(0), weight.stride(0), N, _DT[x.dtype], ks,
                             ws.data_ptr() if ws is not None else None, ws_bytes, _lib.stream_ptr(x.device))
    _lib.check(rc, "ksa_gemm_rows")
    if defer:
        return SplitKPartials(ws, ks, M, (*x.shape[:-1], N), x.dtype)
    return out.view(*x.shape[:-1], N)


def gate_up_silu_rows(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x [..., K] with at most 128 rows in all, weight [2 I, K] (gate rows, then up rows) ->
    SiLU(x W_gate^T) * (x W_up^T) [..., I] in one launch (`ksa_gemm_rows_gate_up_silu`): the MLP's
    `act_fn(gate_proj(x)) * up_proj(x)` (modeling_qwen3sa.py:507-514) at a decode step."""
    assert x.is_cuda and x.dtype in _DT and weight.dtype == x.dtype, "bf16/fp16 GPU tensors"
    K = x.shape[-1]
    I = weight.shape[0] // 2
    assert _weight_ok(weight, 2 * I, K, x.dtype)
    x2 = x.reshape(-1, K)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    assert 1 <= M <= MAX_ROWS, "gate_up_silu_rows is for at most 128 rows"
    out = torch.empty(M, I, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().ksa_gemm_rows_gate_up_silu(x2.data_ptr(), weight.data_ptr(), out.data_ptr(), M, I, K,
                                                   x2.stride(0), weight.stride(0), I, _DT[x.dtype],
                                                   _lib.stream_ptr(x.device))
    _lib.check(rc, "ksa_gemm_rows_gate_up_silu")
    return out.view(*x.shape[:-1], I)


class MlpRowsTimeout(RuntimeError):
    """A `ksa_mlp_rows` / `ksa_add_rmsnorm_mlp_rows` launch gave up waiting inside the kernel: what was
    computed since the last clean check is not valid."""


class MlpRowsWorkspace:
    """Barrier words and the activation buffer of `mlp_rows` for one (device, hidden size, MLP size):
    zeroed once, then shared by every layer's call on that stream (the calls run one after the other,
    with any number of rows each)."""

    def __init__(self, H: int, I: int, device):
        L = _lib.lib()
        self.H, self.I = H, I
        self.buf = torch.zeros(L.ksa_mlp_rows_workspace_bytes(H, I), dtype=torch.uint8, device=device)
        self._status = self.buf[L.ksa_mlp_rows_status_offset():][:8].view(torch.int64)

    def failed(self) -> bool:
        """True if a launch gave up waiting inside the kernel.  Waits for the whole device to be idle
        first (no launch on the workspace may be in flight, on any stream, when its words are read or
        cleared); after a failure the workspace is zeroed again so that it can be used further.
        Recorded graphs that launch on it stay valid (the buffer does not move)."""
        torch.cuda.synchronize(self.buf.device)
        bad = bool(self._status.item() != 0)
        if bad:
            self.buf.zero_()
            torch.cuda.synchronize(self.buf.device)
        return bad


def mlp_rows_supported(M: int, H: int, I: int) -> bool:
    return (1 <= M <= MLP_MAX_ROWS and H % 128 == 0 and I % 32 == 0 and I <= 26624
            and M * (H + 8) * 2 <= 160 * 1024)


def mlp_rows(x: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor, ws: MlpRowsWorkspace) -> SplitKPartials:
    """One launch for `down(SiLU(gate(x)) * up(x))` at a decode step (`ksa_mlp_rows`;
    modeling_qwen3sa.py:507-514).  The result comes as `SplitKPartials` for the next residual add + norm."""
    H = x.shape[-1]
    I = w_gate_up.shape[0] // 2
    dt = x.dtype
    assert x.is_cuda and dt in _DT
    assert _weight_ok(w_gate_up, 2 * I, H, dt) and _weight_ok(w_down, H, I, dt) and ws.H == H and ws.I == I
    x2 = x.reshape(-1, H)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    L = _lib.lib()
    with torch.cuda.device(x2.device):
        ks = L.ksa_mlp_rows_down_splits(H, I)
        part = torch.empty(ks * 16 * H, dtype=torch.float32, device=x2.device)
        rc = L.ksa_mlp_rows(x2.data_ptr(), w_gate_up.data_ptr(), w_down.data_ptr(), part.data_ptr(), M, H, I,
                            x2.stride(0), w_gate_up.stride(0), w_down.stride(0), _DT[dt], ws.buf.data_ptr(),
                            ws.buf.numel(), _lib.stream_ptr(x2.device))
    _lib.check(rc, "ksa_mlp_rows")
    return SplitKPartials(part.view(torch.uint8), ks, M, x.shape, dt)


def add_rmsnorm_mlp_rows(o_partials: SplitKPartials, residual: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                         w_gate_up: torch.Tensor, w_down: torch.Tensor, ws: MlpRowsWorkspace):
    """One launch for `x' = residual + o_proj output; h = norm(x'); d = down(SiLU(gate(h)) * up(h))` at a
    decode step (`ksa_add_rmsnorm_mlp_rows`; modeling_qwen3sa.py:944-952, :507-514).  Returns (x', d) with d
    as `SplitKPartials` for the next residual add + norm."""
    H = o_partials.shape[-1]
    I = w_gate_up.shape[0] // 2
    M = o_partials.rows
    dt = o_partials.dtype
    assert _weight_ok(w_gate_up, 2 * I, H, dt) and _weight_ok(w_down, H, I, dt) and ws.H == H and ws.I == I and H <= 4096
    r2 = residual.reshape(-1, H)
    if r2.stride(1) != 1:
        r2 = r2.contiguous()
    assert r2.shape[0] == M and r2.dtype == dt
    w = norm_weight.to(dt).contiguous()
    L = _lib.lib()
    with torch.cuda.device(r2.device):
        ks = L.ksa_mlp_rows_down_splits(H, I)
        out_sum = torch.empty(M, H, dtype=dt, device=r2.device)
        part = torch.empty(ks * 16 * H, dtype=torch.float32, device=r2.device)
        rc = L.ksa_add_rmsnorm_mlp_rows(o_partials.workspace.data_ptr(), o_partials.ksplit, r2.data_ptr(), w.data_ptr(),
                                        out_sum.data_ptr(), w_gate_up.data_ptr(), w_down.data_ptr(), part.data_ptr(),
                                        M, H, I, r2.stride(0), H, w_gate_up.stride(0), w_down.stride(0), _DT[dt],
                                        float(eps), ws.buf.data_ptr(), ws.buf.numel(), _lib.stream_ptr(r2.device))
    _lib.check(rc, "ksa_add_rmsnorm_mlp_rows")
    return out_sum.view(residual.shape), SplitKPartials(part.view(torch.uint8), ks, M, residual.shape, dt)
