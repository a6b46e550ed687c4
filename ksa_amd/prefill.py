"""Block-sparse Summary-Attention prefill forward on MI355X.

Mirror of the reference's public prefill operator
(summary_attn-0.3.0 wheel, summary_attn/interface.py:271-289 `summary_attn_func`;
call sites: examples/pretrain/hf_template/modeling_qwen3sa.py:806-815 and
muse/layers/summary_attention_func.py:67-73): same positional arguments, same
keywords, same `(out, lse_or_None)` return.  The work is done by the HIP kernels of
libksa_hip.so; there is no other execution path.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional, Tuple

import torch

from . import _lib

TILE_M = 128
TILE_N = 64

# (Sq, C, S, W, P, skip_old, device index) -> (mask_cnt, mask_idx, full_cnt, full_idx)
# The reference keeps the same process-global cache keyed by shape parameters
# (summary_attn/interface.py:26,46-68); the device is added to the key here because the
# tensors live on one.
SUMMARY_ATTN_CACHE: Dict[Tuple, Tuple[torch.Tensor, ...]] = {}

_DTYPES = {torch.bfloat16: 0, torch.float16: 1}

# Workgroup shape handed to ksa_prefill_fwd when a call does not name one: 0 = the library's
# choice, 2 = two heads on 8 waves, 32 = one head on 4 waves, 64 = two heads on 4 waves with 64
# query rows per wave (include/ksa_hip.h, KSA_PREFILL_SHAPE_*).  A tuning knob: results agree to
# the tolerance of the tests, only the speed differs.
PREFILL_SHAPE = 0


class BlockSparseIndex(tuple):
    """(mask_block_cnt, mask_block_idx, full_block_cnt, full_block_idx) with the
    reference's shapes [1,1,M] / [1,1,M,N] (flash_attn/cute/block_sparsity.py:17-34)."""

    block_size = (TILE_M, TILE_N)


def compute_block_sparsity(seqlen_q: int, seqlen_k: int, chunk_size: int, summary_num: int,
                           sliding_chunk_num: int, skip_old_summary: bool = False,
                           tile_m: int = TILE_M, tile_n: int = TILE_N,
                           device=None) -> BlockSparseIndex:
    """Builds the four int32 index tensors on the GPU (bit-exact with the reference's
    BlockSparsityKernel, flash_attn/cute/compute_block_sparsity.py:189-274)."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if device.type != "cuda":
        raise AssertionError("compute_block_sparsity runs on the GPU only")
    M = -(-seqlen_q // tile_m)
    N = -(-seqlen_k // tile_n)
    with torch.cuda.device(device):
        mc = torch.empty((1, 1, M), dtype=torch.int32, device=device)
        fc = torch.empty((1, 1, M), dtype=torch.int32, device=device)
        mi = torch.empty((1, 1, M, N), dtype=torch.int32, device=device)
        fi = torch.empty((1, 1, M, N), dtype=torch.int32, device=device)
        rc = _lib.lib().ksa_block_index(
            seqlen_q, seqlen_k, chunk_size, summary_num, sliding_chunk_num, seqlen_k - seqlen_q,
            int(bool(skip_old_summary)), tile_m, tile_n, mc.data_ptr(), mi.data_ptr(),
            fc.data_ptr(), fi.data_ptr(), _lib.stream_ptr(device))
    _lib.check(rc, "ksa_block_index")
    return BlockSparseIndex((mc, mi, fc, fi))


def _cached_index(Sq, C, S, W, P, skip_old, device) -> BlockSparseIndex:
    key = (Sq, C, S, W, P, bool(skip_old), device.index)
    idx = SUMMARY_ATTN_CACHE.get(key)
    if idx is None:
        idx = compute_block_sparsity(Sq, Sq + P, C, S, W, skip_old, device=device)
        SUMMARY_ATTN_CACHE[key] = idx
    return idx


# summary_pos analysis is cached per buffer: the HF call site hands every layer a fresh
# `summary_mask.squeeze(0)` view of one tensor (modeling_qwen3sa.py:807-815), so the key is the
# storage address, not the Python object.
# An entry holds the tensor it analysed, which keeps that storage alive: while the entry exists
# the address cannot be handed to another mask.
# (data_ptr, numel, device, Sq, C, S) -> (tensor, version or None, result)
_POS_CACHE: Dict[tuple, tuple] = {}
_POS_CACHE_MAX = 16
_POS_ANALYSES = 0   # number of analyses actually run (each costs one host synchronisation)


def _pos_version(t: torch.Tensor):
    """In-place modification counter of `t`, or None for inference tensors, which have none
    (reading `_version` on them raises)."""
    return None if t.is_inference() else t._version


def _analyse_summary_pos(summary_pos: torch.Tensor, Sq: int, C: int, S: int):
    """Returns (P, periodic, rows): P = number of summary rows; periodic = summary_pos
    is exactly `(i % (C+S)) >= C` over whole blocks followed by text rows only, so that
    prefix row j can be read in place at (j//S)*(C+S)+C+j%S; rows = int32 row indices of
    the summary rows (only when not periodic).

    The result is kept per (storage address, length, device, Sq, C, S) together with the
    tensor's in-place modification counter.  Inference tensors have no such counter: a mask made
    under torch.inference_mode() and later rewritten in place must be followed by
    `clear_summary_pos_cache()`."""
    global _POS_ANALYSES
    key = (summary_pos.data_ptr(), summary_pos.numel(), str(summary_pos.device), Sq, C, S)
    ver = _pos_version(summary_pos)
    hit = _POS_CACHE.get(key)
    if hit is not None and hit[1] == ver:
        return hit[2]
    if summary_pos.dtype != torch.bool or summary_pos.dim() != 1 or summary_pos.numel() != Sq:
        raise AssertionError("summary_pos must be a bool tensor of shape [seqlen_q]")
    B = C + S
    i = torch.arange(Sq, device=summary_pos.device)
    n_sum = summary_pos.sum()
    n_full = n_sum // S
    expected = ((i % B) >= C) & (i < n_full * B)
    stats = torch.stack([n_sum, (summary_pos != expected).sum()]).tolist()  # one sync
    P, mismatch = int(stats[0]), int(stats[1])
    periodic = mismatch == 0 and P % S == 0
    rows = None
    if not periodic:
        rows = torch.nonzero(summary_pos, as_tuple=False).flatten().to(torch.int32)
    res = (P, periodic, rows)
    _POS_ANALYSES += 1
    if len(_POS_CACHE) >= _POS_CACHE_MAX:
        _POS_CACHE.clear()
    _POS_CACHE[key] = (summary_pos, ver, res)
    return res


def clear_summary_pos_cache() -> None:
    _POS_CACHE.clear()


def _check_inputs(q, k, v):
    assert q.is_cuda and k.is_cuda and v.is_cuda, "inputs must be on a GPU"
    assert q.dtype in _DTYPES, "inputs must be float16 or bfloat16"
    assert q.dtype == k.dtype == v.dtype, "inputs must have the same dtype"
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q/k/v must be [batch, seq, heads, head_dim]"
    assert k.shape == v.shape, "k and v must have the same shape"
    assert q.shape[0] == k.shape[0], "batch mismatch"
    D = q.shape[-1]
    assert k.shape[-1] == D, "head_dim mismatch"
    assert D <= 256, "head dimension must be at most 256"
    assert D % 8 == 0, "head dimension must be a multiple of 8"
    assert q.shape[2] % k.shape[2] == 0, "num_heads must be divisible by num_heads_kv"


def _lastdim_contig(t):
    return t if t.stride(-1) == 1 else t.contiguous()


KERNEL_HEAD_DIMS = (64, 128, 256)


def kernel_head_dim(D: int) -> int:
    """The head dimension the kernels run a head dimension D at: the next of 64 / 128 / 256.  The
    reference takes any multiple of 8 up to 256 (flash_attn/cute/interface.py:206-209); other
    values are zero-padded to the next kernel size (zero columns add nothing to a score, and the
    padded output columns are dropped), with the soft-max scale of the true D."""
    for d in KERNEL_HEAD_DIMS:
        if D <= d:
            return d
    raise AssertionError("head dimension must be at most 256")


def pad_head_dim(t: torch.Tensor, Dk: int) -> torch.Tensor:
    return t if t.shape[-1] == Dk else torch.nn.functional.pad(t, (0, Dk - t.shape[-1]))


@torch.library.custom_op("ksa_amd::summary_attn_fwd", mutates_args=())
def _summary_attn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      mask_cnt: torch.Tensor, mask_idx: torch.Tensor, full_cnt: torch.Tensor,
                      full_idx: torch.Tensor, C: int, S: int, W: int, P: int, skip_old: bool,
                      phys_prefix: bool, scale: float, want_lse: bool,
                      shape: int) -> Tuple[torch.Tensor, torch.Tensor]:
    b, Sq, Hq, D = q.shape
    Hkv = k.shape[2]
    out = torch.empty_like(q)
    lse = torch.empty((b, Hq, Sq) if want_lse else (0,), dtype=torch.float32, device=q.device)
    sched = torch.empty(8, dtype=torch.int32, device=q.device)   # work queues of this call alone
    dims = (0, 1, 2)
    with torch.cuda.device(q.device):
        rc = _lib.lib().ksa_prefill_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
            lse.data_ptr() if want_lse else None,
            b, Sq, Hq, Hkv, D, _DTYPES[q.dtype],
            _lib.strides3(q, dims), _lib.strides3(k, dims), _lib.strides3(out, dims),
            C, S, W, P, int(skip_old), int(phys_prefix),
            mask_cnt.data_ptr(), mask_idx.data_ptr(), full_cnt.data_ptr(), full_idx.data_ptr(),
            mask_idx.shape[-1], float(scale), int(shape), sched.data_ptr(), _lib.stream_ptr(q.device))
    _lib.check(rc, "ksa_prefill_fwd")
    return out, lse


@_summary_attn_fwd.register_fake
def _(q, k, v, mask_cnt, mask_idx, full_cnt, full_idx, C, S, W, P, skip_old, phys_prefix, scale,
      want_lse, shape):
    b, Sq, Hq, _ = q.shape
    return torch.empty_like(q), q.new_empty((b, Hq, Sq) if want_lse else (0,), dtype=torch.float32)


def _gathered_prefix(t: torch.Tensor, rows: torch.Tensor, P: int) -> torch.Tensor:
    """[prefix rows | in-line rows] of t [b, Sq, H, D], built with the HIP row mover (the
    layout the reference makes with torch.cat((t[:, summary_pos], t), dim=1))."""
    b, Sq, H, D = t.shape
    full = torch.empty((b, P + Sq, H, D), dtype=t.dtype, device=t.device)
    lib = _lib.lib()
    with torch.cuda.device(t.device):
        st = _lib.stream_ptr(t.device)
        rc = lib.ksa_copy_rows(t.data_ptr(), full.data_ptr(), rows.data_ptr(), None, 0, 0, P, b, H, D,
                               _lib.strides3(t, (0, 2, 1)), _lib.strides3(full, (0, 2, 1)), st)
        _lib.check(rc, "ksa_copy_rows")
        rc = lib.ksa_copy_rows(t.data_ptr(), full.data_ptr(), None, None, 0, P, Sq, b, H, D,
                               _lib.strides3(t, (0, 2, 1)), _lib.strides3(full, (0, 2, 1)), st)
        _lib.check(rc, "ksa_copy_rows")
    return full


def summary_attn_func(q, k, v, chunk_size, summary_num, sliding_chunk_num,
                      summary_pos: Optional[torch.Tensor] = None,
                      skip_old_summary: bool = False, *, return_lse: bool = False,
                      softmax_scale: Optional[float] = None, workgroup_shape: Optional[int] = None):
    """q [b, Sq, Hq, D]; k, v [b, Sq (+P), Hkv, D]; returns (out [b, Sq, Hq, D], lse or None).

    With `summary_pos` (bool [Sq]) the summary rows of k/v form the key prefix, as
    `torch.cat((k[:, summary_pos], k), dim=1)` does in the reference.  For the periodic
    summary layout (every C text rows followed by S summary rows) nothing is copied: the
    kernel reads the prefix rows where they are.  Any other `summary_pos` is gathered into
    a [prefix | in-line] buffer first.  Without `summary_pos`, the first
    `k.shape[1] - q.shape[1]` rows of k/v are taken as an already-built prefix.
    Forward only: tensors that require grad under an enabled grad mode are rejected.
    `return_lse` / `softmax_scale` / `workgroup_shape` are extensions (the reference returns lse
    only for autograd and always uses head_dim ** -0.5; `workgroup_shape` is the tuning knob of
    `PREFILL_SHAPE`).
    """
    _check_inputs(q, k, v)
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        raise NotImplementedError("ksa_amd implements the prefill forward only; call it under torch.no_grad()")
    b, Sq, Hq, D = q.shape
    C, S, W = int(chunk_size), int(summary_num), int(sliding_chunk_num)
    assert C > 0 and S > 0 and W >= 0, "chunk_size/summary_num must be positive, sliding_chunk_num >= 0"
    q, k, v = _lastdim_contig(q), _lastdim_contig(k), _lastdim_contig(v)
    phys = False
    if summary_pos is not None:
        assert k.shape[1] == Sq, "with summary_pos, k/v must have the same length as q"
        P, periodic, rows = _analyse_summary_pos(summary_pos, Sq, C, S)
        if P > 0 and not periodic:
            k, v = _gathered_prefix(k, rows, P), _gathered_prefix(v, rows, P)
            phys = True
    else:
        P = k.shape[1] - Sq
        assert P >= 0, "k/v must be at least as long as q"
        phys = P > 0
    if k.stride() != v.stride():
        v = v.contiguous()
        k = k.contiguous()
    idx = _cached_index(Sq, C, S, W, P, skip_old_summary, q.device)
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    Dk = kernel_head_dim(D)
    if Dk != D:   # a head dimension without a kernel of its own: zero-padded copies (see kernel_head_dim)
        q, k, v = pad_head_dim(q, Dk), pad_head_dim(k, Dk), pad_head_dim(v, Dk)
    out, lse = torch.ops.ksa_amd.summary_attn_fwd(
        q, k, v, idx[0], idx[1], idx[2], idx[3], C, S, W, P,
        bool(skip_old_summary), phys, scale, bool(return_lse),
        PREFILL_SHAPE if workgroup_shape is None else int(workgroup_shape))
    if Dk != D:
        out = out[..., :D].contiguous()
    return out, (lse if return_lse else None)
