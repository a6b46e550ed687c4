"""ksa_amd — MI355X (gfx950) kernels for the two attention hot paths of Kwai Summary
Attention: the block-sparse prefill forward and decode over the ring-buffer KV cache,
plus the fused pre-attention step (q/k RMSNorm + rotary embedding + layout write) in front of them
and the end-to-end decoder (`model`) that calls all of them.

Importing the package loads libksa_hip.so (built by `python ksa_amd/build.py`); if it is
missing the import fails — there is no other execution path.
"""
from ._lib import KsaError, lib as _load

_load()

from .prefill import SUMMARY_ATTN_CACHE, compute_block_sparsity, summary_attn_func  # noqa: E402
from .decode import (decode_attention_forward, eager_attention_forward, ksa_decode, ksa_decode_boundary,  # noqa: E402
                     ksa_decode_weights)
from .cache import Qwen3RingBufferCache  # noqa: E402
from . import ops  # noqa: E402  (registers torch.ops.ksa_amd.* for the helper operators)
from .ops import add_rmsnorm, linear_rows, pre_attention, silu_mul  # noqa: E402
from .model import KsaQwen3Config, KsaQwen3ForCausalLM, init_weights  # noqa: E402

__all__ = [
    "KsaError", "SUMMARY_ATTN_CACHE", "compute_block_sparsity", "summary_attn_func",
    "decode_attention_forward", "eager_attention_forward", "ksa_decode", "ksa_decode_boundary", "ksa_decode_weights", "Qwen3RingBufferCache", "pre_attention", "add_rmsnorm", "silu_mul", "linear_rows", "ops",
    "KsaQwen3Config", "KsaQwen3ForCausalLM", "init_weights",
]
