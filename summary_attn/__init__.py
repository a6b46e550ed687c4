"""Drop-in for the reference's `summary_attn` package on MI355X: the HF template does
`from summary_attn import summary_attn_func` (modeling_qwen3sa.py:52) and muse imports it
lazily (muse/layers/summary_attention_func.py:28-34); both get the HIP implementation."""
from ksa_amd.prefill import summary_attn_func

__all__ = ["summary_attn_func"]
