"""MI355X (gfx950) fused RoPE flash-attention and Co-RoPE GQA forward.

The directory name carries a hyphen; import the package as ``corope_amd`` (a one-file alias module at the
repository root) or with ``importlib.import_module("co-rope_amd")``."""
from . import _lib
from .corope_gqa import attention as corope_attention
from .corope_gqa import corope_attn_gqa
from .freqs import precompute_freqs_cis, rope_freqs_device
from .rope_attn import attention, fused_rope_attn, rope_attn_forward_with_lse, rope_rotate

__all__ = ["attention", "fused_rope_attn", "rope_attn_forward_with_lse", "rope_rotate", "corope_attention", "corope_attn_gqa",
           "precompute_freqs_cis", "rope_freqs_device", "_lib"]
