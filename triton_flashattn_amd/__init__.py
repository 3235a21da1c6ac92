"""MI355X-native flash attention with an optional trainable bias (HIP kernels behind a C ABI)."""
from .flash_attention import (  # noqa: F401
    FlashAttentionFn,
    FlashAttentionQKVPackedFn,
    flash_attention_fn,
    flash_attention_qkvpacked_fn,
)

__all__ = [
    "FlashAttentionFn",
    "FlashAttentionQKVPackedFn",
    "flash_attention_fn",
    "flash_attention_qkvpacked_fn",
]
