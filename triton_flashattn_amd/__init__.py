"""MI355X-native flash attention with an optional trainable bias (HIP kernels behind a C ABI)."""
from .flash_attention import (  # noqa: F401
    AlibiBias,
    FlashAttentionFn,
    FlashAttentionQKVPackedFn,
    flash_attention_fn,
    flash_attention_op,
    flash_attention_qkvpacked_fn,
)

__all__ = [
    "AlibiBias",
    "FlashAttentionFn",
    "FlashAttentionQKVPackedFn",
    "flash_attention_fn",
    "flash_attention_op",
    "flash_attention_qkvpacked_fn",
]
