"""Drop-in module name of the reference: ``from flash_attention import flash_attention_fn``."""
from triton_flashattn_amd.flash_attention import (  # noqa: F401
    AlibiBias,
    FlashAttentionFn,
    FlashAttentionQKVPackedFn,
    flash_attention_fn,
    flash_attention_op,
    flash_attention_qkvpacked_fn,
)
