from .flash_attention import FlashAttentionFunction, flash_attn, multi_head_attention  # noqa: F401
