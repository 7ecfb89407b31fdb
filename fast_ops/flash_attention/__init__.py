from fast_ops_amd.flash_attention import FlashAttentionFunction, flash_attn, multi_head_attention  # noqa: F401
