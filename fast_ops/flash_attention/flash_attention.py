"""``fast_ops.flash_attention.flash_attention`` - same names as the reference module of that path."""
from fast_ops_amd.flash_attention.flash_attention import (  # noqa: F401
    FlashAttentionFunction,
    flash_attn,
    multi_head_attention,
)
