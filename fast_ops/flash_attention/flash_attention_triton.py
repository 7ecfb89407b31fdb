"""``fast_ops.flash_attention.flash_attention_triton`` - the names the reference module of that path exports
(flash_attention_triton.py:641,697,961), served by the HIP kernels."""
from fast_ops_amd.flash_attention.flash_attention import (  # noqa: F401
    dropout_mask as triton_dropout_mask,
    flash_attn as flash_attn_triton,
    next_dropout_state as increment_philox_state,
)
