"""FlashAttention forward for MI355X: drop-in for ``fast_ops.flash_attention.flash_attention``.

``multi_head_attention(Q, K, V)`` keeps the reference call (fast_ops/flash_attention/flash_attention.py:48-77):
[B, H, M, D] queries, [B, H, N, D] keys and values, fp16 or bf16, returns [B, H, M, D]. The reference's CUDA kernel
behind that call is unfinished and returns zeros (flash_attention_fwd.cu:120-151,158); this one computes
softmax(scale * Q K^T + mask) V with the numerics of the reference's working Triton forward
(flash_attention_triton.py:128-255) and can return the logsumexp that forward also produces (:255,771).

Keyword-only extras that the reference's README promises or its Triton surface already has
(flash_attention/README.md:34-38, flash_attention_triton.py:722-731): ``causal``, ``softmax_scale``, ``return_lse``.
``flash_attn`` is the [B, S, H, D] surface of ``flash_attn_triton`` without bias and dropout.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional, Tuple, Union

import torch
from torch import Tensor
from torch.autograd import Function

from .. import _lib

_DTYPE_CODE = {torch.float16: _lib.FO_DTYPE_F16, torch.bfloat16: _lib.FO_DTYPE_BF16}
_I64x3 = ctypes.c_int64 * 3


def _check_inputs(q: Tensor, k: Tensor, v: Tensor) -> None:
    # the limits documented at flash_attention.py:61-70; violating them raises, as promised there
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise RuntimeError("Q, K and V must be 4-dimensional")
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("All tensors must have the same type")
    if q.dtype not in _DTYPE_CODE:
        raise RuntimeError("Inputs must be half-precision floating points (float16 and bfloat16)")
    if not (q.is_cuda and k.is_cuda and v.is_cuda) or not (q.device == k.device == v.device):
        raise RuntimeError("Q, K and V must be GPU tensors on the same device (there is no CPU path)")
    if q.stride(-1) != 1 or k.stride(-1) != 1 or v.stride(-1) != 1:
        raise RuntimeError("The last dimension of Q, K and V must be contiguous")


def attn_fwd_strided(
    q: Tensor, k: Tensor, v: Tensor, dims: Tuple[int, int, int, int], causal: bool, softmax_scale: Optional[float]
) -> Tuple[Tensor, Tensor]:
    """Launches fo_attn_fwd. ``dims`` = positions of (batch, head, sequence, head_dim) in the tensors' shapes.
    Returns (O with q's shape, dtype and layout; LSE fp32 [B, H, Sq])."""
    _check_inputs(q, k, v)
    ib, ih, is_, id_ = dims
    B, H, Sq, D = q.shape[ib], q.shape[ih], q.shape[is_], q.shape[id_]
    Sk = k.shape[is_]
    if k.shape[ib] != B or k.shape[ih] != H or k.shape[id_] != D or v.shape != k.shape:
        raise RuntimeError(f"shape mismatch: Q {tuple(q.shape)}, K {tuple(k.shape)}, V {tuple(v.shape)}")
    if D > 128:
        raise RuntimeError("FlashAttention only support head dimensions up to 128")  # flash_attention_triton.py:745
    if D % 8 != 0:
        raise RuntimeError("head_dim must be a multiple of 8")                        # flash_attention.py:65-66
    scale = float(softmax_scale) if softmax_scale else 1.0 / math.sqrt(D)             # flash_attention_triton.py:750
    if D not in (64, 128):
        # The kernels exist for head_dim 64 and 128. Any other multiple of 8 (the reference's contract,
        # flash_attention.py:61-66) runs on zero-padded copies: padded columns add nothing to Q K^T, and the padded
        # columns of V only produce output columns that are dropped; the scale stays that of the true head_dim.
        Dp = 64 if D < 64 else 128
        pad = lambda t: torch.nn.functional.pad(t, (0, Dp - D))
        o_p, lse = attn_fwd_strided(pad(q), pad(k), pad(v), dims, causal, scale)
        o = torch.empty_like(q)
        o.copy_(o_p.narrow(id_, 0, D))
        return o, lse
    o = torch.empty_like(q)
    if o.stride() != q.stride():   # empty_like keeps dense layouts; anything else gets a plain contiguous output
        o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    strides = lambda t: _I64x3(t.stride(ib), t.stride(ih), t.stride(is_))
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        status = _lib.load().fo_attn_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
            B, H, Sq, Sk, D, strides(q), strides(k), strides(v), strides(o),
            scale, int(bool(causal)), _DTYPE_CODE[q.dtype], stream,
        )
    _lib.check(status, "fo_attn_fwd")
    return o, lse


class FlashAttentionFunction(Function):
    @staticmethod
    def forward(ctx, Q: Tensor, K: Tensor, V: Tensor, causal: bool = False, softmax_scale: Optional[float] = None,
                return_lse: bool = False):
        """
        :param Q: (B, H, M, D) Query tensor.
        :param K: (B, H, N, D) Key tensor.
        :param V: (B, H, N, D) Value tensor.
        :returns: (B, H, M, D), and the (B, H, M) fp32 logsumexp when ``return_lse``
        """
        o, lse = attn_fwd_strided(Q, K, V, (0, 1, 2, 3), causal, softmax_scale)
        ctx.save_for_backward(Q, K, V, o, lse)   # what a backward pass needs (flash_attention_triton.py:826)
        ctx.causal = causal
        ctx.softmax_scale = softmax_scale
        if return_lse:
            ctx.mark_non_differentiable(lse)
            return o, lse
        return o

    @staticmethod
    def backward(ctx, *grads):
        """:param dO: (B, H, M, D) Output gradient. Not implemented, as in the reference (flash_attention.py:40-45)."""
        raise NotImplementedError


def multi_head_attention(
    Q: Tensor, K: Tensor, V: Tensor, *, causal: bool = False, softmax_scale: Optional[float] = None, return_lse: bool = False
) -> Union[Tensor, Tuple[Tensor, Tensor]]:
    """FlashAttention forward (https://arxiv.org/abs/2205.14135), B = batch, H = heads, M = queries, N = keys, D = head dim.

    Limitations (violations raise RuntimeError): head_dim a multiple of 8 up to 128 (64 and 128 run in place, the others
    on zero-padded copies); the last dimension of Q, K, V contiguous and rows 16-byte aligned; inputs float16 or
    bfloat16; GPU tensors.

    :param Q: (B, H, M, D) Query tensor.
    :param K: (B, H, N, D) Key tensor.
    :param V: (B, H, N, D) Value tensor.
    :param causal: query i attends keys j <= i
    :param softmax_scale: multiplier of Q K^T, default 1/sqrt(D)
    :param return_lse: also return the (B, H, M) fp32 logsumexp of the scaled scores
    :returns: (B, H, M, D)
    """
    return FlashAttentionFunction.apply(Q, K, V, causal, softmax_scale, return_lse)


def flash_attn(
    q: Tensor, k: Tensor, v: Tensor, bias: Optional[Tensor] = None, causal: bool = False, dropout_p: float = 0.0,
    softmax_scale: Optional[float] = None, return_lse: bool = False,
) -> Union[Tensor, Tuple[Tensor, Tensor]]:
    """The [batch, seqlen, nheads, headdim] surface of flash_attn_triton (flash_attention_triton.py:722-737,961),
    forward only. Bias and dropout are not implemented and raise."""
    if bias is not None:
        raise RuntimeError("attention bias is not implemented")
    if dropout_p != 0.0:
        raise RuntimeError("attention dropout is not implemented")
    o, lse = attn_fwd_strided(q, k, v, (0, 2, 1, 3), causal, softmax_scale)
    return (o, lse) if return_lse else o
