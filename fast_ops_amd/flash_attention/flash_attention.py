"""FlashAttention forward for MI355X: drop-in for ``fast_ops.flash_attention.flash_attention``.

``multi_head_attention(Q, K, V)`` keeps the reference call (fast_ops/flash_attention/flash_attention.py:48-77):
[B, H, M, D] queries, [B, H, N, D] keys and values, fp16 or bf16, returns [B, H, M, D]. The reference's CUDA kernel
behind that call is unfinished and returns zeros (flash_attention_fwd.cu:120-151,158); this one computes
softmax(scale * Q K^T + mask) V with the numerics of the reference's working Triton forward
(flash_attention_triton.py:128-255) and can return the logsumexp that forward also produces (:255,771). The backward
the reference leaves unimplemented (flash_attention.py:40-45) is implemented too, after the Triton backward
(flash_attention_triton.py:832-958), so ``FlashAttentionFunction`` is trainable.

Keyword-only extras that the reference's README promises or its Triton surface already has
(flash_attention/README.md:34-38, flash_attention_triton.py:722-731): ``causal``, ``softmax_scale``, ``return_lse``.
``flash_attn`` is the [B, S, H, D] surface of ``flash_attn_triton``, with its additive bias and its dropout.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional, Tuple, Union

import numpy as np
import torch
from torch import Tensor
from torch.autograd import Function

from .. import _lib

_DTYPE_CODE = {torch.float16: _lib.FO_DTYPE_F16, torch.bfloat16: _lib.FO_DTYPE_BF16}
# the raw hipStream_t that is current on a device, without building a torch.cuda.Stream object around it
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (lambda dev: torch.cuda.current_stream(dev).cuda_stream)
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


Dropout = Tuple[float, int, int]   # (dropout_p, seed, generator offset)


class _AttnExtras(ctypes.Structure):    # fo_attn_extras
    _fields_ = [("bias", ctypes.c_void_p), ("bias_strides", ctypes.c_int64 * 3), ("bias_dtype", ctypes.c_int),
                ("dropout_p", ctypes.c_float), ("dropout_seed", ctypes.c_uint32), ("dropout_offset", ctypes.c_uint64)]


def _expand_bias(bias: Tensor, q: Tensor, B: int, H: int, Sq: int, Sk: int) -> Tensor:
    """The reference's checks and broadcast of the bias (flash_attention_triton.py:752-768): 4-dimensional, the dtype
    of q or fp32, last two dimensions (1, Sk) or (Sq, Sk), expanded (strides of 0) over batch, heads and queries."""
    if bias.dtype not in (q.dtype, torch.float32):
        raise RuntimeError("bias must have the dtype of q or float32")
    if not bias.is_cuda or bias.device != q.device:
        raise RuntimeError("bias must be on the device of q")
    if bias.dim() != 4:
        raise RuntimeError("bias must be 4-dimensional")
    if bias.stride(-1) != 1:
        bias = bias.contiguous()
    if tuple(bias.shape[2:]) not in ((1, Sk), (Sq, Sk)):
        raise RuntimeError("Last 2 dimensions of bias must be (1, seqlen_k) or (seqlen_q, seqlen_k)")
    return bias.expand(B, H, Sq, Sk)


def _extras(bias: Optional[Tensor], dropout: Optional[Dropout]) -> _AttnExtras:
    ex = _AttnExtras()
    if bias is not None:
        ex.bias = bias.data_ptr()
        ex.bias_strides = _I64x3(bias.stride(0), bias.stride(1), bias.stride(2))
        ex.bias_dtype = _lib.FO_DTYPE_F32 if bias.dtype == torch.float32 else _DTYPE_CODE[bias.dtype]
    if dropout is not None:
        ex.dropout_p, ex.dropout_seed, ex.dropout_offset = float(dropout[0]), dropout[1] & 0xFFFFFFFF, dropout[2] % (1 << 64)
    return ex


def next_dropout_state(n_elements: int) -> Tuple[int, int]:
    """(seed, offset) for a dropout mask over ``n_elements`` attention probabilities, taken from torch's generator of the
    current device, whose offset is advanced past them: what increment_philox_state does in the reference
    (flash_attention_triton.py:641-665). The last 16 bytes of the generator state are (seed, offset) as two uint64."""
    state = torch.cuda.get_rng_state()
    words = state.numpy().view(np.uint64)
    seed, offset = int(words[-2]), int(words[-1])
    words[-1] = np.uint64((offset + 4 * math.ceil(n_elements / 4)) % (1 << 64))
    torch.cuda.set_rng_state(state)
    return seed, offset


def dropout_mask(
    dropout_p: float, batch_sz: int, n_heads: int, seqlen_q: int, seqlen_k: int, device: Union[str, torch.device],
    dropout_state: Optional[Tuple[int, int]] = None,
) -> Tensor:
    """The keep-mask (bool [B, H, Sq, Sk], True = kept) that the attention kernels apply for this dropout_p and state:
    triton_dropout_mask of the reference (flash_attention_triton.py:697-717). Without ``dropout_state`` the state comes
    from torch's generator, which is advanced exactly as an attention call of that shape advances it, so seeding, taking
    the mask, seeding again and calling the attention gives the attention's mask (tests/test_flash_attention_triton.py:
    93-103)."""
    if not 0.0 <= dropout_p < 1.0:
        raise RuntimeError(f"dropout_p must be in [0, 1), got {dropout_p}")
    device = torch.device(device)
    n = batch_sz * n_heads * seqlen_q * seqlen_k
    with torch.cuda.device(device):
        seed, offset = dropout_state if dropout_state is not None else next_dropout_state(n)
        keep = torch.empty((batch_sz, n_heads, seqlen_q, seqlen_k), dtype=torch.uint8, device=device)
        status = _lib.load().fo_dropout_mask(keep.data_ptr(), n, float(dropout_p), seed & 0xFFFFFFFF, offset % (1 << 64),
                                             torch.cuda.current_stream(device).cuda_stream)
    _lib.check(status, "fo_dropout_mask")
    return keep.view(torch.bool)


class _FwdPlan:
    """What a forward call of one (shapes, strides, dtype, device, layout) needs besides the data pointers: checked once,
    then reused - the checks, the stride arrays for the C ABI and the sizes cost more host time than a small kernel runs."""
    __slots__ = ("B", "H", "Sq", "Sk", "D", "qs", "ks", "vs", "os", "o_dense_like_q", "dtype_code", "device_index", "lse_shape")


_FWD_PLANS: dict = {}


def _fwd_plan(q: Tensor, k: Tensor, v: Tensor, dims: Tuple[int, int, int, int]) -> _FwdPlan:
    key = (q.shape, q.stride(), k.shape, k.stride(), v.shape, v.stride(), q.dtype, k.dtype, v.dtype, q.device, k.device, v.device, dims)
    plan = _FWD_PLANS.get(key)
    if plan is not None:
        return plan
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
    plan = _FwdPlan()
    plan.B, plan.H, plan.Sq, plan.Sk, plan.D = B, H, Sq, Sk, D
    strides = lambda t: _I64x3(t.stride(ib), t.stride(ih), t.stride(is_))
    plan.qs, plan.ks, plan.vs = strides(q), strides(k), strides(v)
    o = torch.empty_like(q)
    plan.o_dense_like_q = o.stride() == q.stride()    # empty_like keeps dense layouts; anything else gets a plain contiguous output
    if not plan.o_dense_like_q:
        o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    plan.os = strides(o)
    plan.dtype_code = _DTYPE_CODE[q.dtype]
    plan.device_index = q.device.index if q.device.index is not None else torch.cuda.current_device()
    plan.lse_shape = (B, H, Sq)
    if len(_FWD_PLANS) > 4096:
        _FWD_PLANS.clear()
    _FWD_PLANS[key] = plan
    return plan


def attn_fwd_strided(
    q: Tensor, k: Tensor, v: Tensor, dims: Tuple[int, int, int, int], causal: bool, softmax_scale: Optional[float],
    dropout: Optional[Dropout] = None, bias: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """Launches fo_attn_fwd (fo_attn_fwd_dropout when ``dropout`` is given, fo_attn_fwd_ex when ``bias`` is). ``dims`` =
    positions of (batch, head, sequence, head_dim) in the tensors' shapes; ``bias`` is [B|1, H|1, Sq|1, Sk] whatever
    ``dims`` says. Returns (O with q's shape, dtype and layout; LSE fp32 [B, H, Sq])."""
    plan = _fwd_plan(q, k, v, dims)
    scale = float(softmax_scale) if softmax_scale else 1.0 / math.sqrt(plan.D)        # flash_attention_triton.py:750
    o = torch.empty_like(q) if plan.o_dense_like_q else torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty(plan.lse_shape, dtype=torch.float32, device=q.device)
    if bias is not None:
        bias = _expand_bias(bias, q, plan.B, plan.H, plan.Sq, plan.Sk)
    dev = plan.device_index
    lib = _lib.load()
    # (the launch goes to the stream that is current on the tensors' device; the device is made current only when it is not)
    guard = torch.cuda.device(dev) if torch.cuda.current_device() != dev else None
    if guard is not None:
        guard.__enter__()
    try:
        stream = _raw_stream(dev)
        args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                plan.B, plan.H, plan.Sq, plan.Sk, plan.D, plan.qs, plan.ks, plan.vs, plan.os,
                scale, 1 if causal else 0, plan.dtype_code)
        if bias is not None:
            status = lib.fo_attn_fwd_ex(*args, ctypes.byref(_extras(bias, dropout)), stream)
        elif dropout is None or dropout[0] == 0.0:
            status = lib.fo_attn_fwd(*args, stream)
        else:
            status = lib.fo_attn_fwd_dropout(*args, float(dropout[0]), dropout[1] & 0xFFFFFFFF, dropout[2] % (1 << 64), stream)
    finally:
        if guard is not None:
            guard.__exit__(None, None, None)
    if status != 0:
        _lib.check(status, "fo_attn_fwd")
    return o, lse


def attn_bwd_strided(
    q: Tensor, k: Tensor, v: Tensor, o: Tensor, lse: Tensor, d_o: Tensor, dims: Tuple[int, int, int, int], causal: bool,
    softmax_scale: Optional[float], dropout: Optional[Dropout] = None, bias: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Launches fo_attn_bwd. Returns (dQ, dK, dV) with the shapes and dtypes of q, k, v (dense; a K/V whose heads are
    an expanded view gets a full-size gradient, which autograd then reduces)."""
    _check_inputs(q, k, v)
    ib, ih, is_, id_ = dims
    B, H, Sq, D = q.shape[ib], q.shape[ih], q.shape[is_], q.shape[id_]
    Sk = k.shape[is_]
    scale = float(softmax_scale) if softmax_scale else 1.0 / math.sqrt(D)
    if d_o.dtype != q.dtype or d_o.shape != q.shape:
        raise RuntimeError(f"dO must have the output's shape and dtype, got {tuple(d_o.shape)} {d_o.dtype}")
    if d_o.stride(-1) != 1 or any(s % 8 for s in d_o.stride()[:-1]):
        d_o = d_o.contiguous()
    if o.stride(-1) != 1:
        o = o.contiguous()
    lse = lse.contiguous()
    dq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    dk = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    dv = torch.empty(v.shape, dtype=v.dtype, device=v.device)
    delta = torch.empty((2, B, H, Sq), dtype=torch.float32, device=q.device)   # workspace: -delta and -LSE / scale per row
    if bias is not None:
        bias = _expand_bias(bias, q, B, H, Sq, Sk)
    tensors = (q, k, v, o, d_o, dq, dk, dv)
    arrays = [_I64x3(t.stride(ib), t.stride(ih), t.stride(is_)) for t in tensors]
    ptrs = (ctypes.POINTER(ctypes.c_int64) * 8)(*[ctypes.cast(a, ctypes.POINTER(ctypes.c_int64)) for a in arrays])
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, H, Sq, Sk, D, ptrs, scale, int(bool(causal)), _DTYPE_CODE[q.dtype])
        if bias is not None:
            status = _lib.load().fo_attn_bwd_ex(*args, ctypes.byref(_extras(bias, dropout)), stream)
        elif dropout is None or dropout[0] == 0.0:
            status = _lib.load().fo_attn_bwd(*args, stream)
        else:
            status = _lib.load().fo_attn_bwd_dropout(*args, float(dropout[0]), dropout[1] & 0xFFFFFFFF, dropout[2] % (1 << 64), stream)
    _lib.check(status, "fo_attn_bwd")
    return dq, dk, dv


class FlashAttentionFunction(Function):
    @staticmethod
    def forward(ctx, Q: Tensor, K: Tensor, V: Tensor, causal: bool = False, softmax_scale: Optional[float] = None,
                return_lse: bool = False, dropout: Optional[Dropout] = None):
        """
        :param Q: (B, H, M, D) Query tensor.
        :param K: (B, H, N, D) Key tensor.
        :param V: (B, H, N, D) Value tensor.
        :returns: (B, H, M, D), and the (B, H, M) fp32 logsumexp when ``return_lse``
        """
        o, lse = attn_fwd_strided(Q, K, V, (0, 1, 2, 3), causal, softmax_scale, dropout)
        ctx.save_for_backward(Q, K, V, o, lse)   # what a backward pass needs (flash_attention_triton.py:826)
        ctx.causal = causal
        ctx.softmax_scale = softmax_scale
        ctx.dropout = dropout                    # (p, seed, offset): the backward regenerates the mask (:824-828)
        if return_lse:
            ctx.mark_non_differentiable(lse)
            return o, lse
        return o

    @staticmethod
    def backward(ctx, dO: Tensor, *unused):
        """:param dO: (B, H, M, D) Output gradient. The reference leaves this unimplemented (flash_attention.py:40-45);
        here it is what the reference's Triton backward computes (flash_attention_triton.py:832-958)."""
        Q, K, V, o, lse = ctx.saved_tensors
        dq, dk, dv = attn_bwd_strided(Q, K, V, o, lse, dO, (0, 1, 2, 3), ctx.causal, ctx.softmax_scale, ctx.dropout)
        return dq, dk, dv, None, None, None, None


class _FlashAttnBSHD(Function):
    """flash_attn's autograd node: the same kernels on [batch, seqlen, nheads, headdim] tensors."""

    @staticmethod
    def forward(ctx, q: Tensor, k: Tensor, v: Tensor, causal: bool, softmax_scale: Optional[float], return_lse: bool,
                dropout: Optional[Dropout], bias: Optional[Tensor] = None):
        o, lse = attn_fwd_strided(q, k, v, (0, 2, 1, 3), causal, softmax_scale, dropout, bias)
        ctx.save_for_backward(q, k, v, o, lse, bias)
        ctx.causal = causal
        ctx.softmax_scale = softmax_scale
        ctx.dropout = dropout
        if return_lse:
            ctx.mark_non_differentiable(lse)
            return o, lse
        return o

    @staticmethod
    def backward(ctx, dO: Tensor, *unused):
        q, k, v, o, lse, bias = ctx.saved_tensors
        if bias is not None and ctx.needs_input_grad[7]:
            raise RuntimeError("FlashAttention does not support bias gradient yet")   # flash_attention_triton.py:854
        dq, dk, dv = attn_bwd_strided(q, k, v, o, lse, dO, (0, 2, 1, 3), ctx.causal, ctx.softmax_scale, ctx.dropout, bias)
        return dq, dk, dv, None, None, None, None, None


def _dropout_arg(dropout_p: float, dropout_state: Optional[Tuple[int, int]], n_elements: int) -> Optional[Dropout]:
    if dropout_p == 0.0:
        return None
    if not 0.0 <= dropout_p < 1.0:
        raise RuntimeError(f"dropout_p must be in [0, 1), got {dropout_p}")
    seed, offset = dropout_state if dropout_state is not None else next_dropout_state(n_elements)
    return (float(dropout_p), int(seed), int(offset))


def multi_head_attention(
    Q: Tensor, K: Tensor, V: Tensor, *, causal: bool = False, softmax_scale: Optional[float] = None, return_lse: bool = False,
    dropout_p: float = 0.0, dropout_state: Optional[Tuple[int, int]] = None,
) -> Union[Tensor, Tuple[Tensor, Tensor]]:
    """FlashAttention forward (https://arxiv.org/abs/2205.14135), B = batch, H = heads, M = queries, N = keys, D = head dim.

    Limitations (violations raise RuntimeError): head_dim a multiple of 8 up to 128; the last dimension of Q, K, V contiguous and rows 16-byte aligned; inputs float16 or
    bfloat16; GPU tensors.

    :param Q: (B, H, M, D) Query tensor.
    :param K: (B, H, N, D) Key tensor.
    :param V: (B, H, N, D) Value tensor.
    :param causal: query i attends keys j <= i
    :param softmax_scale: multiplier of Q K^T, default 1/sqrt(D)
    :param return_lse: also return the (B, H, M) fp32 logsumexp of the scaled scores
    :param dropout_p: probability of dropping an attention probability (flash_attention_triton.py:216-219)
    :param dropout_state: (seed, offset) of the mask; default: taken from torch's generator, which is advanced
    :returns: (B, H, M, D)
    """
    drop = None if dropout_p == 0.0 else _dropout_arg(dropout_p, dropout_state, Q.shape[0] * Q.shape[1] * Q.shape[2] * K.shape[2])
    if not (torch.is_grad_enabled() and (Q.requires_grad or K.requires_grad or V.requires_grad)):
        # nothing to differentiate: no autograd node (its bookkeeping costs more host time than a small kernel runs)
        o, lse = attn_fwd_strided(Q, K, V, (0, 1, 2, 3), causal, softmax_scale, drop)
        return (o, lse) if return_lse else o
    return FlashAttentionFunction.apply(Q, K, V, causal, softmax_scale, return_lse, drop)


def flash_attn(
    q: Tensor, k: Tensor, v: Tensor, bias: Optional[Tensor] = None, causal: bool = False, dropout_p: float = 0.0,
    softmax_scale: Optional[float] = None, return_lse: bool = False, dropout_state: Optional[Tuple[int, int]] = None,
) -> Union[Tensor, Tuple[Tensor, Tensor]]:
    """The [batch, seqlen, nheads, headdim] surface of flash_attn_triton (flash_attention_triton.py:722-737,961),
    differentiable in q, k and v, with dropout and with an additive bias on the scaled scores: [B|1, H|1, 1, seqlen_k]
    or [B|1, H|1, seqlen_q, seqlen_k], the dtype of q or fp32 (:752-768). A bias that requires grad makes the backward
    raise, as in the reference (:854)."""
    drop = None if dropout_p == 0.0 else _dropout_arg(dropout_p, dropout_state, q.shape[0] * q.shape[2] * q.shape[1] * k.shape[1])
    if not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad or (bias is not None and bias.requires_grad))):
        o, lse = attn_fwd_strided(q, k, v, (0, 2, 1, 3), causal, softmax_scale, drop, bias)
        return (o, lse) if return_lse else o
    return _FlashAttnBSHD.apply(q, k, v, causal, softmax_scale, return_lse, drop, bias)
