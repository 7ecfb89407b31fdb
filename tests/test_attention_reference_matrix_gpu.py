"""The reference's own test matrix for its attention (tests/test_flash_attention_triton.py:26-173) at its own size:
seqlen 3072, head_dim 128, [batch, seqlen, nheads, headdim] tensors, dtype x causal x (batch, heads) x bias shape x
all-masking bias x dropout 0.17 x multi-query K/V, forward and backward, with its criterion (:132-142): the error of O,
dQ, dK and dV against the fp32 evaluation must not exceed twice the error of an evaluation in the operand dtype with
the operations reordered (attention_ref.py:41-73 with upcast=False, reorder_ops=True, restated below and run with torch
on the GPU, as the reference runs it). The fp32 evaluation is the CPU oracle.

The reference's 800 cases are sampled: 18 cases that take every value of every axis at least twice and every bias shape
with and without causal masking, dropout and multi-query K/V. Cases with 32 batch elements run whole on the GPU and are
checked on their first and last batch elements (the dropout indices of a batch element follow from the generator
offset, so a slice has a well-defined mask).
"""
import math

import pytest
import torch

from fast_ops.flash_attention.flash_attention_triton import flash_attn_triton as flash_attn, triton_dropout_mask as dropout_mask
from oracle.attention_oracle import attention_bwd_oracle, attention_fwd_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
S, D = 3072, 128
F16, BF16 = torch.float16, torch.bfloat16

#        dtype causal (B, H)   bias    mask_all dropout multi_query
CASES = [
    (F16, False, (1, 1), None, False, 0.0, False),
    (BF16, True, (1, 1), "1hqk", False, 0.17, True),
    (F16, True, (1, 4), "1h1k", False, 0.17, True),
    (BF16, False, (1, 4), None, False, 0.0, True),
    (BF16, True, (1, 4), None, False, 0.17, False),
    (F16, False, (1, 4), "b1qk", False, 0.17, False),
    (F16, True, (1, 12), "1hqk", False, 0.0, False),
    (BF16, False, (1, 12), "1h1k", False, 0.17, True),
    (BF16, True, (1, 12), "b1qk", False, 0.0, True),
    (F16, False, (1, 12), "b11k", False, 0.0, False),
    (BF16, False, (32, 1), "b11k", False, 0.17, False),
    (F16, True, (32, 1), None, False, 0.0, True),
    (F16, False, (32, 4), "b1qk", False, 0.0, True),
    (BF16, True, (32, 4), "1h1k", False, 0.17, False),
    (F16, True, (1, 4), "b11k", False, 0.17, True),
    (BF16, False, (1, 1), "1hqk", False, 0.0, False),
    # a bias of -inf everywhere: every row's softmax is 0/0. attention_ref.py:59 gives NaN and the reference's comparison
    # of NaN with NaN passes vacuously (:134-141); here the outputs must be NaN like the oracle's, not anything finite
    (F16, False, (1, 4), "1h1k", True, 0.0, False),
    (BF16, True, (1, 1), "b1qk", True, 0.17, True),
]
IDS = [f"{str(c[0])[6:]}-{'causal' if c[1] else 'full'}-b{c[2][0]}h{c[2][1]}-{c[3]}{'-allmasked' if c[4] else ''}-p{c[5]}{'-mq' if c[6] else ''}" for c in CASES]


def _same_dtype_reordered(q, k, v, bias, causal, keep, dropout_p):
    """attention_ref(..., upcast=False, reorder_ops=True) of the reference (attention_ref.py:41-73): everything in the
    operand dtype, K scaled instead of Q. [B, S, H, D] tensors; returns the output."""
    d = q.shape[-1]
    scores = torch.einsum("bthd,bshd->bhts", q, k / math.sqrt(d))
    if bias is not None:
        scores = (scores + bias).to(dtype=scores.dtype)
    if causal:
        scores = scores.masked_fill(torch.triu(torch.ones(q.shape[1], k.shape[1], dtype=torch.bool, device=q.device), 1), float("-inf"))
    attention = torch.softmax(scores, dim=-1)
    if keep is not None:
        attention = attention.masked_fill(~keep, 0.0)
    return torch.einsum("bhts,bshd->bthd", attention, v * (1.0 / (1 - dropout_p)))


@pytest.mark.parametrize("case", CASES, ids=IDS)
def test_reference_matrix_case(case):
    dtype, causal, (B, H), bias_shape, mask_all, dropout_p, multi_query = case
    g = torch.Generator().manual_seed(0)
    Hk = 1 if multi_query else H
    q = torch.randn(B, S, H, D, generator=g).to(dtype)
    k1, v1 = torch.randn(B, S, 2, Hk, D, generator=g).to(dtype).unbind(dim=2)      # :68-73
    go = torch.randn(B, S, H, D, generator=g).to(dtype)
    bias = None
    if bias_shape is not None:
        shape = {"1h1k": (1, H, 1, S), "1hqk": (1, H, S, S), "b11k": (B, 1, 1, S), "b1qk": (B, 1, S, S)}[bias_shape]   # :74-84
        bias = torch.randn(shape, generator=g)
        if mask_all:
            bias.fill_(float("-inf"))                                                      # :86-87
    seed, offset = 20231, 4 * 977
    qd = q.to(DEV).requires_grad_(True)
    k1d, v1d = k1.to(DEV).requires_grad_(True), v1.to(DEV).requires_grad_(True)
    kd, vd = k1d.expand(B, S, H, D), v1d.expand(B, S, H, D)
    bias_d = None if bias is None else bias.to(DEV)
    o, lse = flash_attn(qd, kd, vd, bias=bias_d, causal=causal, dropout_p=dropout_p, return_lse=True,
                        dropout_state=(seed, offset) if dropout_p > 0 else None)
    dq, dk, dv = torch.autograd.grad(o, (qd, k1d, v1d), go.to(DEV))
    torch.cuda.synchronize()
    if mask_all:
        assert bool(torch.isnan(o.float()).all()), "every key of every row is masked: softmax is 0/0 (attention_ref.py:59)"
        return
    failed = []
    for b in sorted({0, B - 1}):
        sl = slice(b, b + 1)
        # the dropout index of (b, h, q, key) is offset + ((b*H + h)*S + q)*S + key: batch element b alone starts b*H*S*S later
        off_b = (offset + b * H * S * S) % (1 << 32)
        drop = (dropout_p, seed, off_b) if dropout_p > 0 else None
        bias_b = None if bias is None else (bias[sl] if bias.shape[0] == B else bias)
        to_bhsd = lambda t: t[sl].transpose(1, 2)
        qb, kb, vb, gb = to_bhsd(q), to_bhsd(k1.expand(B, S, H, D)), to_bhsd(v1.expand(B, S, H, D)), to_bhsd(go)
        o_ref, lse_ref = attention_fwd_oracle(qb, kb, vb, causal=causal, dropout=drop, bias=bias_b)
        dq_ref, dk_ref, dv_ref = attention_bwd_oracle(qb, kb, vb, gb, causal=causal, dropout=drop, bias=bias_b)
        if multi_query:
            dk_ref, dv_ref = dk_ref.sum(dim=1, keepdim=True), dv_ref.sum(dim=1, keepdim=True)
        # the yardstick: the same expression in the operand dtype (torch on the GPU), under the same dropout mask
        keep = dropout_mask(dropout_p, 1, H, S, S, DEV, dropout_state=(seed, off_b)) if dropout_p > 0 else None
        qp, kp, vp = (t[sl].detach().clone().requires_grad_(True) for t in (qd, k1d, v1d))
        o_pt = _same_dtype_reordered(qp, kp.expand(1, S, H, D), vp.expand(1, S, H, D), None if bias_b is None else bias_b.to(DEV), causal, keep, dropout_p)
        dq_pt, dk_pt, dv_pt = torch.autograd.grad(o_pt, (qp, kp, vp), go[sl].to(DEV))
        bshd = lambda t: t.transpose(1, 2)                     # oracle results [1, H, S, D] -> [1, S, H, D]
        for name, mine, pt, ref in (("out", o[sl], o_pt, bshd(o_ref)), ("dQ", dq[sl], dq_pt, bshd(dq_ref)),
                                    ("dK", dk[sl], dk_pt, bshd(dk_ref)), ("dV", dv[sl], dv_pt, bshd(dv_ref))):
            err = (mine.detach().float().cpu() - ref).abs().max().item()
            err_pt = (pt.detach().float().cpu() - ref).abs().max().item()
            if not (math.isfinite(err) and err <= 2 * err_pt):                       # :132-141
                failed.append(f"{name}[b={b}]: error {err:.3e} > 2 x {err_pt:.3e}")
        lse_err = (lse[sl].cpu() - lse_ref).abs().max().item()
        if not lse_err <= 1e-3:
            failed.append(f"LSE[b={b}]: error {lse_err:.3e}")
    assert not failed, failed
