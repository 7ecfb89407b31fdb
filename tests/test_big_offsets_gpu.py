"""Attention forward and backward on operands of more than 4 GiB each: every (batch, head) base offset beyond 2^32
bytes has to come out of 64-bit arithmetic (the reference's launcher has the same kind of trap in its Lion kernel,
`int numel`: lion_update.cu:130,143). Checked against the CPU oracle on the first and the last (batch, head) slice and
on the slices either side of the 2^32-byte offset; tolerances as everywhere else (O atol 2e-2 / rtol 1e-2, LSE 1e-3;
gradients within 2 % of the gradient's largest magnitude, the criterion of the other full-size backward tests).
Inputs are drawn on the device (the slices that are checked are copied back for the oracle)."""
import ctypes
import math

import pytest
import torch

from fast_ops.flash_attention.flash_attention import multi_head_attention
from fast_ops_amd import _lib
from oracle.attention_oracle import attention_bwd_oracle, attention_fwd_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
O_ATOL, O_RTOL, LSE_ATOL = 2e-2, 1e-2, 1e-3


def _kernel_taken(B, H, S, D, k, v, causal):
    I3 = ctypes.c_int64 * 3
    return _lib.load().fo_attn_fwd_kernel(B, H, S, S, D, I3(*k.stride()[:3]), I3(*v.stride()[:3]), int(causal), 0, 0)


def _run(B, H, S, D, causal, expect_kernel, seed):
    gen = torch.Generator(device=DEV).manual_seed(seed)
    shape = (B, H, S, D)
    q, k, v, go = (torch.empty(shape, device=DEV, dtype=torch.bfloat16).normal_(generator=gen) for _ in range(4))
    nbytes = q.numel() * 2
    assert nbytes > (1 << 32)
    assert _kernel_taken(B, H, S, D, k, v, causal) == expect_kernel
    slice_bytes = S * D * 2
    cross = (1 << 32) // slice_bytes                   # the first (batch, head) slice that starts at or beyond byte 2^32
    picks = sorted({0, cross - 1, cross, cross + 1, B * H - 1})
    print(f"\n  B={B} H={H} S={S} D={D}: {nbytes / 2**30:.2f} GiB per operand, slices {picks}", flush=True)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    o, lse = multi_head_attention(q, k, v, causal=causal, return_lse=True)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), go)
    torch.cuda.synchronize()
    for bh in picks:
        b, h = divmod(bh, H)
        sl = (slice(b, b + 1), slice(h, h + 1))
        qc, kc, vc, gc = (t[sl].detach().cpu() for t in (q, k, v, go))
        o_ref, lse_ref = attention_fwd_oracle(qc, kc, vc, causal=causal)
        err = (o[sl].detach().float().cpu() - o_ref).abs()
        worst = float((err - (O_ATOL + O_RTOL * o_ref.abs())).max())
        assert worst <= 0, f"slice {bh}: O outside tolerance by {worst:.3e}"
        lse_err = float((lse[sl].cpu() - lse_ref).abs().max())
        assert lse_err <= LSE_ATOL, f"slice {bh}: LSE error {lse_err:.3e}"
        ref = attention_bwd_oracle(qc, kc, vc, gc, causal=causal)
        for name, a, r in zip(("dQ", "dK", "dV"), (dq, dk, dv), ref):
            e = (a[sl].float().cpu() - r).abs().max().item()
            assert math.isfinite(e) and e <= 2e-2 * max(1.0, r.abs().max().item()), f"slice {bh} {name}: error {e:.3e} vs magnitude {r.abs().max().item():.3e}"
        print(f"    slice {bh} (byte offset {bh * slice_bytes}): ok", flush=True)


def test_headline_kernel_operands_beyond_4_gib():
    # the benchmark's kernel (256 rows, four waves) and the pipelined dK/dV kernel: 17 x 128 heads of S=8192, D=128
    _run(17, 128, 8192, 128, True, _lib.FO_ATTN_KERNEL_ROWS256_W4, seed=1)


def test_128_row_kernel_operands_beyond_4_gib():
    # the 128-row kernel at head_dim 64: 33 x 1024 heads of S=1024 (270,336 workgroups)
    _run(33, 1024, 1024, 64, True, _lib.FO_ATTN_KERNEL_ROWS128, seed=2)
