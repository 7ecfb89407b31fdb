"""Seeded random sweep over the attention paths: every case draws a shape (ragged lengths on both sides of the tile
sizes, 1 to 17 heads so that the workgroup orders with and without XCD grouping are taken), head_dim, dtype, mask,
multi-query K/V, a bias kind (flash_attention_triton.py:752-768) and dropout, runs forward and backward through the
[B,S,H,D] surface and checks O, LSE, dQ, dK, dV against the oracle: O within atol 2e-2 / rtol 1e-2, LSE within 1e-3,
gradients within 2 % of their largest magnitude."""
import random

import pytest
import torch

from fast_ops.flash_attention.flash_attention import flash_attn
from fast_ops_amd import _lib
from oracle.attention_oracle import attention_bwd_oracle, attention_fwd_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
O_ATOL, O_RTOL, LSE_ATOL = 2e-2, 1e-2, 1e-3
LENGTHS = [1, 7, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 191, 200, 256, 257, 320, 383, 450, 512, 640, 777]
BIAS_KINDS = [None, None, "1h1k", "1hqk", "b11k", "b1qk", "bhqk", "111k", "11qk"]


def _case(seed):
    r = random.Random(seed)
    B, H = r.choice([1, 2, 3]), r.choice([1, 2, 3, 4, 5, 8, 16, 17])
    Sq, Sk = r.choice(LENGTHS), r.choice(LENGTHS)
    causal = r.random() < 0.5
    if causal and r.random() < 0.7:
        Sk = Sq                                   # the usual causal case; unequal lengths stay in the mix
    return dict(B=B, H=H, Sq=Sq, Sk=Sk, D=r.choice([64, 128]), dtype=r.choice([torch.bfloat16, torch.float16]), causal=causal,
                multi_query=r.random() < 0.2, bias=r.choice(BIAS_KINDS), bias_f32=r.random() < 0.5,
                dropout=r.choice([0.0, 0.0, 0.1, 0.5]), scale=r.choice([None, None, 0.05, 0.3]),
                # forward kernel (attn.variant): the library's choice, the 128-row kernel, the 256-row kernel with eight or
                # four waves (drawn last, so that the other draws of a seed stay what they were; dropout and a bias with a
                # query stride run on the 128-row kernel whatever is asked, a per-key bias on the forms that exist for it)
                variant=r.choice([-1, 0, 8, 8, 16, 16, 32, 32]))


@pytest.mark.parametrize("seed", range(96))
def test_random_case(seed):
    c = _case(seed)
    B, H, Sq, Sk, D, dtype = c["B"], c["H"], c["Sq"], c["Sk"], c["D"], c["dtype"]
    g = torch.Generator().manual_seed(1000 + seed)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    go = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    Hk = 1 if c["multi_query"] else H
    k1 = torch.randn(B, Hk, Sk, D, generator=g).to(dtype)
    v1 = torch.randn(B, Hk, Sk, D, generator=g).to(dtype)
    k, v = k1.expand(B, H, Sk, D), v1.expand(B, H, Sk, D)      # multi-query: every head reads the same K and V (stride 0)
    bias = None
    if c["bias"] is not None:
        kind = c["bias"]
        shape = (B if kind[0] == "b" else 1, H if kind[1] == "h" else 1, Sq if kind[2] == "q" else 1, Sk)
        bias = (torch.randn(shape, generator=g) * 2.0).to(torch.float32 if c["bias_f32"] else dtype)
    drop = (c["dropout"], 12345 + seed, 4 * seed) if c["dropout"] > 0 else None
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=c["causal"], softmax_scale=c["scale"], dropout=drop, bias=bias)
    ref = attention_bwd_oracle(q, k, v, go, causal=c["causal"], softmax_scale=c["scale"], dropout=drop, bias=bias)
    if c["multi_query"]:
        ref = (ref[0], ref[1].sum(dim=1, keepdim=True), ref[2].sum(dim=1, keepdim=True))

    qd = q.to(DEV).transpose(1, 2).requires_grad_(True)                                  # [B,S,H,D] views
    kd1, vd1 = k1.to(DEV).requires_grad_(True), v1.to(DEV).requires_grad_(True)
    kd, vd = kd1.expand(B, H, Sk, D).transpose(1, 2), vd1.expand(B, H, Sk, D).transpose(1, 2)
    _lib.tune_set("attn.variant", c["variant"])
    try:
        o, lse = flash_attn(qd, kd, vd, bias=None if bias is None else bias.to(DEV), causal=c["causal"], dropout_p=c["dropout"],
                            softmax_scale=c["scale"], return_lse=True, dropout_state=None if drop is None else (drop[1], drop[2]))
    finally:
        _lib.tune_set("attn.variant", -1)
    dq, dk, dv = torch.autograd.grad(o, (qd, kd1, vd1), go.to(DEV).transpose(1, 2))
    torch.cuda.synchronize()
    what = str({k_: v_ for k_, v_ in c.items()})
    err = (o.detach().transpose(1, 2).float().cpu() - o_ref).abs()
    # rows whose every key is masked away (causal with more queries than keys never does that; a bias of -inf would) do
    # not occur here, so everything is finite
    assert torch.isfinite(err).all(), what
    assert float((err - (O_ATOL + O_RTOL * o_ref.abs())).max()) <= 0, f"O: max abs err {float(err.max()):.3e} {what}"
    assert float((lse.detach().cpu() - lse_ref).abs().max()) <= LSE_ATOL, what
    for name, a, r_ in zip(("dQ", "dK", "dV"), (dq.transpose(1, 2), dk, dv), ref):
        e = (a.float().cpu() - r_).abs().max().item()
        assert e <= 2e-2 * max(1.0, r_.abs().max().item()), f"{name}: error {e:.3e} vs magnitude {r_.abs().max().item():.3e} {what}"
