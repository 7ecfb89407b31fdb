"""Pins the attention oracle (oracle/attention_oracle.py) on the CPU.

The reference has no golden vectors for this path (tests/test_flash_attention.py asserts nothing,
tests/test_flash_attention_triton.py:104-142 is differential), so the oracle is pinned against an independent
library routine (scaled_dot_product_attention, logsumexp), a float64 brute force, closed-form invariants, the
reference's tile recurrence restated in numpy, and the committed fixture tests/golden/attn_small.npz.
"""
import math
import os

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from oracle.attention_oracle import attention_fwd_oracle, online_softmax_tiles

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "attn_small.npz")


def _qkv(B, H, M, N, D, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, M, D, generator=g).to(dtype)
    k = torch.randn(B, H, N, D, generator=g).to(dtype)
    v = torch.randn(B, H, N, D, generator=g).to(dtype)
    return q, k, v


def _brute_force(q, k, v, causal, scale):
    """float64 loops straight from the definition: O_i = sum_j softmax_j(scale q_i.k_j) v_j over allowed j."""
    q, k, v = (t.double().numpy() for t in (q, k, v))
    B, H, M, D = q.shape
    N = k.shape[2]
    o = np.zeros((B, H, M, D))
    lse = np.zeros((B, H, M))
    for b in range(B):
        for h in range(H):
            for i in range(M):
                js = [j for j in range(N) if (not causal) or j <= i]
                s = np.array([scale * float(np.dot(q[b, h, i], k[b, h, j])) for j in js])
                mx = s.max()
                w = np.exp(s - mx)
                lse[b, h, i] = mx + math.log(w.sum())
                o[b, h, i] = sum(w[t] * v[b, h, j] for t, j in enumerate(js)) / w.sum()
    return o, lse


@pytest.mark.parametrize("causal", [False, True])
def test_against_float64_brute_force(causal):
    q, k, v = _qkv(1, 2, 13, 13, 8, seed=1)
    o, lse = attention_fwd_oracle(q, k, v, causal=causal, softmax_scale=0.3)
    o64, lse64 = _brute_force(q, k, v, causal, 0.3)
    assert np.allclose(o.numpy(), o64, atol=2e-6, rtol=1e-5)
    assert np.allclose(lse.numpy(), lse64, atol=2e-6, rtol=1e-6)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 4, 128, 64), (1, 3, 257, 128)])
def test_against_library_sdpa_and_logsumexp(causal, shape):
    B, H, S, D = shape
    q, k, v = _qkv(B, H, S, S, D, seed=2, dtype=torch.bfloat16)
    o, lse = attention_fwd_oracle(q, k, v, causal=causal, q_chunk=100)
    scale = 1 / math.sqrt(D)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal, scale=scale)
    assert torch.allclose(o, ref, atol=1e-5, rtol=1e-5)
    s = (q.float() @ k.float().transpose(-1, -2)) * scale
    if causal:
        s = s.masked_fill(torch.ones(S, S, dtype=torch.bool).triu(1), float("-inf"))
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-5, rtol=1e-6)


def test_invariants():
    B, H, S, D = 1, 2, 64, 16
    q, k, v = _qkv(B, H, S, S, D, seed=3)
    # V == 1 => O == 1
    o, _ = attention_fwd_oracle(q, k, torch.ones_like(v), causal=True)
    assert torch.allclose(o, torch.ones_like(o), atol=1e-6)
    # Q == 0 => O_i = mean of the allowed V rows, LSE_i = ln(#allowed)
    o, lse = attention_fwd_oracle(torch.zeros_like(q), k, v, causal=True)
    cm = torch.cumsum(v, dim=2) / torch.arange(1, S + 1).view(1, 1, S, 1)
    assert torch.allclose(o, cm, atol=1e-5)
    assert torch.allclose(lse, torch.log(torch.arange(1, S + 1, dtype=torch.float32)).expand(B, H, S), atol=1e-6)
    o, lse = attention_fwd_oracle(torch.zeros_like(q), k, v, causal=False)
    assert torch.allclose(o, v.mean(dim=2, keepdim=True).expand_as(o), atol=1e-5)
    assert torch.allclose(lse, torch.full_like(lse, math.log(S)), atol=1e-6)
    # causal row 0 sees only key 0
    o, lse = attention_fwd_oracle(q, k, v, causal=True)
    assert torch.allclose(o[:, :, 0], v[:, :, 0], atol=1e-6)
    assert torch.allclose(lse[:, :, 0], (q[:, :, 0] * k[:, :, 0]).sum(-1) / math.sqrt(D), atol=1e-5)
    # non-causal: permuting the keys (and values with them) changes nothing
    perm = torch.randperm(S, generator=torch.Generator().manual_seed(9))
    o1, l1 = attention_fwd_oracle(q, k, v, causal=False)
    o2, l2 = attention_fwd_oracle(q, k[:, :, perm], v[:, :, perm], causal=False)
    assert torch.allclose(o1, o2, atol=1e-5) and torch.allclose(l1, l2, atol=1e-5)
    # exp(scale*qk - LSE) is the softmax: rows sum to 1 and reproduce O
    s = (q @ k.transpose(-1, -2)) / math.sqrt(D)
    pr = torch.exp(s - l1.unsqueeze(-1))
    assert torch.allclose(pr.sum(-1), torch.ones(B, H, S), atol=1e-5)
    assert torch.allclose(pr @ v, o1, atol=1e-5)
    # a dominant key selects its value row
    q2 = torch.zeros(1, 1, 4, D); k2 = torch.zeros(1, 1, 4, D); v2 = torch.randn(1, 1, 4, D)
    for i in range(4):
        q2[0, 0, i, i] = 60.0
        k2[0, 0, (i + 1) % 4, i] = 60.0
    o, _ = attention_fwd_oracle(q2, k2, v2, causal=False, softmax_scale=1.0)
    assert torch.allclose(o[0, 0], v2[0, 0, [1, 2, 3, 0]], atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_tile_recurrence_equals_closed_form(causal):
    """The reference's online recurrence (running reference = lse_i) equals the closed form."""
    q, k, v = _qkv(1, 1, 384, 384, 32, seed=4)
    scale = 1 / math.sqrt(32)
    o, lse = attention_fwd_oracle(q, k, v, causal=causal)
    o_t, lse_t = online_softmax_tiles(q[0, 0].numpy(), k[0, 0].numpy(), v[0, 0].numpy(), causal, scale)
    assert np.allclose(o_t, o[0, 0].numpy(), atol=2e-5, rtol=1e-5)
    assert np.allclose(lse_t, lse[0, 0].numpy(), atol=2e-5, rtol=1e-6)


def test_golden_fixture():
    z = np.load(GOLDEN)
    to16 = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.float16)
    q, k, v = to16(z["q"]), to16(z["k"]), to16(z["v"])
    for tag, causal in (("full", False), ("causal", True)):
        o, lse = attention_fwd_oracle(q, k, v, causal=causal, softmax_scale=float(z["scale"]))
        assert np.allclose(o.numpy(), z[f"o_{tag}"], atol=1e-5, rtol=1e-5)
        assert np.allclose(lse.numpy(), z[f"lse_{tag}"], atol=1e-5, rtol=1e-6)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 2, 37, 53, 16), (2, 1, 64, 64, 32), (1, 1, 5, 9, 8)])
def test_backward_closed_form_equals_autograd(shape, causal):
    # the closed-form gradients against torch.autograd on the forward expression, both in float64
    B, H, M, N, D = shape
    g = torch.Generator().manual_seed(M * N)
    q, k, v, go = (torch.randn(B, H, n, D, generator=g, dtype=torch.float64) for n in (M, N, N, M))
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    s = (qa / math.sqrt(D)) @ ka.transpose(-1, -2)
    if causal:
        s = s.masked_fill(torch.arange(N)[None, :] > torch.arange(M)[:, None], float("-inf"))
    o = torch.softmax(s, dim=-1) @ va
    dq_a, dk_a, dv_a = torch.autograd.grad(o, (qa, ka, va), go)
    dq, dk, dv = ao.attention_bwd_oracle(q, k, v, go, causal=causal, dtype=torch.float64)
    for name, a, b in (("dQ", dq, dq_a), ("dK", dk, dk_a), ("dV", dv, dv_a)):
        assert torch.allclose(a, b, rtol=1e-10, atol=1e-12), f"{name}: max diff {(a - b).abs().max().item():.3e}"
    # fp32 arithmetic of the same formulas stays within fp32 rounding of the float64 result
    dq32, dk32, dv32 = ao.attention_bwd_oracle(q.float(), k.float(), v.float(), go.float(), causal=causal)
    for a, b in ((dq32, dq), (dk32, dk), (dv32, dv)):
        assert (a.double() - b).abs().max().item() <= 1e-4 * max(1.0, b.abs().max().item())
    # invariants: a key no query may attend gets zero gradient (causal, keys beyond the last query)
    if causal and N > M:
        assert float(dk[:, :, M:].abs().max()) == 0.0 and float(dv[:, :, M:].abs().max()) == 0.0


def _hash_python(index, seed):
    a = (index ^ seed) & 0xFFFFFFFF
    a ^= a >> 4
    a = ((a ^ 0xDEADBEEF) + ((a << 5) & 0xFFFFFFFF)) & 0xFFFFFFFF
    a ^= a >> 11
    return a


def test_dropout_mask_restatements_and_statistics():
    # (1) numpy restatement == pure-Python-integer restatement, including 32-bit wrap of the index
    B, H, M, N, p, seed, off = 2, 3, 5, 7, 0.3, 0x12345678, (1 << 32) - 50
    mask = ao.dropout_keep_mask(p, seed, off, B, H, M, N)
    thr = int(np.float32(p) * np.float32(4294967295))
    for b in range(B):
        for h in range(H):
            for m in range(M):
                for n in range(N):
                    idx = (off + (b * H + h) * M * N + m * N + n) & 0xFFFFFFFF
                    assert bool(mask[b, h, m, n]) == (_hash_python(idx, seed) > thr)
    # (2) the hash on inputs worked out by hand: a = 0 -> 0 ^ 0 = 0; (0 ^ 0xDEADBEEF) + 0 = 0xDEADBEEF;
    #     0xDEADBEEF ^ (0xDEADBEEF >> 11) = 0xDEADBEEF ^ 0x001BD5B7 = 0xDEB66B58
    assert _hash_python(0, 0) == 0xDEB66B58
    #     a = 16: 16 ^ 1 = 17; (17 ^ 0xDEADBEEF) + (17 << 5) = 0xDEADBEFE + 0x220 = 0xDEADC11E; ^ (>> 11 = 0x001BD5B8) = 0xDEB614A6
    assert _hash_python(16, 0) == 0xDEB614A6
    # (3) threshold: p = 0 keeps everything whose hash is non-zero, p -> 1 keeps nothing
    assert ao.dropout_keep_mask(0.0, 1, 0, 1, 1, 64, 64).mean() > 0.999
    assert ao.dropout_keep_mask(0.999999, 1, 0, 1, 1, 64, 64).mean() < 1e-3
    # (4) statistics, in the reference's own style (tests/test_flash_attention_triton.py:176-280 accumulates keeps over
    #     1000 calls with advancing offsets): averaged over offsets that span the 32-bit index range the kept fraction
    #     is 1 - p. (Within ONE mask of fewer than 2^22 elements the hash is far from uniform - its top bits depend only
    #     on index bits 22 and up - so a single mask is almost entirely kept or almost entirely dropped; that is the
    #     reference's definition and is reproduced as it is.)
    for p in (0.1, 0.17, 0.5):
        for seed in (0, 123, 0xDEADBEEF):
            fracs = [ao.dropout_keep_mask(p, seed, off, 1, 1, 64, 64).mean() for off in range(0, 1 << 32, 1 << 23)]
            assert abs(np.mean(fracs) - (1 - p)) < 1.5e-2, (p, seed, np.mean(fracs))
    # shifting the offset by the mask's size gives the continuation of the same index stream
    a = ao.dropout_keep_mask(0.2, 5, 0, 1, 2, 8, 16)
    b = ao.dropout_keep_mask(0.2, 5, 8 * 16, 1, 1, 8, 16)
    assert np.array_equal(a[0, 1], b[0, 0])


@pytest.mark.parametrize("causal", [False, True])
def test_backward_with_dropout_equals_autograd(causal):
    B, H, M, N, D = 1, 2, 33, 41, 16
    drop = (0.25, 99, 1000)
    g = torch.Generator().manual_seed(5)
    q, k, v, go = (torch.randn(B, H, n, D, generator=g, dtype=torch.float64) for n in (M, N, N, M))
    z = torch.from_numpy(ao.dropout_keep_mask(*drop, B, H, M, N)).double() * float(np.float32(1.0) / (np.float32(1.0) - np.float32(drop[0])))
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    s = (qa / math.sqrt(D)) @ ka.transpose(-1, -2)
    if causal:
        s = s.masked_fill(torch.arange(N)[None, :] > torch.arange(M)[:, None], float("-inf"))
    o = (torch.softmax(s, dim=-1) * z) @ va
    ref = torch.autograd.grad(o, (qa, ka, va), go)
    got = ao.attention_bwd_oracle(q, k, v, go, causal=causal, dtype=torch.float64, dropout=drop)
    for a, b in zip(got, ref):
        assert torch.allclose(a, b, rtol=1e-10, atol=1e-12)
    o32, lse32 = attention_fwd_oracle(q.float(), k.float(), v.float(), causal=causal, dropout=drop)
    assert torch.allclose(o32.double(), o.detach(), rtol=1e-4, atol=1e-5)
    # LSE is that of the undropped scores
    assert torch.allclose(lse32.double(), torch.logsumexp(s.detach(), dim=-1), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("kind", ["vector", "matrix"])
def test_bias_against_library_and_invariants(causal, kind):
    # (1) the library's additive float mask is the same thing as the reference's bias (attention_ref.py:50-51)
    B, H, M, N, D = 2, 3, 19, 19, 16
    q, k, v = _qkv(B, H, M, N, D, seed=11)
    g = torch.Generator().manual_seed(12)
    bias = torch.randn(B, H, 1 if kind == "vector" else M, N, generator=g) * 2.0
    o, lse = attention_fwd_oracle(q, k, v, causal=causal, bias=bias)
    mask = bias.expand(B, H, M, N).clone()
    if causal:
        mask = mask.masked_fill(torch.ones(M, N, dtype=torch.bool).triu(1), float("-inf"))
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    assert torch.allclose(o, ref, atol=1e-5, rtol=1e-5)
    s = (q @ k.transpose(-1, -2)) / math.sqrt(D) + mask
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-5, rtol=1e-6)
    # (2) a bias constant along the keys leaves O alone and shifts the logsumexp by that constant
    o0, lse0 = attention_fwd_oracle(q, k, v, causal=causal)
    const = torch.randn(B, H, M, 1, generator=g).expand(B, H, M, N)
    o1, lse1 = attention_fwd_oracle(q, k, v, causal=causal, bias=const)
    assert torch.allclose(o1, o0, atol=1e-5, rtol=1e-5)
    assert torch.allclose(lse1, lse0 + const[..., 0], atol=1e-5, rtol=1e-6)
    # (3) a bias of -inf on the last keys is attention over the remaining keys; broadcast over batch and heads
    cut = torch.zeros(1, 1, 1, N)
    cut[..., N - 4:] = float("-inf")
    o2, lse2 = attention_fwd_oracle(q, k, v, causal=causal, bias=cut)
    o3, lse3 = attention_fwd_oracle(q, k[:, :, :N - 4], v[:, :, :N - 4], causal=causal)
    assert torch.allclose(o2, o3, atol=1e-6, rtol=1e-6) and torch.allclose(lse2, lse3, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("with_dropout", [False, True])
def test_backward_with_bias_equals_autograd(causal, with_dropout):
    B, H, M, N, D = 2, 2, 21, 35, 8
    drop = (0.2, 7, 123456) if with_dropout else None
    g = torch.Generator().manual_seed(6)
    q, k, v, go = (torch.randn(B, H, n, D, generator=g, dtype=torch.float64) for n in (M, N, N, M))
    bias = torch.randn(1, H, M, N, generator=g, dtype=torch.float64)
    z = 1.0
    if drop:
        z = torch.from_numpy(ao.dropout_keep_mask(*drop, B, H, M, N)).double() * float(np.float32(1.0) / (np.float32(1.0) - np.float32(drop[0])))
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    s = (qa / math.sqrt(D)) @ ka.transpose(-1, -2) + bias
    if causal:
        s = s.masked_fill(torch.arange(N)[None, :] > torch.arange(M)[:, None], float("-inf"))
    o = (torch.softmax(s, dim=-1) * z) @ va
    ref = torch.autograd.grad(o, (qa, ka, va), go)
    got = ao.attention_bwd_oracle(q, k, v, go, causal=causal, dtype=torch.float64, dropout=drop, bias=bias)
    for a, b in zip(got, ref):
        assert torch.allclose(a, b, rtol=1e-10, atol=1e-12)
    o32, _ = attention_fwd_oracle(q.float(), k.float(), v.float(), causal=causal, dropout=drop, bias=bias.float())
    assert torch.allclose(o32.double(), o.detach(), rtol=1e-4, atol=1e-5)
