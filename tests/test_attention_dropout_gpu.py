"""Dropout of the attention probabilities: the kernels' mask must be the reference's (flash_attention_triton.py:38-50,
:125,:216-219), bit for bit, which shows as forward and backward parity with the oracle that applies the same mask.

The reference's hash is far from uniform inside one call (see tests/test_oracle_attention.py), so the cases here pick
dropout probabilities and offsets for which the mask of the tested shape is genuinely mixed, and say so."""
import math

import numpy as np
import pytest
import torch

from fast_ops.flash_attention.flash_attention import flash_attn, multi_head_attention
from fast_ops_amd.flash_attention.flash_attention import next_dropout_state
from oracle.attention_oracle import attention_bwd_oracle, attention_fwd_oracle, dropout_keep_mask

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
O_ATOL, O_RTOL, LSE_ATOL = 2e-2, 1e-2, 1e-3


def _mixed_state(p, B, H, M, N, seed):
    """An offset at which the reference's mask for this shape keeps between 25 % and 75 % of the elements."""
    for off in range(0, 1 << 32, (1 << 20) + 12345):
        f = dropout_keep_mask(p, seed, off, B, H, M, N).mean()
        if 0.25 < f < 0.75:
            return off
    raise AssertionError("no mixed mask found")


def _inputs(B, H, Sq, Sk, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Sq, Sk, Sk, Sq))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("shape", [(2, 3, 200, 300), (1, 2, 129, 65)])
def test_forward_and_backward_with_dropout(shape, D, causal, dtype):
    B, H, Sq, Sk = shape
    p, seed = 0.45, 1234567
    off = _mixed_state(p, B, H, Sq, Sk, seed)
    drop = (p, seed, off)
    q, k, v, go = _inputs(B, H, Sq, Sk, D, dtype, seed=Sq + D)
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal, dropout=drop)
    ref = attention_bwd_oracle(q, k, v, go, causal=causal, dropout=drop)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    o, lse = multi_head_attention(qd, kd, vd, causal=causal, return_lse=True, dropout_p=p, dropout_state=(seed, off))
    got = torch.autograd.grad(o, (qd, kd, vd), go.to(DEV))
    torch.cuda.synchronize()
    err = (o.detach().float().cpu() - o_ref).abs()
    assert float((err - (O_ATOL + O_RTOL * o_ref.abs())).max()) <= 0, f"O: max abs err {float(err.max()):.3e}"
    assert float((lse.cpu() - lse_ref).abs().max()) <= LSE_ATOL       # LSE is that of the undropped scores
    for name, a, r in zip(("dQ", "dK", "dV"), got, ref):
        e = (a.float().cpu() - r).abs().max().item()
        assert e <= 2e-2 * max(1.0, r.abs().max().item()), f"{name}: error {e:.3e} vs magnitude {r.abs().max().item():.3e}"
    # a different seed gives a different result; the same state reproduces it exactly
    o2 = multi_head_attention(qd, kd, vd, causal=causal, dropout_p=p, dropout_state=(seed, off))
    assert torch.equal(o2, o)
    # (a wrong mask would be off by O(1): every dropped or kept element moves O by its whole contribution)


def test_mask_is_the_references_element_by_element():
    # V = identity (Sk = D = 64), Q = 0: softmax is uniform, O[q, key] = Z[q, key] / Sk with Z = keep / (1 - p), so the
    # output IS the mask
    B, H, Sq, Sk, D = 2, 2, 70, 64, 64
    p, seed = 0.87, 42
    off = _mixed_state(p, B, H, Sq, Sk, seed)
    q = torch.zeros(B, H, Sq, D, dtype=torch.float16, device=DEV)
    k = torch.randn(B, H, Sk, D, dtype=torch.float16, device=DEV)
    v = torch.eye(D, dtype=torch.float16, device=DEV).expand(B, H, Sk, D).contiguous()
    o = multi_head_attention(q, k, v, dropout_p=p, dropout_state=(seed, off))
    keep = dropout_keep_mask(p, seed, off, B, H, Sq, Sk)
    got = (o.float().cpu().numpy() > 0)
    assert 0.25 < keep.mean() < 0.75
    assert np.array_equal(got, keep)
    scale = float(np.float32(1.0) / (np.float32(1.0) - np.float32(p))) / Sk
    assert np.allclose(o.float().cpu().numpy()[keep], scale, rtol=2e-3)


def test_generator_state_is_consumed_like_the_reference():
    # flash_attention_triton.py:641-665: seed and offset come from torch's generator; the offset advances by the number
    # of probabilities rounded up to a multiple of 4
    torch.manual_seed(77)
    s0, o0 = next_dropout_state(10)
    s1, o1 = next_dropout_state(1)
    assert s0 == s1 == 77 and o1 == o0 + 12
    q, k, v, _ = (t.to(DEV) for t in _inputs(1, 2, 64, 64, 64, torch.bfloat16, 0))
    torch.manual_seed(5)
    a = flash_attn(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), dropout_p=0.87)
    b = flash_attn(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), dropout_p=0.87)   # next offsets
    torch.manual_seed(5)
    c = flash_attn(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), dropout_p=0.87)
    assert torch.equal(a, c)
    with pytest.raises(RuntimeError, match="dropout_p"):
        multi_head_attention(q, k, v, dropout_p=1.0)


def test_dropout_mask_tensor_is_the_kernels_mask():
    # triton_dropout_mask of the reference (flash_attention_triton.py:697-717): the mask as a tensor, bit for bit the
    # oracle's, for explicit states (including a 32-bit wrap of the index) and ragged sizes that end inside a 16-byte store
    from fast_ops.flash_attention.flash_attention_triton import flash_attn_triton, increment_philox_state, triton_dropout_mask
    from fast_ops_amd.flash_attention.flash_attention import dropout_mask
    for (B, H, Sq, Sk, p, seed, off) in [(2, 3, 70, 64, 0.87, 42, 5), (1, 1, 1, 1, 0.5, 7, 0), (1, 2, 33, 17, 0.3, 99, (1 << 32) - 500),
                                         (2, 2, 128, 256, 0.17, 123, 3 << 20)]:
        got = dropout_mask(p, B, H, Sq, Sk, DEV, dropout_state=(seed, off))
        assert got.dtype == torch.bool and tuple(got.shape) == (B, H, Sq, Sk)
        assert np.array_equal(got.cpu().numpy(), dropout_keep_mask(p, seed, off, B, H, Sq, Sk))
    # the reference's test flow (tests/test_flash_attention_triton.py:93-103): seed, run the attention, seed again, take
    # the mask: it is the mask the attention used
    B, H, Sq, Sk, D, p = 2, 2, 96, 80, 64, 0.87
    q, k, v, _ = (t.to(DEV).transpose(1, 2) for t in _inputs(B, H, Sq, Sk, D, torch.float16, 3))
    torch.manual_seed(1234567)
    increment_philox_state(_mixed_state(p, B, H, Sq, Sk, 1234567))   # to offsets where this hash mixes a small mask
    state = torch.cuda.get_rng_state()
    out = flash_attn_triton(q, k, v, None, False, p)
    after = torch.cuda.get_rng_state()
    torch.cuda.set_rng_state(state)
    keep = triton_dropout_mask(p, B, H, Sq, Sk, device=DEV)
    assert torch.equal(torch.cuda.get_rng_state(), after)     # both consume the generator alike
    words = state.numpy().view(np.uint64)
    o_ref, _ = attention_fwd_oracle(*(t.transpose(1, 2) for t in (q, k, v)), dropout=(p, int(words[-2]), int(words[-1])))
    assert np.array_equal(keep.cpu().numpy(), dropout_keep_mask(p, int(words[-2]), int(words[-1]), B, H, Sq, Sk))
    assert 0.2 < float(keep.float().mean()) < 0.8
    err = (out.transpose(1, 2).float().cpu() - o_ref).abs()
    assert float((err - (O_ATOL + O_RTOL * o_ref.abs())).max()) <= 0


@pytest.mark.parametrize("seed", [123, 0])
def test_dropout_statistics_like_the_reference(seed):
    # tests/test_flash_attention_triton.py:204-236: 1000 masks from consecutive generator states; every element must be
    # kept in a fraction of them that a binomial test against 1 - p does not reject at 1e-8. (p-values are computed per
    # distinct count instead of per element: the same numbers without the reference's 10^6 x 10^3 table.)
    import scipy.stats
    from fast_ops.flash_attention.flash_attention_triton import triton_dropout_mask
    B, H, Sq, Sk, p, n_trials = 8, 4, 128, 256, 0.17, 1000
    torch.manual_seed(seed)
    sums = torch.zeros(B, H, Sq, Sk, dtype=torch.int32, device=DEV)
    for _ in range(n_trials):
        sums += triton_dropout_mask(p, B, H, Sq, Sk, device=DEV)
    counts = np.unique(sums.cpu().numpy())
    pvals = {int(c): scipy.stats.binomtest(int(c), n_trials, 1.0 - p).pvalue for c in counts}
    worst = min(pvals, key=pvals.get)
    assert pvals[worst] > 1e-8, f"failed binomial test: kept {worst / n_trials}, expected {1 - p}, p-value {pvals[worst]}"
