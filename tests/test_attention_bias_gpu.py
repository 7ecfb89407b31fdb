"""Additive attention bias (flash_attention_triton.py:176-198,497-509,752-768; attention_ref.py:50-51): forward and
backward parity with the oracle for the bias shapes the reference tests (tests/test_flash_attention_triton.py:36,
74-82: "1h1k", "1hqk", "b11k", "b1qk"), fp32 and half-precision bias, with multi-query K/V and with dropout."""
import math

import pytest
import torch

from fast_ops.flash_attention.flash_attention import flash_attn
from fast_ops_amd.flash_attention.flash_attention import attn_bwd_strided, attn_fwd_strided
from oracle.attention_oracle import attention_bwd_oracle, attention_fwd_oracle, dropout_keep_mask

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
O_ATOL, O_RTOL, LSE_ATOL = 2e-2, 1e-2, 1e-3


def _bias(kind, B, H, Sq, Sk, dtype, g):
    shape = {"1h1k": (1, H, 1, Sk), "1hqk": (1, H, Sq, Sk), "b11k": (B, 1, 1, Sk), "b1qk": (B, 1, Sq, Sk), "bhqk": (B, H, Sq, Sk)}[kind]
    return torch.randn(shape, generator=g).to(dtype)


def _bshd(t):
    return t.transpose(1, 2)    # [B,H,S,D] -> the [B,S,H,D] view flash_attn takes


def _check(o, lse, grads, o_ref, lse_ref, grads_ref):
    err = (o.detach().float().cpu() - o_ref).abs()
    assert float((err - (O_ATOL + O_RTOL * o_ref.abs())).max()) <= 0, f"O: max abs err {float(err.max()):.3e}"
    assert float((lse.cpu() - lse_ref).abs().max()) <= LSE_ATOL
    for name, a, r in zip(("dQ", "dK", "dV"), grads, grads_ref):
        e = (a.float().cpu() - r).abs().max().item()
        assert e <= 2e-2 * max(1.0, r.abs().max().item()), f"{name}: error {e:.3e} vs magnitude {r.abs().max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("kind", ["1h1k", "1hqk", "b11k", "b1qk", "bhqk"])
@pytest.mark.parametrize("D", [64, 128])
def test_bias_shapes_of_the_reference(D, kind, causal, dtype):
    B, H, Sq, Sk = 2, 3, 200, 331      # ragged: both lengths off the tile sizes
    g = torch.Generator().manual_seed(D + len(kind))
    q, k, v, go = (torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Sq, Sk, Sk, Sq))
    bias = _bias(kind, B, H, Sq, Sk, torch.float32, g) * 2.0
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal, bias=bias)
    ref = attention_bwd_oracle(q, k, v, go, causal=causal, bias=bias)
    qd, kd, vd = (_bshd(t.to(DEV)).requires_grad_(True) for t in (q, k, v))
    o, lse = flash_attn(qd, kd, vd, bias=bias.to(DEV), causal=causal, return_lse=True)
    got = torch.autograd.grad(o, (qd, kd, vd), _bshd(go.to(DEV)))
    torch.cuda.synchronize()
    _check(_bshd(o), lse, [_bshd(t) for t in got], o_ref, lse_ref, ref)


@pytest.mark.parametrize("bias_dtype", ["f32", "operand"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("kind", ["1h1k", "1hqk", "b11k", "bhqk"])
@pytest.mark.parametrize("shape", [(200, 320, 128), (130, 200, 64), (64, 64, 128), (300, 1032, 64)])
def test_bias_rows_on_16_byte_boundaries(shape, kind, causal, bias_dtype):
    # key counts that put every bias row on a 16-byte boundary: complete 64-key tiles of the bias then reach the forward
    # kernel through its tile copies (the last, partial tile and every other alignment through per-element loads)
    Sq, Sk, D = shape
    B, H, dtype = 2, 2, torch.bfloat16
    g = torch.Generator().manual_seed(Sq + Sk)
    q, k, v, go = (torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Sq, Sk, Sk, Sq))
    bias = _bias(kind, B, H, Sq, Sk, torch.float32 if bias_dtype == "f32" else dtype, g) * 2.0
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal, bias=bias)
    ref = attention_bwd_oracle(q, k, v, go, causal=causal, bias=bias)
    qd, kd, vd = (_bshd(t.to(DEV)).requires_grad_(True) for t in (q, k, v))
    o, lse = flash_attn(qd, kd, vd, bias=bias.to(DEV), causal=causal, return_lse=True)
    got = torch.autograd.grad(o, (qd, kd, vd), _bshd(go.to(DEV)))
    _check(_bshd(o), lse, [_bshd(t) for t in got], o_ref, lse_ref, ref)
    # a view whose rows do not start on 16-byte boundaries gives the same result through the other path
    shifted = torch.empty(bias.shape[:-1] + (Sk + 1,), dtype=bias.dtype, device=DEV)[..., 1:]
    shifted.copy_(bias)
    o2 = flash_attn(qd, kd, vd, bias=shifted, causal=causal)
    assert torch.equal(o2, o)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("kind", ["1h1k", "b1qk"])
def test_bias_in_the_operand_dtype(kind, dtype):
    # flash_attention_triton.py:755: bias.dtype in [q.dtype, torch.float]
    B, H, Sq, Sk, D = 2, 2, 130, 257, 128
    g = torch.Generator().manual_seed(3)
    q, k, v, go = (torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Sq, Sk, Sk, Sq))
    bias = _bias(kind, B, H, Sq, Sk, dtype, g)
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=True, bias=bias)
    ref = attention_bwd_oracle(q, k, v, go, causal=True, bias=bias)
    qd, kd, vd = (_bshd(t.to(DEV)).requires_grad_(True) for t in (q, k, v))
    o, lse = flash_attn(qd, kd, vd, bias=bias.to(DEV), causal=True, return_lse=True)
    got = torch.autograd.grad(o, (qd, kd, vd), _bshd(go.to(DEV)))
    _check(_bshd(o), lse, [_bshd(t) for t in got], o_ref, lse_ref, ref)
    other = torch.float16 if dtype == torch.bfloat16 else torch.bfloat16
    with pytest.raises(RuntimeError, match="dtype"):
        flash_attn(qd, kd, vd, bias=bias.to(DEV).to(other))


@pytest.mark.parametrize("causal", [False, True])
def test_bias_with_dropout_and_multi_query(causal):
    # the reference's test crosses bias with dropout and with K/V heads that are an expanded view (:38-39,66-72)
    B, H, Sq, Sk, D, dtype = 2, 4, 150, 200, 64, torch.bfloat16
    p, seed = 0.45, 4242
    off = next(o for o in range(0, 1 << 32, (1 << 20) + 12345) if 0.25 < dropout_keep_mask(p, seed, o, B, H, Sq, Sk).mean() < 0.75)
    g = torch.Generator().manual_seed(9)
    q, go = (torch.randn(B, H, Sq, D, generator=g).to(dtype) for _ in range(2))
    k1, v1 = (torch.randn(B, 1, Sk, D, generator=g).to(dtype) for _ in range(2))
    bias = _bias("1hqk", B, H, Sq, Sk, torch.float32, g)
    k, v = k1.expand(B, H, Sk, D), v1.expand(B, H, Sk, D)
    drop = (p, seed, off)
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal, dropout=drop, bias=bias)
    dq_r, dk_r, dv_r = attention_bwd_oracle(q, k, v, go, causal=causal, dropout=drop, bias=bias)
    qd = _bshd(q.to(DEV)).requires_grad_(True)
    k1d, v1d = (t.to(DEV).requires_grad_(True) for t in (k1, v1))
    kd, vd = (_bshd(t.expand(B, H, Sk, D)) for t in (k1d, v1d))
    o, lse = flash_attn(qd, kd, vd, bias=bias.to(DEV), causal=causal, dropout_p=p, return_lse=True, dropout_state=(seed, off))
    dq, dk1, dv1 = torch.autograd.grad(o, (qd, k1d, v1d), _bshd(go.to(DEV)))
    _check(_bshd(o), lse, [_bshd(dq), dk1, dv1], o_ref, lse_ref, [dq_r, dk_r.sum(1, keepdim=True), dv_r.sum(1, keepdim=True)])


def test_bias_as_key_padding_mask():
    # -inf on padded keys, including the whole first tile of keys (left padding): equals attention over the kept keys.
    # (A bias of -inf on every key of a row gives NaN in attention_ref.py:59 as well; the reference's mask_all cases
    # compare NaN with NaN and assert nothing, tests/test_flash_attention_triton.py:86-87,131-139.)
    B, H, S, D, dtype = 2, 2, 300, 128, torch.float16
    g = torch.Generator().manual_seed(21)
    q, k, v, go = (torch.randn(B, H, S, D, generator=g).to(dtype) for _ in range(4))
    left, right = 70, 13
    bias = torch.zeros(B, 1, 1, S)
    bias[..., :left] = float("-inf")
    bias[..., S - right:] = float("-inf")
    o_ref, lse_ref = attention_fwd_oracle(q, k[:, :, left:S - right], v[:, :, left:S - right])
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    o, lse = attn_fwd_strided(qd, kd, vd, (0, 1, 2, 3), False, None, None, bias.to(DEV))
    dq, dk, dv = attn_bwd_strided(qd, kd, vd, o, lse, go.to(DEV), (0, 1, 2, 3), False, None, None, bias.to(DEV))
    dq_r, dk_r, dv_r = attention_bwd_oracle(q, k[:, :, left:S - right], v[:, :, left:S - right], go)
    assert torch.isfinite(o.float()).all()
    _check(o, lse, [dq, dk[:, :, left:S - right], dv[:, :, left:S - right]], o_ref, lse_ref, [dq_r, dk_r, dv_r])
    assert float(dk[:, :, :left].abs().max()) == 0.0 and float(dv[:, :, S - right:].abs().max()) == 0.0


def test_bias_odd_head_dim_and_large_magnitude():
    # head_dim 40 runs on padded copies; a bias much larger than the scores decides the softmax alone
    B, H, Sq, Sk, D, dtype = 1, 2, 100, 190, 40, torch.bfloat16
    g = torch.Generator().manual_seed(2)
    q, k, v, go = (torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Sq, Sk, Sk, Sq))
    bias = torch.randn(1, 1, Sq, Sk, generator=g) * 30.0
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=False, bias=bias)
    ref = attention_bwd_oracle(q, k, v, go, bias=bias)
    qd, kd, vd = (_bshd(t.to(DEV)).requires_grad_(True) for t in (q, k, v))
    o, lse = flash_attn(qd, kd, vd, bias=bias.to(DEV), return_lse=True)
    got = torch.autograd.grad(o, (qd, kd, vd), _bshd(go.to(DEV)))
    _check(_bshd(o), lse, [_bshd(t) for t in got], o_ref, lse_ref, ref)


def test_bias_rejections():
    q = torch.randn(1, 64, 2, 64, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="Last 2 dimensions"):          # flash_attention_triton.py:764-767
        flash_attn(q, q, q, bias=torch.zeros(1, 2, 3, 64, device=DEV))
    with pytest.raises(RuntimeError, match="4-dimensional"):
        flash_attn(q, q, q, bias=torch.zeros(64, 64, device=DEV))
    # a bias that wants a gradient: the backward refuses, as the reference's does (:854)
    qg = q.clone().requires_grad_(True)
    bias = torch.zeros(1, 2, 64, 64, device=DEV, requires_grad=True)
    out = flash_attn(qg, q, q, bias=bias)
    with pytest.raises(RuntimeError, match="bias gradient"):
        out.sum().backward()
    # non-contiguous last dimension is made contiguous (:758-759)
    b2 = torch.randn(1, 2, 64, 128, device=DEV)[..., ::2]
    a = flash_attn(q, q, q, bias=b2)
    b = flash_attn(q, q, q, bias=b2.contiguous())
    assert torch.equal(a, b)


# ---- a bias that is the same for every query ("1h1k", "b11k": the reference's vector bias, flash_attention_triton.py:
# 176-186, the one its benchmark uses, benchmarks/benchmark_flash_attention.py:198) also runs in the pipelined kernels
def _kernel_with_key_bias(B, H, Sq, Sk, D, causal, has_bias=2):
    import ctypes

    from fast_ops_amd import _lib

    I3 = ctypes.c_int64 * 3
    dense = I3(H * Sk * D, Sk * D, D)
    code = _lib.load().fo_attn_fwd_kernel(B, H, Sq, Sk, D, dense, dense, int(causal), has_bias, 0)
    assert code >= 0
    return code


@pytest.mark.parametrize("bias_dtype", ["f32", "operand"])
@pytest.mark.parametrize("kind", ["1h1k", "b11k"])
@pytest.mark.parametrize("case", [
    # B, H, Sq, Sk, D, causal, kernel expected (8: 128 rows pipelined, 32: 256 rows as four waves)
    (1, 12, 2048, 2048, 128, False, 8), (1, 12, 2048, 2048, 128, True, 8), (1, 12, 4000, 4072, 64, True, 8),
    (2, 12, 1100, 2091, 128, False, 8), (4, 16, 2048, 2048, 128, False, 32), (2, 64, 1024, 1500, 128, True, 32),
    (2, 8, 8192, 8192, 128, True, 32), (2, 16, 4099, 8190, 128, False, 32), (4, 8, 4096, 4100, 64, False, 32), (2, 16, 8192, 8192, 64, True, 32),
], ids=lambda c: "-".join(str(x) for x in c))
def test_per_key_bias_in_the_pipelined_kernels(case, kind, bias_dtype):
    from fast_ops_amd import _lib

    B, H, Sq, Sk, D, causal, expected = case
    assert _kernel_with_key_bias(B, H, Sq, Sk, D, causal) == expected
    assert _kernel_with_key_bias(B, H, Sq, Sk, D, causal, has_bias=1) == 0          # a bias with a query stride: plain kernel
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(Sq + Sk + D)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    k, v = (torch.randn(B, H, Sk, D, generator=g).to(dtype) for _ in range(2))
    bias = (_bias(kind, B, H, Sq, Sk, torch.float32 if bias_dtype == "f32" else dtype, g) * 3.0)
    qd, kd, vd, bd = (t.to(DEV) for t in (q, k, v, bias))
    o, lse = attn_fwd_strided(qd, kd, vd, (0, 1, 2, 3), causal, None, None, bd)
    # against the oracle on some heads and query rows (the whole of the large shapes would take the CPU minutes) ...
    heads = [(0, 0), (B - 1, H - 1)]
    for b, h in heads:
        rows = slice(0, Sq) if Sq * Sk <= 2048 * 2048 else slice(Sq - 700, Sq)
        qs = q[b:b + 1, h:h + 1, rows]
        bsl = bias[b if bias.shape[0] > 1 else 0, h if bias.shape[1] > 1 else 0][None, None].float()
        if causal:
            # rows of the slice keep their causal limit: the oracle masks top-left aligned, so give it the mask as bias
            qi = torch.arange(Sq)[rows, None]
            bsl = bsl.expand(1, 1, qs.shape[2], Sk).clone()
            bsl[0, 0][torch.arange(Sk)[None, :] > qi] = float("-inf")
        o_ref, lse_ref = attention_fwd_oracle(qs, k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], causal=False, bias=bsl)
        err = (o[b, h, rows].float().cpu() - o_ref[0, 0]).abs()
        assert float((err - (O_ATOL + O_RTOL * o_ref[0, 0].abs())).max()) <= 0, f"O head {b},{h}: max abs err {float(err.max()):.3e}"
        assert float((lse[b, h, rows].cpu() - lse_ref[0, 0]).abs().max()) <= LSE_ATOL
    # ... and everywhere against the plain 128-row kernel, whose bias path the tests above pin
    _lib.tune_set("attn.variant", 0)
    try:
        assert _kernel_with_key_bias(B, H, Sq, Sk, D, causal) == 0
        o0, lse0 = attn_fwd_strided(qd, kd, vd, (0, 1, 2, 3), causal, None, None, bd)
    finally:
        _lib.tune_set("attn.variant", -1)
    # (both round O to the operand type: one unit in the last place of the larger outputs is 2^-5)
    assert float(((o.float() - o0.float()).abs() - (2e-2 + 2e-2 * o0.float().abs())).max()) <= 0 and float((lse - lse0).abs().max()) <= 1e-4
    assert not torch.equal(o, torch.zeros_like(o))


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
def test_key_padding_mask_in_the_pipelined_kernels(D, causal):
    # -inf on the first keys (more than a tile of them: rows start without any key that counts) and on the last ones
    B, H, S, dtype = 2, 6, 4096 if D == 64 else 2048, torch.float16
    assert _kernel_with_key_bias(B, H, S, S, D, causal) == 8
    g = torch.Generator().manual_seed(5 + D)
    q, k, v = (torch.randn(B, H, S, D, generator=g).to(dtype) for _ in range(3))
    left, right = 150, 333
    bias = torch.zeros(B, 1, 1, S)
    bias[0, ..., :left] = float("-inf")
    bias[..., S - right:] = float("-inf")
    o, lse = attn_fwd_strided(q.to(DEV), k.to(DEV), v.to(DEV), (0, 1, 2, 3), causal, None, None, bias.to(DEV))
    for b in range(B):
        lo = left if b == 0 else 0
        rows = slice(lo, S)                  # causal: the rows before the first kept key have no key at all (NaN, as in attention_ref.py:59)
        kk, vv = k[b:b + 1, :2, lo:S - right], v[b:b + 1, :2, lo:S - right]
        if causal:
            o_ref, lse_ref = attention_fwd_oracle(q[b:b + 1, :2, lo:S - right], kk, vv, causal=True)
            rows = slice(lo, S - right)
        else:
            o_ref, lse_ref = attention_fwd_oracle(q[b:b + 1, :2, rows], kk, vv)
        got = o[b, :2, rows].float().cpu()
        assert torch.isfinite(got).all()
        err = (got - o_ref[0]).abs()
        assert float((err - (O_ATOL + O_RTOL * o_ref[0].abs())).max()) <= 0, f"batch {b}: max abs err {float(err.max()):.3e}"
        assert float((lse[b, :2, rows].cpu() - lse_ref[0]).abs().max()) <= LSE_ATOL


def test_per_key_bias_longer_than_the_pipelined_kernels_keep():
    # more than 8192 keys: the row of the bias no longer fits beside the tile rings, the plain kernel takes the call
    assert _kernel_with_key_bias(1, 12, 2048, 8256, 128, False) == 0
    assert _kernel_with_key_bias(1, 12, 2048, 8192, 128, False) in (8, 32)
    B, H, Sq, Sk, D, dtype = 1, 12, 300, 8300, 128, torch.bfloat16
    g = torch.Generator().manual_seed(8300)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    k, v = (torch.randn(B, H, Sk, D, generator=g).to(dtype) for _ in range(2))
    bias = torch.randn(B, 1, 1, Sk, generator=g) * 2.0
    bias[..., 8200:8250] = float("-inf")
    o, lse = attn_fwd_strided(q.to(DEV), k.to(DEV), v.to(DEV), (0, 1, 2, 3), False, None, None, bias.to(DEV))
    o_ref, lse_ref = attention_fwd_oracle(q[:, :2], k[:, :2], v[:, :2], bias=bias)
    err = (o[:, :2].float().cpu() - o_ref).abs()
    assert float((err - (O_ATOL + O_RTOL * o_ref.abs())).max()) <= 0 and float((lse[:, :2].cpu() - lse_ref).abs().max()) <= LSE_ATOL


# ---- backward with a bias that is the same for every query: the dQ kernel starts its score accumulators from it, the
# pipelined dK/dV kernel adds one value per lane (attn_bwd.variant 0 keeps the general bias kernels pinned above)
@pytest.mark.parametrize("bias_dtype", ["f32", "operand"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 3, 200, 331, 128), (2, 3, 200, 331, 64), (1, 2, 700, 513, 128), (1, 4, 1024, 1024, 64),
                                   (2, 2, 130, 1, 128), (1, 2, 333, 900, 40)], ids=lambda s: "x".join(map(str, s)))
def test_backward_with_per_key_bias(shape, causal, bias_dtype):
    from fast_ops_amd import _lib

    B, H, Sq, Sk, D = shape
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(Sq * 3 + Sk + D)
    q, k, v, go = (torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Sq, Sk, Sk, Sq))
    bias = _bias("b11k" if B > 1 else "1h1k", B, H, Sq, Sk, torch.float32 if bias_dtype == "f32" else dtype, g) * 2.0
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal, bias=bias)
    ref = attention_bwd_oracle(q, k, v, go, causal=causal, bias=bias)
    qd, kd, vd, god, bd = (t.to(DEV) for t in (q, k, v, go, bias))
    o, lse = attn_fwd_strided(qd, kd, vd, (0, 1, 2, 3), causal, None, None, bd)
    got = attn_bwd_strided(qd, kd, vd, o, lse, god, (0, 1, 2, 3), causal, None, None, bd)
    _check(o, lse, got, o_ref, lse_ref, ref)
    _lib.tune_set("attn_bwd.variant", 0)
    try:
        other = attn_bwd_strided(qd, kd, vd, o, lse, god, (0, 1, 2, 3), causal, None, None, bd)
    finally:
        _lib.tune_set("attn_bwd.variant", -1)
    for name, a, r in zip(("dQ", "dK", "dV"), got, other):
        # (the same arithmetic up to where the bias enters the exponent: a few units in the last place of the operand type)
        assert float(((a.float() - r.float()).abs() - (1e-2 + 2e-2 * r.float().abs())).max()) <= 0, name


def test_backward_with_key_padding_mask_at_a_longer_shape():
    # -inf on whole key tiles at both ends; keys that are masked get exactly zero gradients
    B, H, S, D, dtype = 2, 2, 1500, 128, torch.float16
    g = torch.Generator().manual_seed(77)
    q, k, v, go = (torch.randn(B, H, S, D, generator=g).to(dtype) for _ in range(4))
    left, right = 200, 170
    bias = torch.zeros(B, 1, 1, S)
    bias[..., :left] = float("-inf")
    bias[..., S - right:] = float("-inf")
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    o, lse = attn_fwd_strided(qd, kd, vd, (0, 1, 2, 3), False, None, None, bias.to(DEV))
    dq, dk, dv = attn_bwd_strided(qd, kd, vd, o, lse, go.to(DEV), (0, 1, 2, 3), False, None, None, bias.to(DEV))
    o_ref, lse_ref = attention_fwd_oracle(q, k[:, :, left:S - right], v[:, :, left:S - right])
    dq_r, dk_r, dv_r = attention_bwd_oracle(q, k[:, :, left:S - right], v[:, :, left:S - right], go)
    _check(o, lse, [dq, dk[:, :, left:S - right], dv[:, :, left:S - right]], o_ref, lse_ref, [dq_r, dk_r, dv_r])
    for t in (dk, dv):
        assert float(t[:, :, :left].abs().max()) == 0.0 and float(t[:, :, S - right:].abs().max()) == 0.0


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("p_drop", [0.0, 0.3])
def test_per_key_bias_in_the_128_row_kernel_with_and_without_dropout(p_drop, D, causal):
    # small shapes stay on the 128-row kernel: its per-key form (score accumulators start from the bias) against the
    # oracle and against the general bias kernel (attn.variant 1), forward and backward, also with dropout
    from fast_ops_amd import _lib

    B, H, Sq, Sk, dtype = 2, 3, 260, 459, torch.bfloat16
    seed = 99
    off = 0 if p_drop == 0 else next(o for o in range(0, 1 << 32, (1 << 20) + 777) if 0.5 < dropout_keep_mask(p_drop, seed, o, B, H, Sq, Sk).mean() < 0.9)
    drop = None if p_drop == 0 else (p_drop, seed, off)
    g = torch.Generator().manual_seed(D + int(causal))
    q, k, v, go = (torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Sq, Sk, Sk, Sq))
    bias = _bias("b11k", B, H, Sq, Sk, torch.float32, g) * 2.0
    bias[0, ..., 100:180] = float("-inf")
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal, dropout=drop, bias=bias)
    ref = attention_bwd_oracle(q, k, v, go, causal=causal, dropout=drop, bias=bias)
    qd, kd, vd, god, bd = (t.to(DEV) for t in (q, k, v, go, bias))
    o, lse = attn_fwd_strided(qd, kd, vd, (0, 1, 2, 3), causal, None, drop, bd)
    got = attn_bwd_strided(qd, kd, vd, o, lse, god, (0, 1, 2, 3), causal, None, drop, bd)
    _check(o, lse, got, o_ref, lse_ref, ref)
    _lib.tune_set("attn.variant", 1)
    try:
        o1, lse1 = attn_fwd_strided(qd, kd, vd, (0, 1, 2, 3), causal, None, drop, bd)
    finally:
        _lib.tune_set("attn.variant", -1)
    assert float(((o.float() - o1.float()).abs() - (2e-2 + 2e-2 * o1.float().abs())).max()) <= 0 and float((lse - lse1).abs().max()) <= 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("causal", [False, True])
def test_per_key_bias_properties_at_the_headline_size(causal, dtype):
    # B=2 H=16 S=8192 D=128 bf16 (the 256-row kernel with the bias row in LDS), by what the mathematics fixes: a bias that
    # is the same for every key changes nothing but LSE, which moves by that constant; -inf on the last keys is attention
    # over the keys before them; and the backward of both agrees with the backward without bias
    B, H, S, D = 2, 16, 8192, 128
    assert _kernel_with_key_bias(B, H, S, S, D, causal) == 32
    g = torch.Generator().manual_seed(123)
    q, k, v, go = (torch.randn(B, H, S, D, generator=g).to(dtype).to(DEV) for _ in range(4))
    dims = (0, 1, 2, 3)
    o0, lse0 = attn_fwd_strided(q, k, v, dims, causal, None, None, None)
    const = torch.full((B, 1, 1, S), 1.75, device=DEV)
    o1, lse1 = attn_fwd_strided(q, k, v, dims, causal, None, None, const)
    assert float((o1.float() - o0.float()).abs().max()) <= 2e-2 and float((lse1 - lse0 - 1.75).abs().max()) <= 1e-3
    cut = 5000
    pad = torch.zeros(B, 1, 1, S, device=DEV)
    pad[..., cut:] = float("-inf")
    o2, lse2 = attn_fwd_strided(q, k, v, dims, causal, None, None, pad)
    o3, lse3 = attn_fwd_strided(q, k[:, :, :cut], v[:, :, :cut], dims, causal, None, None, None)
    assert float((o2.float() - o3.float()).abs().max()) <= 2e-2 and float((lse2 - lse3).abs().max()) <= 1e-3
    d0 = attn_bwd_strided(q, k, v, o0, lse0, go, dims, causal, None, None, None)
    d1 = attn_bwd_strided(q, k, v, o1, lse1, go, dims, causal, None, None, const)
    d2 = attn_bwd_strided(q, k, v, o2, lse2, go, dims, causal, None, None, pad)
    d3 = attn_bwd_strided(q, k[:, :, :cut], v[:, :, :cut], o3, lse3, go, dims, causal, None, None, None)
    for name, a, b_ in zip(("dQ", "dK", "dV"), d1, d0):
        assert float((a.float() - b_.float()).abs().max()) <= 2e-2 * max(1.0, float(b_.float().abs().max())), name
    assert float((d2[0].float() - d3[0].float()).abs().max()) <= 2e-2 * max(1.0, float(d3[0].float().abs().max()))
    for a, b_ in ((d2[1], d3[1]), (d2[2], d3[2])):
        assert float((a[:, :, :cut].float() - b_.float()).abs().max()) <= 2e-2 * max(1.0, float(b_.float().abs().max()))
        assert float(a[:, :, cut:].abs().max()) == 0.0
