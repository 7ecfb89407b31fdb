"""Parity of the attention backward kernels (through the C ABI and the autograd Function) with the CPU oracle.

Criterion: the reference's own (tests/test_flash_attention_triton.py:137-141) - the error against the fp32 closed form
must not exceed twice the error of a plain half-precision PyTorch implementation of the same expression, plus an
absolute floor of 1e-3 of the gradient's magnitude for the cases where that implementation happens to be almost exact.
Inputs are drawn on the CPU from a seeded generator, rounded to the operand type, then copied."""
import math

import pytest
import torch

from fast_ops.flash_attention.flash_attention import FlashAttentionFunction, flash_attn, multi_head_attention
from oracle.attention_oracle import attention_bwd_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(B, H, Sq, Sk, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    k = torch.randn(B, H, Sk, D, generator=g).to(dtype)
    v = torch.randn(B, H, Sk, D, generator=g).to(dtype)
    go = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    return q, k, v, go


def _half_precision_torch(q, k, v, go, causal, scale):
    """The expression evaluated by autograd with tensors of the operand type (matmuls accumulate in fp32 inside, results
    and the softmax are rounded to the operand type): the 'PyTorch implementation' of the reference's criterion."""
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    s = (qa * scale) @ ka.transpose(-1, -2)
    if causal:
        M, N = q.shape[2], k.shape[2]
        s = s.masked_fill(torch.arange(N, device=q.device)[None, :] > torch.arange(M, device=q.device)[:, None], float("-inf"))
    o = torch.softmax(s.float(), dim=-1).to(q.dtype) @ va
    return torch.autograd.grad(o, (qa, ka, va), go)


def _check(got, ref, pt, what):
    for name, a, r, p in zip(("dQ", "dK", "dV"), got, ref, pt):
        a = a.float().cpu()
        err = (a - r).abs().max().item()
        base = (p.float() - r).abs().max().item()
        bound = 2.0 * base + 1e-3 * max(1.0, r.abs().max().item())
        assert math.isfinite(err) and err <= bound, f"{what} {name}: error {err:.3e} > 2 x {base:.3e} + floor"


def _run(B, H, Sq, Sk, D, dtype, causal, seed=0, scale=None):
    q, k, v, go = _inputs(B, H, Sq, Sk, D, dtype, seed)
    sc = scale if scale is not None else 1.0 / math.sqrt(D)
    ref = attention_bwd_oracle(q, k, v, go, causal=causal, softmax_scale=sc)
    pt = _half_precision_torch(q, k, v, go, causal, sc)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    o = multi_head_attention(qd, kd, vd, causal=causal, softmax_scale=scale)
    got = torch.autograd.grad(o, (qd, kd, vd), go.to(DEV))
    torch.cuda.synchronize()
    assert all(gr.dtype == dtype and gr.shape == t.shape for gr, t in zip(got, (q, k, v)))
    _check(got, ref, pt, f"B{B} H{H} Sq{Sq} Sk{Sk} D{D} {dtype} causal={causal}")


@pytest.fixture(params=[-1, 0], ids=["dkdv-pipelined", "dkdv-plain"])
def dkdv_variant(request):
    """Both dK/dV kernels: the software-pipelined one (default without dropout and bias) and the plain one."""
    from fast_ops_amd import _lib
    _lib.tune_set("attn_bwd.variant", request.param)
    yield request.param
    _lib.tune_set("attn_bwd.variant", -1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
def test_dtype_causal_headdim_grid(dtype, causal, D, dkdv_variant):
    _run(2, 3, 256, 256, D, dtype, causal, seed=D)


@pytest.mark.parametrize("causal", [False, True])
def test_long_sequence_many_tiles_per_key_block(causal, dkdv_variant):
    # 1024 queries = 16 tiles per key block: the steady state of the tile pipeline, and (causal) every wave's own start
    _run(1, 2, 1024, 1024, 128, torch.bfloat16, causal, seed=11)


@pytest.mark.parametrize("group", [-1, 0, 3, 8, 16, 1000])
@pytest.mark.parametrize("heads", [(4, 5), (3, 8)])
def test_workgroup_order_head_groups(group, heads):
    # attn_bwd.order: how many heads form a group in the order of the workgroups of the dQ and dK/dV kernels (0: all,
    # -1: the library's choice). Every (head, block) must be computed exactly once whatever the grouping, also when the
    # last group is smaller than the others (20 heads in groups of 3, 8 or 16).
    from fast_ops_amd import _lib
    B, H = heads
    _lib.tune_set("attn_bwd.order", group)
    try:
        _run(B, H, 300, 300, 64, torch.bfloat16, True, seed=21)
    finally:
        _lib.tune_set("attn_bwd.order", -1)


@pytest.mark.parametrize("causal", [True, False])
def test_long_context_slice_of_headline_shape(causal, dkdv_variant):
    # one (batch, head) slice of the benchmark shape S=8192 D=128 bf16 against the fp32 closed form: 128 query tiles per
    # key block, the last ones far behind the first. Absolute criterion (the half-precision PyTorch yardstick of the
    # other tests takes minutes on a CPU at this size): error within 2 % of the gradient's largest magnitude.
    q, k, v, go = _inputs(1, 1, 8192, 8192, 128, torch.bfloat16, seed=8192)
    ref = attention_bwd_oracle(q, k, v, go, causal=causal)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    o = multi_head_attention(qd, kd, vd, causal=causal)
    got = torch.autograd.grad(o, (qd, kd, vd), go.to(DEV))
    for name, a, r in zip(("dQ", "dK", "dV"), got, ref):
        e = (a.float().cpu() - r).abs().max().item()
        assert math.isfinite(e) and e <= 2e-2 * max(1.0, r.abs().max().item()), f"{name}: error {e:.3e} vs magnitude {r.abs().max().item():.3e}"


def test_headline_shape_whole_with_the_benchmarks_dispatch():
    # B=2 H=16 S=8192 D=128 bf16 causal as bench.py runs it: 32 heads dealt to the 8 XCDs, 64 key blocks and 64 query
    # blocks per head, the library's own choice of kernels and workgroup order. Six (batch, head) slices that lie on six
    # different XCDs, first and last head included, against the fp32 closed form: the first and the last slice by the
    # reference's criterion (tests/test_flash_attention_triton.py:137-141: at most twice the error of the same expression in
    # the operand dtype, which is run on the GPU here as the reference runs it), the others by the absolute criterion.
    B, H, S, D = 2, 16, 8192, 128
    q, k, v, go = _inputs(B, H, S, S, D, torch.bfloat16, seed=4)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    o = multi_head_attention(qd, kd, vd, causal=True)
    got = [g.cpu() for g in torch.autograd.grad(o, (qd, kd, vd), go.to(DEV))]
    slices = [(0, 0), (0, 5), (0, 10), (1, 3), (1, 9), (1, 15)]
    assert len({(b * H + h) % 8 for b, h in slices}) == 6
    for b, h in slices:
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = attention_bwd_oracle(q[sl], k[sl], v[sl], go[sl], causal=True)
        if (b, h) in ((0, 0), (1, 15)):
            pt = [t.cpu() for t in _half_precision_torch(q[sl].to(DEV), k[sl].to(DEV), v[sl].to(DEV), go[sl].to(DEV), True, 1.0 / math.sqrt(D))]
            _check([a[sl] for a in got], ref, pt, f"headline shape, slice ({b},{h})")
            continue
        for name, a, r in zip(("dQ", "dK", "dV"), got, ref):
            e = (a[sl].float() - r).abs().max().item()
            assert math.isfinite(e) and e <= 2e-2 * max(1.0, r.abs().max().item()), f"slice ({b},{h}) {name}: error {e:.3e} vs magnitude {r.abs().max().item():.3e}"


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (1, 2, 7, 5), (2, 1, 100, 100), (1, 3, 129, 257), (1, 2, 257, 129), (1, 1, 64, 300),
                                   (1, 1, 300, 64), (2, 2, 191, 191), (1, 1, 385, 513)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
def test_ragged_and_unequal_lengths(shape, causal, D, dkdv_variant):
    # lengths that are not multiples of the 128-row blocks / 64-row tiles, Sq != Sk (causal mask top-left aligned: keys
    # beyond the last query get exactly zero gradient)
    B, H, Sq, Sk = shape
    _run(B, H, Sq, Sk, D, torch.bfloat16, causal, seed=Sq * 1000 + Sk)


def test_config2_gpt2_small_shape_slice():
    _run(2, 12, 1024, 1024, 64, torch.bfloat16, True, seed=2)


@pytest.mark.parametrize("D", [8, 16, 24, 32, 40, 48, 56, 72, 80, 88, 96, 104, 112, 120])
def test_every_other_head_dim_of_the_reference_contract(D):
    # any multiple of 8 up to 128 (flash_attention.py:61-66), inside the kernels: no padded copies
    _run(1, 2, 150, 210, D, torch.float16, True, seed=D)
    _run(1, 2, 97, 97, D, torch.bfloat16, False, seed=D + 1, scale=0.3)


def test_keys_no_query_attends_get_zero_gradient():
    q, k, v, go = _inputs(1, 2, 100, 400, 128, torch.bfloat16, 5)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    o = multi_head_attention(qd, kd, vd, causal=True)
    _, dk, dv = torch.autograd.grad(o, (qd, kd, vd), go.to(DEV))
    assert float(dk[:, :, 100:].abs().max()) == 0.0 and float(dv[:, :, 100:].abs().max()) == 0.0


def test_bshd_surface_multi_query_and_packed_views():
    # [batch, seqlen, nheads, headdim] inputs; K/V shared across heads through expand: autograd sums the per-head
    # gradients the kernel writes; Q/K/V as slices of one packed projection output
    B, S, H, D = 2, 200, 4, 64
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16)
    kv = torch.randn(B, S, 2, 1, D, generator=g).to(torch.bfloat16)
    go = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16)
    k1, v1 = kv.unbind(2)
    kx, vx = k1.expand(B, S, H, D), v1.expand(B, S, H, D)
    tr = lambda t: t.transpose(1, 2)
    dq_r, dk_r, dv_r = attention_bwd_oracle(tr(q), tr(kx), tr(vx), tr(go), causal=True)
    pt = _half_precision_torch(tr(q).contiguous(), tr(kx).contiguous(), tr(vx).contiguous(), tr(go).contiguous(), True, 1 / math.sqrt(D))
    qd = q.to(DEV).requires_grad_(True)
    kvd = kv.to(DEV).requires_grad_(True)
    kd, vd = (t.expand(B, S, H, D) for t in kvd.unbind(2))
    o = flash_attn(qd, kd, vd, causal=True)
    dq, dkv = torch.autograd.grad(o, (qd, kvd), go.to(DEV))
    ref = (tr(dq_r), tr(dk_r).sum(2, keepdim=True), tr(dv_r).sum(2, keepdim=True))
    ptr = (tr(pt[0]), tr(pt[1]).float().sum(2, keepdim=True), tr(pt[2]).float().sum(2, keepdim=True))
    _check((dq, dkv[:, :, 0], dkv[:, :, 1]), ref, ptr, "BSHD multi-query")
    # packed projection
    qkv = torch.randn(B, S, 3, H, D, generator=g).to(torch.bfloat16)
    qkvd = qkv.to(DEV).requires_grad_(True)
    o = flash_attn(qkvd[:, :, 0], qkvd[:, :, 1], qkvd[:, :, 2], causal=False)
    (dqkv,) = torch.autograd.grad(o, (qkvd,), go.to(DEV))
    r = attention_bwd_oracle(tr(qkv[:, :, 0]), tr(qkv[:, :, 1]), tr(qkv[:, :, 2]), tr(go), causal=False)
    p = _half_precision_torch(*(tr(qkv[:, :, i]).contiguous() for i in range(3)), tr(go).contiguous(), False, 1 / math.sqrt(D))
    _check(tuple(dqkv[:, :, i] for i in range(3)), tuple(tr(x) for x in r), tuple(tr(x) for x in p), "packed qkv")


def test_gradients_are_deterministic():
    q, k, v, go = _inputs(2, 4, 512, 512, 128, torch.bfloat16, 9)
    outs = []
    for _ in range(2):
        qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
        o = FlashAttentionFunction.apply(qd, kd, vd, True)
        outs.append(torch.autograd.grad(o, (qd, kd, vd), go.to(DEV)))
    assert all(torch.equal(a, b) for a, b in zip(*outs))


@pytest.mark.parametrize("D,row", [(40, 48), (8, 16), (104, 128), (56, 64)])
@pytest.mark.parametrize("causal", [False, True])
def test_columns_past_the_head_dim_are_neither_read_nor_written(D, row, causal):
    """Operands and results as views of wider tensors (row stride `row` > head_dim D) whose extra columns hold NaN: a
    kernel that read a column past D would turn its results into NaN, one that wrote there would overwrite the NaN."""
    B, H, Sq, Sk = 2, 3, 150, 210
    q, k, v, go = _inputs(B, H, Sq, Sk, D, torch.bfloat16, seed=D + row)
    sc = 1.0 / math.sqrt(D)
    ref = attention_bwd_oracle(q, k, v, go, causal=causal, softmax_scale=sc)
    pt = _half_precision_torch(q, k, v, go, causal, sc)

    def wide(t):
        w = torch.full(t.shape[:-1] + (row,), float("nan"), dtype=t.dtype, device=DEV)
        w[..., :D] = t.to(DEV)
        return w

    qw, kw, vw, gw = wide(q), wide(k), wide(v), wide(go)
    from fast_ops_amd.flash_attention.flash_attention import attn_bwd_strided, attn_fwd_strided
    o, lse = attn_fwd_strided(qw[..., :D], kw[..., :D], vw[..., :D], (0, 1, 2, 3), causal, sc)
    assert bool(torch.isfinite(o.float()).all()) and bool(torch.isfinite(lse).all())
    from oracle.attention_oracle import attention_fwd_oracle
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal, softmax_scale=sc)
    assert float((o.float().cpu() - o_ref).abs().max()) <= 2e-2 and float((lse.cpu() - lse_ref).abs().max()) <= 1e-3
    ow = wide(o.cpu())
    got = attn_bwd_strided(qw[..., :D], kw[..., :D], vw[..., :D], ow[..., :D], lse, gw[..., :D], (0, 1, 2, 3), causal, sc)
    torch.cuda.synchronize()
    _check(got, ref, pt, f"D{D} in rows of {row} causal={causal}")
    # results written into views of wider buffers through the C ABI: the columns past D keep their contents
    import ctypes
    from fast_ops_amd import _lib
    I3 = ctypes.c_int64 * 3
    P64 = ctypes.POINTER(ctypes.c_int64)
    outs = [torch.full(t.shape[:-1] + (row,), 7.0, dtype=torch.bfloat16, device=DEV) for t in (q, k, v)]
    o_out = torch.full(q.shape[:-1] + (row,), 7.0, dtype=torch.bfloat16, device=DEV)
    lse2 = torch.empty(B, H, Sq, dtype=torch.float32, device=DEV)
    st = lambda t: I3(*t.stride()[:3])
    stream = torch.cuda.current_stream().cuda_stream
    rc = _lib.load().fo_attn_fwd(qw.data_ptr(), kw.data_ptr(), vw.data_ptr(), o_out.data_ptr(), lse2.data_ptr(), B, H, Sq, Sk, D,
                                 st(qw), st(kw), st(vw), st(o_out), sc, int(causal), _lib.FO_DTYPE_BF16, stream)
    assert rc == 0, _lib.strerror(rc)
    delta = torch.empty(2, B, H, Sq, dtype=torch.float32, device=DEV)
    tensors = (qw, kw, vw, ow, gw, outs[0], outs[1], outs[2])
    arrays = [st(t) for t in tensors]
    strides = (P64 * 8)(*[ctypes.cast(a, P64) for a in arrays])
    rc = _lib.load().fo_attn_bwd(qw.data_ptr(), kw.data_ptr(), vw.data_ptr(), ow.data_ptr(), gw.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                                 outs[0].data_ptr(), outs[1].data_ptr(), outs[2].data_ptr(), B, H, Sq, Sk, D, strides, sc, int(causal),
                                 _lib.FO_DTYPE_BF16, stream)
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    assert torch.equal(o_out[..., :D], o)
    for w, g_ in zip(outs + [o_out], list(got) + [o]):
        assert torch.equal(w[..., :D], g_)
        assert bool((w[..., D:] == 7.0).all()), "a column past the head_dim was written"
