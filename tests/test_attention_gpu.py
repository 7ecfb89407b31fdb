"""Parity of the attention forward kernel (through the C ABI) with the CPU oracle.

Tolerances are the ones the task states: O within atol 2e-2 / rtol 1e-2 of fp32 softmax(scale Q K^T) V computed
from the same half-precision inputs, LSE within 1e-3 (absolute). Inputs are drawn on the CPU from a seeded
generator in fp32, rounded to the operand type, then copied, so both sides see identical bits."""
import math
import os

import numpy as np
import pytest
import torch

from fast_ops.flash_attention.flash_attention import FlashAttentionFunction, flash_attn, multi_head_attention
from fast_ops_amd import _lib
from oracle.attention_oracle import attention_fwd_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
O_ATOL, O_RTOL, LSE_ATOL = 2e-2, 1e-2, 1e-3
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "attn_small.npz")


def _qkv(B, H, Sq, Sk, D, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    k = torch.randn(B, H, Sk, D, generator=g).to(dtype)
    v = torch.randn(B, H, Sk, D, generator=g).to(dtype)
    return q, k, v


def _check(o, lse, o_ref, lse_ref, what=""):
    o = o.float().cpu()
    lse = lse.cpu()
    err = (o - o_ref).abs()
    bound = O_ATOL + O_RTOL * o_ref.abs()
    worst = float((err - bound).max())
    assert worst <= 0, f"{what}: O outside atol {O_ATOL} / rtol {O_RTOL} by {worst:.3e} (max abs err {float(err.max()):.3e})"
    lse_err = float((lse - lse_ref).abs().max())
    assert lse_err <= LSE_ATOL, f"{what}: LSE error {lse_err:.3e} > {LSE_ATOL}"
    return float(err.max()), lse_err


# attn.variant values: -1 = the library's choice (which depends on head_dim and on how many workgroups the shape gives),
# 8 = 128 rows per workgroup in the pipelined kernel (four waves x 32 rows),
# 0 = the 128-row kernel, 16 / 32 = the 256-row kernel with eight / four waves
KERNELS_D128 = [-1, 0, 8, 16, 32]


@pytest.fixture
def kernel_variant(request):
    _lib.tune_set("attn.variant", request.param)
    yield request.param
    _lib.tune_set("attn.variant", -1)


def _kernel_taken(t_q, t_k, t_v, causal):
    """The kernel the library launches for these [B, H, S, D] tensors with the current attn.variant (fo_attn_fwd_kernel)."""
    import ctypes

    I3 = ctypes.c_int64 * 3
    B, H, Sq, D = t_q.shape
    code = _lib.load().fo_attn_fwd_kernel(B, H, Sq, t_k.shape[2], D, I3(*t_k.stride()[:3]), I3(*t_v.stride()[:3]), int(causal), 0, 0)
    assert code >= 0, _lib.strerror(code)
    return code


def _run_and_check(B, H, Sq, Sk, D, dtype, causal, seed=0, scale=None):
    q, k, v = _qkv(B, H, Sq, Sk, D, dtype, seed)
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal, softmax_scale=scale)
    o, lse = multi_head_attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, softmax_scale=scale, return_lse=True)
    torch.cuda.synchronize()
    assert o.dtype == dtype and o.shape == q.shape and lse.dtype == torch.float32 and lse.shape == (B, H, Sq)
    return _check(o, lse, o_ref, lse_ref, f"B{B} H{H} Sq{Sq} Sk{Sk} D{D} {dtype} causal={causal}")


def test_config1_tiny_fp16_noncausal():
    # B=2 H=4 S=128 D=64, fp16, non-causal, scale 1/8
    _run_and_check(2, 4, 128, 128, 64, torch.float16, False, seed=0, scale=0.125)


def test_config2_gpt2_small_bf16_causal():
    # B=8 H=12 S=1024 D=64, bf16, causal, scale 1/8
    _run_and_check(8, 12, 1024, 1024, 64, torch.bfloat16, True, seed=0, scale=0.125)


@pytest.mark.parametrize("group", [-1, 0, 1, 2, 3, 5, 1000])
@pytest.mark.parametrize("heads", [(2, 4), (5, 8), (3, 5)])
def test_causal_workgroup_order_of_128_row_kernel(group, heads):
    # attn.order: how many of an XCD's heads form a group whose heaviest query blocks run first (0: head by head, -1:
    # the library's choice). Every (head, query block) must be computed exactly once whatever the grouping, also when the
    # last group is smaller than the others (40 heads = 5 per XCD in groups of 2 or 3) and when the number of heads is no
    # multiple of the 8 XCDs (15 heads: the grouping does not apply).
    B, H = heads
    _lib.tune_set("attn.variant", 0)
    _lib.tune_set("attn.order", group)
    try:
        _run_and_check(B, H, 700, 700, 64, torch.bfloat16, True, seed=11)
    finally:
        _lib.tune_set("attn.variant", -1)
        _lib.tune_set("attn.order", -1)


@pytest.mark.parametrize("balance", [-1, 0])
@pytest.mark.parametrize("shape", [(8, 12, 1024, 64), (4, 16, 1024, 64), (5, 8, 700, 64), (2, 20, 1100, 64), (8, 5, 1536, 128), (3, 8, 900, 128), (8, 9, 1024, 64)])
def test_balanced_order_of_a_launch_that_fits_the_chip_at_once(shape, balance):
    # attn.balance: a causal launch of the 128-row kernel whose workgroups are all resident at once takes its order from a
    # table (heaviest first, each to the compute unit with the least work so far) - whole shapes against the oracle, with
    # the table (33 to 96 workgroups per XCD: full and ragged last layers, two and three layers) and without it
    B, H, S, D = shape
    _lib.tune_set("attn.variant", 0)
    _lib.tune_set("attn.balance", balance)
    try:
        _run_and_check(B, H, S, S, D, torch.bfloat16, True, seed=S + H)
    finally:
        _lib.tune_set("attn.variant", -1)
        _lib.tune_set("attn.balance", -1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
def test_dtype_causal_headdim_grid(dtype, causal, D):
    _run_and_check(2, 3, 512, 512, D, dtype, causal, seed=3)


@pytest.mark.parametrize("kernel_variant", [0, 8, 16, 32], indirect=True)
def test_long_context_slice_of_headline_shape(kernel_variant):
    # the headline shape is B=2 H=16 S=8192 D=128 bf16 causal; two of its (batch, head) slices against the oracle, on each
    # of the three kernels (so few slices leave the choice to the 128-row kernel; the full shape is tested below)
    _run_and_check(1, 2, 8192, 8192, 128, torch.bfloat16, True, seed=0)


@pytest.mark.parametrize("shape", [(1, 12, 2048, 128, True), (1, 12, 2048, 128, False), (1, 12, 4096, 64, True), (2, 6, 1024, 128, True)])
def test_few_heads_take_the_128_row_pipelined_form(shape):
    # the reference's own benchmark shapes, 12 heads per GPU (flash_attention/README.md:69-70): too few workgroups for the
    # chip, so the library picks 128-row workgroups in the pipelined kernel; whole shape against the oracle
    B, H, S, D, causal = shape
    q, k, v = _qkv(B, H, S, S, D, torch.bfloat16, seed=S + D)
    assert _kernel_taken(q, k, v, causal) == _lib.FO_ATTN_KERNEL_ROWS128_PIPE
    _run_and_check(B, H, S, S, D, torch.bfloat16, causal, seed=S + D)


def test_throughput_shape_slice_fp16_noncausal():
    # B=16 H=32 S=2048 D=128 fp16 non-causal; 8 of its (batch, head) slices (the full shape is tested below)
    _run_and_check(1, 8, 2048, 2048, 128, torch.float16, False, seed=0)


def _full_shape_against_oracle(B, H, S, D, dtype, causal, slices, expect_kernel):
    """The whole benchmark shape through multi_head_attention with the library's own kernel choice (asserted, not
    assumed), then the listed (batch, head) slices of the result against the oracle."""
    q, k, v = _qkv(B, H, S, S, D, dtype, seed=0)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    assert _lib.load().fo_tune_get(b"attn.variant") == -1
    assert _kernel_taken(qd, kd, vd, causal) == expect_kernel, "the benchmark shape does not take the kernel this test is for"
    o, lse = multi_head_attention(qd, kd, vd, causal=causal, return_lse=True)
    torch.cuda.synchronize()
    o, lse = o.cpu(), lse.cpu()
    worst_o = worst_lse = 0.0
    for b, h in slices:
        o_ref, lse_ref = attention_fwd_oracle(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], causal=causal)
        eo, el = _check(o[b:b + 1, h:h + 1], lse[b:b + 1, h:h + 1], o_ref, lse_ref, f"B{B} H{H} S{S} D{D} {dtype} causal={causal} slice ({b},{h})")
        worst_o, worst_lse = max(worst_o, eo), max(worst_lse, el)
    print(f"{len(slices)} slices: max |O err| {worst_o:.3e}, max |LSE err| {worst_lse:.3e}")


def test_headline_shape_on_the_kernel_the_benchmark_times():
    # B=2 H=16 S=8192 D=128 bf16 causal, all 32 (batch, head) slices: 256-row kernel (four waves x 64 rows at this length),
    # XCD-mapped workgroup order, 16 items of two query blocks per head
    _full_shape_against_oracle(2, 16, 8192, 128, torch.bfloat16, True, [(b, h) for b in range(2) for h in range(16)],
                               _lib.FO_ATTN_KERNEL_ROWS256_W4)


def test_throughput_shape_on_the_kernel_the_benchmark_times():
    # B=16 H=32 S=2048 D=128 fp16 non-causal (512 heads x 8 items): the first and the last batch element complete and every
    # fifth slice in between - 154 slices, heads 0..31 and every XCD among them
    slices = [(b, h) for b in range(16) for h in range(32) if b in (0, 15) or (b * 32 + h) % 5 == 0]
    assert {(b * 32 + h) % 8 for b, h in slices} == set(range(8)) and max(h for _, h in slices) == 31
    _full_shape_against_oracle(16, 32, 2048, 128, torch.float16, False, slices, _lib.FO_ATTN_KERNEL_ROWS256_W4)


def test_mid_length_causal_shape_takes_the_eight_wave_form_by_default():
    # B=2 H=16 S=4096 D=128 bf16 causal: long enough for the 256-row kernel, too short for its four-wave form
    _full_shape_against_oracle(2, 16, 4096, 128, torch.bfloat16, True, [(b, h) for b in range(2) for h in range(16)],
                               _lib.FO_ATTN_KERNEL_ROWS256_W8)


@pytest.mark.parametrize("kernel_variant", [16, 32], indirect=True)
def test_headline_shape_on_both_forms_of_the_256_row_kernel(kernel_variant):
    # the whole headline shape forced onto each form (8 of its 32 slices against the oracle; the default form is checked on
    # all of them above)
    B, H, S, D = 2, 16, 8192, 128
    q, k, v = _qkv(B, H, S, S, D, torch.bfloat16, seed=0)
    o, lse = multi_head_attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=True, return_lse=True)
    torch.cuda.synchronize()
    o, lse = o.cpu(), lse.cpu()
    for b, h in [(0, 0), (0, 5), (0, 10), (0, 15), (1, 3), (1, 6), (1, 9), (1, 12)]:
        o_ref, lse_ref = attention_fwd_oracle(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], causal=True)
        _check(o[b:b + 1, h:h + 1], lse[b:b + 1, h:h + 1], o_ref, lse_ref, f"variant {kernel_variant} slice ({b},{h})")


@pytest.mark.parametrize("shape", [(1, 8, 1300, 1300), (2, 8, 800, 1000), (3, 8, 1111, 900), (1, 16, 1537, 1537)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("kernel_variant", [8, 16, 32], indirect=True)
def test_256_row_kernel_with_heads_dealt_to_xcds_and_several_items_per_head(shape, causal, D, kernel_variant):
    # 8, 16 and 24 heads (a multiple of the 8 XCDs: workgroup id -> (XCD, head, item)) with 3 to 7 items per head, ragged
    # lengths; causal items are pairs of query blocks, the middle one single when their number is odd
    B, H, Sq, Sk = shape
    q, k, v = _qkv(B, H, Sq, Sk, D, torch.bfloat16, seed=Sq + Sk + D)
    assert _kernel_taken(q, k, v, causal) == kernel_variant
    _run_and_check(B, H, Sq, Sk, D, torch.bfloat16, causal, seed=Sq + Sk + D)


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (1, 2, 7, 5), (2, 1, 100, 100), (1, 3, 129, 257), (1, 2, 257, 129), (1, 1, 64, 1000), (1, 1, 1000, 64), (3, 5, 191, 191)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("kernel_variant", KERNELS_D128, indirect=True)
def test_ragged_and_unequal_lengths(shape, causal, D, kernel_variant):
    # sequence lengths that are not multiples of the 128-row / 64-key tiles, Sq != Sk (causal mask is top-left aligned)
    B, H, Sq, Sk = shape
    _run_and_check(B, H, Sq, Sk, D, torch.bfloat16, causal, seed=Sq * 1000 + Sk)


# (B, H, Sq, Sk, D, causal): more work items than the chip has CUs, so that with attn.keep_on 2 (the default) a workgroup of
# the 256-row kernel (both forms) walks several of them and copies the next block's first tiles during a block's last ones
# (key counts that are a multiple of 256) or falls back to waiting (the others); heads in and out of the XCD dealing
# (multiples of 8 or not); a ragged last key tile; fewer key tiles than the three copied ahead; Sq above Sk when causal.
WALKED = [(4, 40, 1024, 1024, 128, False), (4, 40, 1000, 1000, 128, True), (3, 37, 900, 700, 64, False), (5, 24, 1536, 100, 128, False),
          (2, 64, 2048, 2048, 64, True), (2, 72, 2048, 512, 128, True), (3, 24, 1280, 1280, 128, True), (2, 40, 1792, 1000, 64, False)]


@pytest.mark.parametrize("shape", WALKED)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("form", [_lib.FO_ATTN_KERNEL_ROWS256_W4, _lib.FO_ATTN_KERNEL_ROWS256_W8])
def test_work_items_walked_by_one_workgroup_per_cu(shape, dtype, form):
    B, H, Sq, Sk, D, causal = shape
    q, k, v = _qkv(B, H, Sq, Sk, D, dtype, seed=Sq + Sk)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    got = {}
    _lib.tune_set("attn.variant", form)
    try:
        assert _kernel_taken(qd, kd, vd, causal) == form
        for mode in (0, 1, 2, -1):
            _lib.tune_set("attn.keep_on", mode)
            # (the allocator hands the blocks freed last to the next request of their size: the outputs start as NaN, and
            # a block that nobody worked on would show)
            o = lse = None
            junk = (torch.full_like(qd, float("nan")), torch.full((B, H, Sq), float("nan"), device=DEV))
            del junk
            o, lse = multi_head_attention(qd, kd, vd, causal=causal, return_lse=True)
            torch.cuda.synchronize()
            got[mode] = (o.cpu(), lse.cpu())
            assert torch.isfinite(got[mode][0].float()).all() and torch.isfinite(got[mode][1]).all(), f"attn.keep_on {mode}"
    finally:
        _lib.tune_set("attn.keep_on", -1)
        _lib.tune_set("attn.variant", -1)
    # the same arithmetic in the same order whoever walks the items: identical bits
    for mode in (1, 2, -1):
        assert torch.equal(got[0][0], got[mode][0]) and torch.equal(got[0][1], got[mode][1]), f"attn.keep_on {mode} differs from 0"
    o, lse = got[2]
    for b, h in [(0, 0), (B - 1, H - 1), (B // 2, H // 3), (B - 1, 7)]:
        o_ref, lse_ref = attention_fwd_oracle(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], causal=causal)
        _check(o[b:b + 1, h:h + 1], lse[b:b + 1, h:h + 1], o_ref, lse_ref, f"{shape} {dtype} slice ({b},{h})")


# (B, H, Sq, Sk): non-causal head_dim 128 shapes whose 256-row work items fill one or more rounds of one workgroup per CU
# and leave a last round that is at most half full (on 256 CUs: 384 = 256 + 128, 640 = 512 + 128, 264 = 256 + 8, and 330
# with heads that are not dealt to XCDs and a last block of 44 rows, whose second 128-row half does not exist): the items
# of that round go to a second launch of the 128-row pipelined form (attn.tail, default on).
TAILS = [(1, 12, 8192, 2048), (4, 40, 1024, 2100), (1, 8, 8448, 2048), (2, 15, 2604, 2500)]


@pytest.mark.parametrize("shape", TAILS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("with_bias", [False, True])
def test_last_round_handed_to_the_128_row_form(shape, dtype, with_bias):
    from fast_ops_amd.flash_attention.flash_attention import attn_fwd_strided

    B, H, Sq, Sk = shape
    D = 128
    q, k, v = _qkv(B, H, Sq, Sk, D, dtype, seed=Sq)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    bias = None
    if with_bias:
        bias = torch.randn(B, 1, 1, Sk, generator=torch.Generator().manual_seed(Sk)).to(dtype)   # one value per key
    got = {}
    _lib.tune_set("attn.variant", _lib.FO_ATTN_KERNEL_ROWS256_W4)
    try:
        assert _kernel_taken(qd, kd, vd, False) == _lib.FO_ATTN_KERNEL_ROWS256_W4
        for mode in (0, 1):
            _lib.tune_set("attn.tail", mode)
            junk = (torch.full_like(qd, float("nan")), torch.full((B, H, Sq), float("nan"), device=DEV))   # (see the test above)
            del junk
            o, lse = attn_fwd_strided(qd, kd, vd, (0, 1, 2, 3), False, None, None, None if bias is None else bias.to(DEV))
            torch.cuda.synchronize()
            got[mode] = (o.cpu(), lse.cpu())
            assert torch.isfinite(got[mode][0].float()).all() and torch.isfinite(got[mode][1]).all(), f"attn.tail {mode}"
    finally:
        _lib.tune_set("attn.tail", -1)
        _lib.tune_set("attn.variant", -1)
    # two forms of one pipeline: the same scores and sums, P rounded against references that may differ
    assert float((got[0][1] - got[1][1]).abs().max()) <= 1e-4
    assert float(((got[0][0].float() - got[1][0].float()).abs() - (2e-2 + 2e-2 * got[0][0].float().abs())).max()) <= 0
    o, lse = got[1]
    for b, h in [(0, 0), (B - 1, H - 1), (B - 1, H // 2)]:          # the last heads are the ones in the last round
        o_ref, lse_ref = attention_fwd_oracle(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1],
                                              bias=None if bias is None else bias[b:b + 1])
        _check(o[b:b + 1, h:h + 1], lse[b:b + 1, h:h + 1], o_ref, lse_ref, f"{shape} {dtype} bias={with_bias} slice ({b},{h})")


@pytest.mark.parametrize("shape", [(1, 2, 600, 700), (1, 1, 513, 1025), (2, 2, 255, 64), (1, 1, 770, 770)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("kernel_variant", KERNELS_D128, indirect=True)
def test_ragged_across_256_row_blocks_and_ring_wraps(shape, causal, dtype, kernel_variant):
    # head_dim 128 works on 256-row query blocks (two per workgroup when causal) and a four-slot ring of key tiles
    B, H, Sq, Sk = shape
    _run_and_check(B, H, Sq, Sk, 128, dtype, causal, seed=Sq + Sk)


@pytest.mark.parametrize("shape", [(1, 2, 600, 700), (1, 1, 513, 1025), (2, 2, 255, 64), (1, 1, 770, 770)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("kernel_variant", KERNELS_D128, indirect=True)
def test_ragged_across_256_row_blocks_head_dim_64(shape, causal, dtype, kernel_variant):
    B, H, Sq, Sk = shape
    _run_and_check(B, H, Sq, Sk, 64, dtype, causal, seed=Sq + Sk + 64)


@pytest.mark.parametrize("causal,S,heads", [(True, 16384, 8), (True, 8192, 16), (False, 8192, 8), (False, 4096, 16)])
def test_head_dim_64_long_shape_takes_the_256_row_kernel_by_default(causal, S, heads):
    # head_dim 64 takes the 256-row kernel, as four waves x 64 rows, only for long rows of keys (from 4096 non-causal,
    # 8192 causal) and at least one workgroup per CU: the library's own choice, and it must agree with the oracle
    q, k, v = _qkv(1, heads, S, S, 64, torch.bfloat16, seed=5)
    assert _kernel_taken(q, k, v, causal) == _lib.FO_ATTN_KERNEL_ROWS256_W4
    _run_and_check(1, heads, S, S, 64, torch.bfloat16, causal, seed=5)


@pytest.mark.parametrize("causal,S", [(True, 2304), (False, 1024)])
def test_head_dim_64_shorter_shape_takes_the_128_row_kernel_by_default(causal, S):
    q, k, v = _qkv(2, 40, S, S, 64, torch.bfloat16, seed=5)
    assert _kernel_taken(q, k, v, causal) == _lib.FO_ATTN_KERNEL_ROWS128
    _run_and_check(2, 40, S, S, 64, torch.bfloat16, causal, seed=5)


@pytest.mark.parametrize("heads,expect", [(128, "rows256_w8"), (192, "rows128")])
def test_short_causal_head_dim_128_choice_follows_the_fill_of_the_rounds(heads, expect):
    # B*H heads x 1024 queries, causal: two workgroups of two 256-row blocks per head. 128 heads fill the 256 CUs once
    # (256-row kernel); 192 heads would leave half of a second round empty (128-row kernel). Checked against the oracle
    # on a sample of heads that covers every XCD.
    B, H, S, D = heads // 16, 16, 1024, 128
    q, k, v = _qkv(B, H, S, S, D, torch.bfloat16, seed=heads)
    want = {"rows256_w8": _lib.FO_ATTN_KERNEL_ROWS256_W8, "rows128": _lib.FO_ATTN_KERNEL_ROWS128}[expect]
    assert _kernel_taken(q, k, v, True) == want
    o, lse = multi_head_attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=True, return_lse=True)
    torch.cuda.synchronize()
    o, lse = o.cpu(), lse.cpu()
    for i in range(0, heads, 11):
        b, h = divmod(i, H)
        o_ref, lse_ref = attention_fwd_oracle(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], causal=True)
        _check(o[b:b + 1, h:h + 1], lse[b:b + 1, h:h + 1], o_ref, lse_ref, f"{expect} head {i}")


def test_causal_up_to_2048_queries_takes_the_128_row_kernel_by_default():
    q, k, v = _qkv(2, 40, 2048, 2048, 64, torch.bfloat16, seed=5)
    assert _kernel_taken(q, k, v, True) == _lib.FO_ATTN_KERNEL_ROWS128
    _run_and_check(2, 40, 2048, 2048, 64, torch.bfloat16, True, seed=5)


@pytest.mark.parametrize("pattern", ["growing", "shrinking", "spikes"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("kernel_variant", KERNELS_D128, indirect=True)
def test_moving_row_maximum(pattern, causal, D, dtype, kernel_variant):
    # scores whose row maximum keeps moving (or sits far above the rest) exercise the rescaling of the running
    # softmax state: keys scaled so that scaled scores span tens of units
    B, H, Sq, Sk = 1, 2, 384, 640
    q, k, v = _qkv(B, H, Sq, Sk, D, torch.float32, seed=7)
    pos = torch.arange(Sk, dtype=torch.float32)
    if pattern == "growing":
        gain = 0.5 + 6.0 * pos / Sk
    elif pattern == "shrinking":
        gain = 6.5 - 6.0 * pos / Sk
    else:
        gain = torch.where(pos % 97 == 5, torch.tensor(12.0), torch.tensor(1.0))
    k = k * gain[None, None, :, None]
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=causal)
    o, lse = multi_head_attention(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, return_lse=True)
    torch.cuda.synchronize()
    _check(o, lse, o_ref, lse_ref, f"{pattern} D{D} {dtype} causal={causal}")


@pytest.mark.parametrize("D", [8, 16, 24, 32, 40, 48, 56, 72, 80, 88, 96, 104, 112, 120])
@pytest.mark.parametrize("causal", [False, True])
def test_every_head_dim_of_the_reference_contract(D, causal):
    # head_dim any multiple of 8 up to 128 (flash_attention.py:61-66), inside the kernels (no padded copies); default
    # scale is 1/sqrt(true head_dim)
    _run_and_check(2, 3, 150, 210, D, torch.float16, causal, seed=D)
    _run_and_check(1, 2, 97, 97, D, torch.bfloat16, causal, seed=D + 1, scale=0.3)


def test_golden_fixture():
    z = np.load(GOLDEN)
    to16 = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.float16)
    q, k, v = (to16(z[n]).to(DEV) for n in "qkv")
    for tag, causal in (("full", False), ("causal", True)):
        o, lse = multi_head_attention(q, k, v, causal=causal, softmax_scale=float(z["scale"]), return_lse=True)
        _check(o, lse, torch.from_numpy(z[f"o_{tag}"]), torch.from_numpy(z[f"lse_{tag}"]), f"golden {tag}")


@pytest.mark.parametrize("kernel_variant", KERNELS_D128, indirect=True)
def test_bshd_surface_and_multi_query(kernel_variant):
    # [batch, seqlen, nheads, headdim] inputs (flash_attention_triton.py:734-737); K/V shared across heads via expand,
    # as tests/test_flash_attention_triton.py:71-73 does
    B, S, H, D = 2, 300, 4, 128
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16)
    kv = torch.randn(B, S, 2, 1, D, generator=g).to(torch.bfloat16)
    k, v = kv.unbind(2)
    k, v = k.expand(B, S, H, D), v.expand(B, S, H, D)
    o_ref, lse_ref = attention_fwd_oracle(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), causal=True)
    qd = q.to(DEV)
    kd, vd = (t.to(DEV).expand(B, S, H, D) for t in kv.unbind(2))
    o, lse = flash_attn(qd, kd, vd, causal=True, return_lse=True)
    assert o.shape == (B, S, H, D)
    _check(o.transpose(1, 2), lse, o_ref, lse_ref, "BSHD multi-query")
    with pytest.raises(RuntimeError, match="bias"):
        flash_attn(qd, kd, vd, bias=torch.zeros(1, device=DEV))
    with pytest.raises(RuntimeError, match="dropout_p"):
        flash_attn(qd, kd, vd, dropout_p=1.5)


@pytest.mark.parametrize("kernel_variant", KERNELS_D128, indirect=True)
def test_non_contiguous_head_slices(kernel_variant):
    # Q/K/V as slices of one packed [B, S, 3, H, D] projection output
    B, S, H, D = 1, 256, 2, 64
    g = torch.Generator().manual_seed(6)
    qkv = torch.randn(B, S, 3, H, D, generator=g).to(torch.float16)
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))   # [B, H, S, D] views, not contiguous
    o_ref, lse_ref = attention_fwd_oracle(q, k, v, causal=False)
    qd = qkv.to(DEV)
    o, lse = multi_head_attention(*(qd[:, :, i].permute(0, 2, 1, 3) for i in range(3)), return_lse=True)
    _check(o, lse, o_ref, lse_ref, "packed qkv views")


def test_closed_form_invariants_at_full_headline_size():
    """B=2 H=16 S=8192 D=128 bf16 causal (the benchmark shape): properties that need no oracle.
    V == 1 => O == 1 exactly; Q == 0 => LSE_i = ln(i+1) and O_i = running mean of V; the last causal row equals the
    non-causal result for that row; two runs give identical bits."""
    B, H, S, D = 2, 16, 8192, 128
    g = torch.Generator(device=DEV).manual_seed(0)
    q = torch.randn(B, H, S, D, device=DEV, generator=g).to(torch.bfloat16)
    k = torch.randn(B, H, S, D, device=DEV, generator=g).to(torch.bfloat16)
    v = torch.randn(B, H, S, D, device=DEV, generator=g).to(torch.bfloat16)
    o1, lse1 = multi_head_attention(q, k, v, causal=True, return_lse=True)
    o2, lse2 = multi_head_attention(q, k, v, causal=True, return_lse=True)
    assert torch.equal(o1, o2) and torch.equal(lse1, lse2), "kernel is not deterministic"
    assert bool(torch.isfinite(o1.float()).all()) and bool(torch.isfinite(lse1).all())
    o_ones = multi_head_attention(q, k, torch.ones_like(v), causal=True)
    assert float((o_ones.float() - 1).abs().max()) <= 2 ** -7          # sum of bf16-rounded weights / fp32 sum
    oz, lsez = multi_head_attention(torch.zeros_like(q), k, v, causal=True, return_lse=True)
    want = torch.log(torch.arange(1, S + 1, device=DEV, dtype=torch.float32)).expand(B, H, S)
    assert float((lsez - want).abs().max()) <= 1e-4
    mean = torch.cumsum(v.float(), dim=2) / torch.arange(1, S + 1, device=DEV).view(1, 1, S, 1)
    assert float((oz.float() - mean).abs().max()) <= 2e-2
    o_nc, lse_nc = multi_head_attention(q[:, :, -128:], k, v, causal=False, return_lse=True)
    assert float((o_nc[:, :, -1].float() - o1[:, :, -1].float()).abs().max()) <= 2e-2
    assert float((lse_nc[:, :, -1] - lse1[:, :, -1]).abs().max()) <= 1e-3
    # row 0 attends key 0 only
    assert torch.equal(o1[:, :, 0], v[:, :, 0])


def test_autograd_function_surface():
    q, k, v = (t.to(DEV) for t in _qkv(1, 1, 128, 128, 64, torch.bfloat16, seed=9))
    q.requires_grad_(True)
    o = FlashAttentionFunction.apply(q, k, v)
    assert o.requires_grad
    o.sum().backward()          # the backward itself is checked in test_attention_bwd_gpu.py
    assert q.grad is not None and q.grad.shape == q.shape and k.grad is None


def test_rejected_inputs_raise():
    q, k, v = (t.to(DEV) for t in _qkv(1, 1, 16, 16, 20, torch.bfloat16))
    with pytest.raises(RuntimeError, match="multiple of 8"):
        multi_head_attention(q, k, v)
    q, k, v = (t.to(DEV) for t in _qkv(1, 1, 16, 16, 256, torch.bfloat16))
    with pytest.raises(RuntimeError, match="up to 128"):
        multi_head_attention(q, k, v)
    q, k, v = (t.to(DEV) for t in _qkv(1, 1, 16, 16, 64, torch.float32))
    with pytest.raises(RuntimeError, match="half-precision"):
        multi_head_attention(q, k, v)
    q, k, v = (t.to(DEV) for t in _qkv(1, 2, 16, 16, 64, torch.bfloat16))
    with pytest.raises(RuntimeError, match="shape mismatch"):
        multi_head_attention(q, k[:, :1], v)
