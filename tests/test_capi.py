"""CPU-side checks of the C ABI: the library loads, exports every symbol include/fastops.h declares, rejects bad
arguments with the documented codes before touching a device, and its host-only helpers agree with the oracle."""
import ctypes
import os
import re

import numpy as np
import pytest

from fast_ops_amd import _lib
from fast_ops_amd.lion import lion_optimizer as lo_host
from oracle import lion_oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fastops.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fo_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert set(declared) == set(_lib.SIGNATURES), "ctypes signature table and header disagree"
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/fastops.h but not exported"


def test_version_and_strerror():
    lib = _lib.load()
    assert lib.fo_version() // 1000 == _lib.ABI_MAJOR == 2
    assert _lib.strerror(0) == "ok"
    for code in range(-8, 0):
        assert "unknown" not in _lib.strerror(code)
    assert "unknown" in _lib.strerror(-99)


def test_struct_layouts_match_header():
    assert ctypes.sizeof(_lib.FoLionConsts) == 24
    assert ctypes.sizeof(_lib.FoLionChunk) == 32
    assert _lib.FoLionChunk.n.offset == 24
    m = re.search(r"#define\s+FO_LION_CHUNK\s+(\d+)", open(HEADER).read())
    assert int(m.group(1)) == _lib.FO_LION_CHUNK


def test_attn_argument_validation_without_device():
    lib = _lib.load()
    s = (ctypes.c_int64 * 3)(128 * 64, 64 * 128 * 4, 64)   # dummy but well-formed strides
    ok_ptr = 0x1000
    call = lambda **kw: lib.fo_attn_fwd(
        kw.get("q", ok_ptr), kw.get("k", ok_ptr), kw.get("v", ok_ptr), kw.get("o", ok_ptr), kw.get("lse", None),
        kw.get("B", 1), kw.get("H", 1), kw.get("Sq", 128), kw.get("Sk", 128), kw.get("D", 64),
        kw.get("qs", s), kw.get("ks", s), kw.get("vs", s), kw.get("os", s),
        kw.get("scale", 0.125), 0, kw.get("dtype", 1), None)
    assert call(q=None) == -1
    assert call(qs=None) == -1
    assert call(dtype=2) == -2
    assert call(D=68) == -3 and call(D=0) == -3 and call(D=136) == -3      # multiples of 8 from 8 to 128 only
    assert call(D=256) == -3
    assert call(Sq=0) == -4
    assert call(B=-1) == -4
    bad = (ctypes.c_int64 * 3)(128 * 64, 64 * 128, 60)
    assert call(ks=bad) == -5
    assert call(q=0x1008) == -6
    assert call(scale=float("nan")) == -4
    assert call(scale=0.0) == -4 and call(scale=-1.0) == -4


def test_attn_backward_bias_dropout_argument_validation_without_device():
    lib = _lib.load()
    I3 = ctypes.c_int64 * 3
    s = I3(128 * 64, 64 * 128 * 4, 64)
    P = ctypes.POINTER(ctypes.c_int64)
    strides = lambda bad=None: (P * 8)(*[ctypes.cast(bad if (bad is not None and i == 5) else s, P) for i in range(8)])
    ok = 0x1000
    bwd = lambda **kw: lib.fo_attn_bwd(
        kw.get("q", ok), ok, ok, ok, ok, kw.get("lse", ok), kw.get("ws", ok), ok, ok, ok,
        1, 1, kw.get("Sq", 128), 128, kw.get("D", 64), kw.get("strides", strides()), kw.get("scale", 0.125), 0, kw.get("dtype", 1), None)
    assert bwd(q=None) == -1 and bwd(ws=None) == -1 and bwd(strides=None) == -1
    assert bwd(dtype=2) == -2
    assert bwd(D=100) == -3 and bwd(D=136) == -3
    assert bwd(Sq=0) == -4 and bwd(scale=0.0) == -4
    assert bwd(strides=strides(I3(128 * 64, 64 * 128, 60))) == -5      # dQ rows not 16-byte aligned / shorter than D
    assert bwd(lse=0x1002) == -6

    class Extras(ctypes.Structure):
        _fields_ = [("bias", ctypes.c_void_p), ("bias_strides", ctypes.c_int64 * 3), ("bias_dtype", ctypes.c_int),
                    ("dropout_p", ctypes.c_float), ("dropout_seed", ctypes.c_uint32), ("dropout_offset", ctypes.c_uint64)]
    def fwd_ex(ex):
        return lib.fo_attn_fwd_ex(ok, ok, ok, ok, None, 1, 1, 128, 128, 64, s, s, s, s, 0.125, 0, 1, ctypes.byref(ex), None)
    ex = Extras(); ex.bias = ok; ex.bias_strides = I3(0, 0, 128); ex.bias_dtype = 0      # fp16 bias with bf16 operands
    assert fwd_ex(ex) == -2
    ex.bias_dtype = 2; ex.bias_strides = I3(0, 0, -1)
    assert fwd_ex(ex) == -5
    ex.bias_strides = I3(0, 0, 128); ex.bias = 0x1002                                  # fp32 bias on a 2-byte boundary
    assert fwd_ex(ex) == -6
    ex.bias = None; ex.dropout_p = 1.0
    assert fwd_ex(ex) == -4
    assert lib.fo_attn_fwd_dropout(ok, ok, ok, ok, None, 1, 1, 128, 128, 64, s, s, s, s, 0.125, 0, 1, -0.1, 1, 0, None) == -4
    assert lib.fo_dropout_mask(None, 16, 0.5, 1, 0, None) == -1
    assert lib.fo_dropout_mask(ok, -1, 0.5, 1, 0, None) == -4
    assert lib.fo_dropout_mask(ok, 16, 1.5, 1, 0, None) == -4
    assert lib.fo_dropout_mask(ok, 0, 0.5, 1, 0, None) == 0                            # nothing to do, nothing launched


def test_lion_argument_validation_without_device():
    lib = _lib.load()
    c = _lib.FoLionConsts()
    assert lib.fo_lion_make_consts(1e-4, 0.9, 0.99, 0.1, None) == -1
    assert lib.fo_lion_update(0x1000, 0x1000, 0x1000, 16, None, None) == -1
    assert lib.fo_lion_update(None, 0x1000, 0x1000, 16, ctypes.byref(c), None) == -1
    assert lib.fo_lion_update(0x1000, 0x1000, 0x1000, -1, ctypes.byref(c), None) == -4
    assert lib.fo_lion_update(0x1002, 0x1000, 0x1000, 16, ctypes.byref(c), None) == -6
    assert lib.fo_lion_update(None, None, None, 0, ctypes.byref(c), None) == 0      # empty tensor: nothing to do
    assert lib.fo_lion_step(None, 0, ctypes.byref(c), None) == 0
    assert lib.fo_lion_step(None, 4, ctypes.byref(c), None) == -1
    assert lib.fo_lion_step(0x1000, -1, ctypes.byref(c), None) == -4
    assert lib.fo_lion_step(0x1004, 4, ctypes.byref(c), None) == -6


@pytest.mark.parametrize("hp", [(1e-4, 0.9, 0.99, 0.1), (1e-3, 0.95, 0.98, 0.5), (3e-5, 0.0, 1.0, 0.0)])
def test_make_consts_matches_python_double_arithmetic(hp):
    lr, b1, b2, wd = hp
    c = lo_host.make_consts(lr, (b1, b2), wd)
    got = np.array([c.c_wd, c.c_b1, c.c_1b1, c.c_nlr, c.c_b2, c.c_1b2], dtype=np.float32)
    want = np.array(lion_oracle.lion_consts(lr, (b1, b2), wd), dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_fill_chunks_matches_python_table():
    lib = _lib.load()
    for numel in (1, 8191, 8192, 8193, 50257 * 768):
        n = lib.fo_lion_fill_chunks(0x10000000, 0x20000000, 0x30000000, numel, None)
        assert n == -(-numel // _lib.FO_LION_CHUNK)
        buf = (_lib.FoLionChunk * n)()
        assert lib.fo_lion_fill_chunks(0x10000000, 0x20000000, 0x30000000, numel, buf) == n
        table = lo_host.build_chunk_table([(0x10000000, 0x20000000, 0x30000000, numel)])
        mine = np.frombuffer(buf, dtype=table.dtype)
        assert np.array_equal(mine, table)
        assert int(table["n"].sum()) == numel
    assert lib.fo_lion_fill_chunks(0x1000, 0x1000, 0x1000, 0, None) == 0


def test_tune_hook():
    lib = _lib.load()
    assert lib.fo_tune_get(b"lion.variant") == -1
    assert lib.fo_tune_set(b"lion.variant", 3) == 0 and lib.fo_tune_get(b"lion.variant") == 3
    assert lib.fo_tune_set(b"lion.variant", -1) == 0
    assert lib.fo_tune_set(b"no.such.key", 1) == -8
    # every key the kernels read: default -1 (the library's choice), settable, readable
    for key, value in ((b"attn.variant", 16), (b"attn_bwd.variant", 0), (b"attn.order", 2), (b"attn.balance", 0), (b"attn.keep_on", 1), (b"attn.tail", 0), (b"attn_bwd.order", 2)):
        assert lib.fo_tune_get(key) == -1
        assert lib.fo_tune_set(key, value) == 0 and lib.fo_tune_get(key) == value
        assert lib.fo_tune_set(key, -1) == 0 and lib.fo_tune_get(key) == -1


def test_tune_hook_accepts_only_kernels_that_compute_the_function():
    # the shipped library holds no timing ablations (kernel variants that leave work out): their numbers select nothing
    lib = _lib.load()
    assert lib.fo_tune_get(b"build.ablations") == 0
    for ok in (-1, 0, 1, 8, 16, 32):
        assert lib.fo_tune_set(b"attn.variant", ok) == 0
    for bad in (2, 3, 7, 9, 15, 17, 33, 257, 258, 260, 263, 320, 384, 519, 520, 640, -2):
        assert lib.fo_tune_set(b"attn.variant", bad) == -8, bad
        assert lib.fo_tune_get(b"attn.variant") == 32          # a refused value changes nothing
    assert lib.fo_tune_set(b"attn.variant", -1) == 0
    assert lib.fo_tune_set(b"attn_bwd.variant", 2) == -8
    assert lib.fo_tune_set(b"attn.keep_on", 3) == -8
    assert lib.fo_tune_set(b"lion.variant", 32) == -8


def test_attn_kernel_query_and_stride_limit_without_device_work():
    lib = _lib.load()
    I3 = ctypes.c_int64 * 3
    dense = lambda S, D: I3(S * D * 4, S * D, D)
    k = lambda B, H, Sq, Sk, D, causal, bias=0, drop=0, ks=None: lib.fo_attn_fwd_kernel(
        B, H, Sq, Sk, D, ks or dense(Sk, D), ks or dense(Sk, D), causal, bias, drop)
    # small shapes, bias and dropout always take the 128-row kernel, whatever the device
    assert k(1, 1, 128, 128, 64, 0) == _lib.FO_ATTN_KERNEL_ROWS128
    assert k(2, 16, 8192, 8192, 128, 1, bias=1) == _lib.FO_ATTN_KERNEL_ROWS128
    assert k(2, 16, 8192, 8192, 128, 1, drop=1) == _lib.FO_ATTN_KERNEL_ROWS128
    # forced choices are honoured where the kernel exists
    assert lib.fo_tune_set(b"attn.variant", 32) == 0
    try:
        assert k(1, 1, 512, 512, 128, 0) == _lib.FO_ATTN_KERNEL_ROWS256_W4
        assert k(1, 1, 512, 512, 64, 0) == _lib.FO_ATTN_KERNEL_ROWS256_W4
        assert lib.fo_tune_set(b"attn.variant", 1) == 0
        assert k(1, 1, 512, 512, 64, 1) == _lib.FO_ATTN_KERNEL_ROWS128_EXACT
    finally:
        lib.fo_tune_set(b"attn.variant", -1)
    assert k(1, 1, 128, 128, 76, 0) == -3 and k(0, 1, 128, 128, 64, 0) == -4
    # the query refuses what the call refuses: sizes beyond the launch limits, strides that are negative or no multiple of 8
    assert k(1 << 15, 1 << 15, 1 << 12, 128, 64, 0) == -4 and k(1 << 10, 1 << 10, 1 << 21, 128, 64, 0) == -4
    assert k(1, 1, 128, 128, 64, 0, ks=I3(0, -8, 64)) == -5 and k(1, 1, 128, 128, 64, 0, ks=I3(0, 12, 64)) == -5
    # the library's own choice on 256 CUs (an MI355X, or what the library assumes where it finds no device); on a device
    # with another number of compute units the thresholds move, and the expectations below do not apply
    import torch

    on_256_cus = not torch.cuda.is_available() or torch.cuda.get_device_properties(0).multi_processor_count == 256
    R128, W8, W4, PIPE = _lib.FO_ATTN_KERNEL_ROWS128, _lib.FO_ATTN_KERNEL_ROWS256_W8, _lib.FO_ATTN_KERNEL_ROWS256_W4, _lib.FO_ATTN_KERNEL_ROWS128_PIPE
    if on_256_cus:
        assert k(2, 16, 8192, 8192, 128, 1) == W4            # the headline shape: 512 workgroups of two query blocks
        assert k(16, 32, 2048, 2048, 128, 0) == W4           # B=16 H=32 S=2048 non-causal
        assert k(8, 12, 1024, 1024, 64, 1) == R128           # the GPT-2-small shape
        assert k(2, 16, 4096, 4096, 128, 1) == W8 and k(4, 16, 6144, 6144, 128, 1) == W8   # fewer than 8192 keys, causal: eight waves
        assert k(8, 16, 1024, 1024, 128, 1) == W8            # causal from 1024 queries on: 256 workgroups, one round
        assert k(12, 16, 1024, 1024, 128, 1) == R128         # 384 workgroups would leave half of the second round empty
        assert k(32, 16, 512, 512, 128, 1) == R128           # causal below 1024 queries
        assert k(16, 16, 512, 512, 128, 0) == W4 and k(10, 16, 512, 512, 128, 0) == R128   # 512 / 320 workgroups; non-causal: four waves
        assert k(32, 16, 256, 256, 128, 0) == W8             # (below 512 keys the eight-wave form stays)
        # a last round that is at most half full goes to a second launch of the 128-row form and counts 0.6 of a round:
        # 528 items = 2 rounds + 16, 288 = 1 round + 32 (from 4096 keys on the rounds need to be filled to 70 %); not causal
        assert k(1, 33, 4096, 4096, 128, 0) == W4 and k(1, 12, 6144, 6144, 128, 0) == W4 and k(1, 33, 4096, 4096, 128, 1) != W4
        assert k(1, 36, 2048, 2048, 128, 0) == R128          # 288 items, but below 4096 keys the bar is 80 %
        assert k(1, 8, 8192, 8192, 64, 0) == W4 and k(4, 8, 4096, 4096, 64, 0) == W4 and k(8, 8, 2048, 2048, 64, 0) == R128   # head_dim 64: long rows only,
        assert k(1, 8, 16384, 16384, 64, 1) == W4 and k(2, 16, 8192, 8192, 64, 1) == W4 and k(4, 16, 4096, 4096, 64, 1) == W4  # and four waves
        assert k(8, 16, 2048, 2048, 64, 1) == R128 and k(4, 16, 4096, 4096, 64, 1, bias=2) == R128   # (causal from 4096 keys, with a per-key bias from 8192)
        # too few workgroups for the chip (12 heads of a tensor-parallel split): 128-row workgroups in the pipelined kernel
        assert k(1, 12, 2048, 2048, 128, 1) == PIPE and k(1, 12, 2048, 2048, 128, 0) == PIPE and k(1, 12, 4096, 4096, 128, 1) == PIPE
        # long rows of keys at head_dim 128: the 256-row kernel already with three quarters of one round of workgroups
        assert k(1, 12, 8192, 8192, 128, 1) == W4 and k(1, 12, 4096, 4096, 128, 0) == W4 and k(1, 12, 8192, 8192, 128, 0) == W4
        assert k(1, 10, 8192, 8192, 128, 1) == R128 and k(1, 12, 512, 512, 128, 0) == R128
        assert k(1, 12, 4096, 4096, 64, 1) == PIPE and k(1, 12, 1024, 1024, 64, 1) == R128
        # a bias that is the same for every query (has_bias 2) takes part in the choice, with the forms that exist for it:
        # 128 rows pipelined, 256 rows as four waves (head_dim 128), the 128-row kernel; a bias with a query stride does not
        assert k(1, 12, 2048, 2048, 128, 1, bias=2) == PIPE and k(1, 12, 2048, 2048, 128, 1, bias=1) == R128
        assert k(2, 16, 8192, 8192, 128, 1, bias=2) == W4 and k(2, 16, 4096, 4096, 128, 1, bias=2) == W4    # (W8 without bias)
        assert k(1, 8, 8192, 8192, 64, 0, bias=2) == W4 and k(1, 12, 4096, 4096, 64, 1, bias=2) == PIPE
        assert k(2, 16, 8192, 8256, 128, 0, bias=2) == R128 and k(2, 16, 8192, 8130, 128, 0, bias=2) == W4  # at most 8192 keys in LDS
        assert k(2, 16, 8192, 8192, 128, 1, bias=2, drop=1) == R128
    # head dims other than 64 and 128 take the 128-row kernel, whatever is forced
    assert k(2, 16, 8192, 8192, 96, 1) == _lib.FO_ATTN_KERNEL_ROWS128
    assert lib.fo_attn_fwd_kernel(1, 1, 128, 128, 64, None, dense(128, 64), 0, 0, 0) == -1
    # K/V row strides of 2^24 elements and more do not fit the kernels' 32-bit tile offsets: rejected, not wrapped
    wide_rows = I3(0, 0, 1 << 24)
    assert k(1, 1, 128, 128, 64, 0, ks=wide_rows) == -5
    ok_ptr = 0x1000
    s = dense(128, 64)
    assert lib.fo_attn_fwd(ok_ptr, ok_ptr, ok_ptr, ok_ptr, None, 1, 1, 128, 128, 64, s, wide_rows, s, s, 0.125, 0, 1, None) == -5
    assert lib.fo_attn_fwd(ok_ptr, ok_ptr, ok_ptr, ok_ptr, None, 1, 1, 128, 128, 64, s, s, wide_rows, s, 0.125, 0, 1, None) == -5


def test_python_surfaces_validate_like_the_reference():
    import torch

    from fast_ops.lion.lion_optimizer import Lion
    from fast_ops.flash_attention.flash_attention import multi_head_attention

    p = [torch.nn.Parameter(torch.zeros(4))]
    with pytest.raises(RuntimeError, match="expected positive LR"):
        Lion(p, lr=0.0)
    with pytest.raises(RuntimeError, match="betas must be between 0 and 1"):
        Lion(p, betas=(1.5, 0.9))
    opt = Lion(p, lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)
    assert opt.defaults == {"lr": 1e-4, "betas": (0.9, 0.99), "weight_decay": 0.1}
    # CPU tensors: there is no CPU path, the call must raise rather than compute something else
    p[0].grad = torch.ones(4)
    with pytest.raises(RuntimeError, match="GPU only"):
        opt.step()
    q = torch.zeros(1, 1, 8, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU tensors"):
        multi_head_attention(q, q, q)
    with pytest.raises(RuntimeError, match="half-precision"):
        multi_head_attention(q.float(), q.float(), q.float())
