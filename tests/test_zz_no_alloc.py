"""fo_attn_bwd_static_ws - the attention backward for callers that cannot allocate: no workspace argument, the delta
buffer lives in a device array of the library - against fo_attn_bwd with a caller-supplied workspace, through the
C ABI. The kernels are the same and deterministic, so dQ, dK and dV must agree bit for bit. Two calls in a row, the
second on a smaller input (the array then still holds the first call's values past the part the second one uses)."""
import ctypes

import pytest
import torch

from fast_ops_amd import _lib

DEV = "cuda:0"
I3 = ctypes.c_int64 * 3
P64 = ctypes.POINTER(ctypes.c_int64)


def _inputs(B, H, Sq, Sk, D, dtype, causal, seed):
    from fast_ops.flash_attention.flash_attention import multi_head_attention

    g = torch.Generator().manual_seed(seed)
    q, go = (torch.randn(B, H, Sq, D, generator=g).to(dtype).to(DEV) for _ in range(2))
    k, v = (torch.randn(B, H, Sk, D, generator=g).to(dtype).to(DEV) for _ in range(2))
    o, lse = multi_head_attention(q, k, v, causal=causal, return_lse=True)
    return q, k, v, o, lse, go


def _backward(entry, q, k, v, o, lse, go, causal, delta=None):
    """Calls fo_attn_bwd (delta given) or fo_attn_bwd_static_ws (delta None) on fresh output tensors."""
    lib = _lib.load()
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    tensors = (q, k, v, o, go, dq, dk, dv)
    arrays = [I3(*t.stride()[:3]) for t in tensors]
    strides = (P64 * 8)(*[ctypes.cast(a, P64) for a in arrays])
    stream = torch.cuda.current_stream().cuda_stream
    ptrs = [t.data_ptr() for t in (q, k, v, o, go)] + [lse.data_ptr()]
    if delta is not None:
        ptrs.append(delta.data_ptr())
    ptrs += [dq.data_ptr(), dk.data_ptr(), dv.data_ptr()]
    code = {torch.float16: _lib.FO_DTYPE_F16, torch.bfloat16: _lib.FO_DTYPE_BF16}[q.dtype]
    status = getattr(lib, entry)(*ptrs, B, H, Sq, Sk, D, strides, D ** -0.5, int(causal), code, stream)
    assert status == 0, _lib.strerror(status)
    return dq, dk, dv


CALLS = [
    # (B, H, Sq, Sk, D, dtype, causal): a larger call, then a smaller one
    [(2, 8, 1024, 1024, 128, torch.bfloat16, True), (1, 3, 200, 333, 128, torch.bfloat16, True)],
    [(3, 4, 640, 900, 64, torch.float16, False), (2, 2, 129, 65, 64, torch.float16, False)],
]


@pytest.mark.gpu
@pytest.mark.parametrize("calls", CALLS, ids=["d128_bf16_causal", "d64_fp16_full"])
def test_static_workspace_backward_equals_the_workspace_argument_form(calls):
    for i, (B, H, Sq, Sk, D, dtype, causal) in enumerate(calls):
        q, k, v, o, lse, go = _inputs(B, H, Sq, Sk, D, dtype, causal, seed=17 + i)
        delta = torch.empty(2, B, H, Sq, dtype=torch.float32, device=DEV)
        want = _backward("fo_attn_bwd", q, k, v, o, lse, go, causal, delta)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        dq = dk = dv = None
        got = _backward("fo_attn_bwd_static_ws", q, k, v, o, lse, go, causal)
        torch.cuda.synchronize()
        for name, a, b in zip(("dQ", "dK", "dV"), got, want):
            assert torch.isfinite(a.float()).all(), f"call {i}: {name} not finite"
            assert torch.equal(a, b), f"call {i} {(B, H, Sq, Sk, D)}: {name} differs, max abs diff {float((a.float() - b.float()).abs().max()):.3e}"
        # the only device memory the call's Python side took is the three outputs this helper allocated
        grown = torch.cuda.memory_allocated() - before
        assert grown <= sum(t.numel() * t.element_size() for t in got) + 3 * 512


def test_static_workspace_limit():
    # B*H*Sq beyond the array is refused with a clear error before anything is launched (no GPU needed: every argument
    # check comes before the first HIP call)
    lib = _lib.load()
    s = I3(128 * 64, 64 * 128 * 4, 64)
    strides = (P64 * 8)(*[ctypes.cast(s, P64) for _ in range(8)])
    ok = 0x1000
    rows = _lib.FO_ATTN_BWD_STATIC_ROWS
    assert lib.fo_attn_bwd_static_ws(ok, ok, ok, ok, ok, ok, ok, ok, ok, 1, 1, rows + 1, 128, 64, strides, 0.125, 0, 1, None) == -4
    assert lib.fo_attn_bwd_static_ws(ok, ok, ok, ok, ok, ok, ok, ok, ok, 4, 8, rows // 32 + 1, 128, 64, strides, 0.125, 0, 1, None) == -4
    assert "too large" in _lib.strerror(-4)
    assert lib.fo_attn_bwd_static_ws(None, ok, ok, ok, ok, ok, ok, ok, ok, 1, 1, 128, 128, 64, strides, 0.125, 0, 1, None) == -1
