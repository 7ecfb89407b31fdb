"""Host side of Lion.step() without a GPU: the library call, the device table and torch.cuda are replaced by recorders, the
tensors live on the CPU (`_check_tensors` is relaxed to accept that), so that what the step decides can be looked at:
which tensors go into a launch, when every tensor is looked at again, and that no gradient is kept alive. The reference
holds no tensor beyond state["exp_avg"] and launches for every parameter that has a gradient
(fast_ops/lion/lion_optimizer.py:57-76)."""
import gc
import weakref

import numpy as np
import pytest
import torch

from fast_ops_amd.lion import lion_optimizer as L


class _Recorder:
    def __init__(self):
        self.launches = []        # (n_chunks, p dtype code, m dtype code) per fo_lion_step_typed
        self.keys = []            # the (p, g, m addresses, numels) handed to the table per launch

    def fo_lion_make_consts_typed(self, *a):
        return 0

    def fo_lion_step_typed(self, table, n_chunks, p_code, m_code, consts, stream):
        self.launches.append((n_chunks, p_code, m_code))
        return 0


@pytest.fixture
def host(monkeypatch):
    rec = _Recorder()
    looks = []

    class Table(L._Table):
        def update(self, key, p_size, m_size, stream):
            rec.keys.append(tuple(list(col) for col in key))
            if key == self.key:
                return
            t = L._chunk_table_of_columns(*key, p_size, m_size)
            self.key, self.n_chunks = tuple(list(col) for col in key), int(t.shape[0])
            self.dev = torch.zeros(1)
            self.rebuilds += 1

    class Stream:
        cuda_stream = 0

    class Guard:
        def __enter__(self):
            return self

        def __exit__(self, *a):
            return False

    def relaxed_check(param, grad, exp_avg):
        if grad.is_sparse:
            raise RuntimeError("Lion does not support sparse gradients")
        if not L._dense_same_layout(param, grad, exp_avg):
            raise RuntimeError("expected tensor to be contiguous")

    real_look = L.Lion._look_at_group

    def counting_look(self, gi, plist, grads):
        looks.append(gi)
        return real_look(self, gi, plist, grads)

    monkeypatch.setattr(L._lib, "load", lambda: rec)
    monkeypatch.setattr(L, "_Table", Table)
    monkeypatch.setattr(L, "_check_tensors", relaxed_check)
    monkeypatch.setattr(L.Lion, "_look_at_group", counting_look)
    monkeypatch.setattr(torch.cuda, "device", lambda d: Guard())
    monkeypatch.setattr(torch.cuda, "current_stream", lambda d=None: Stream())
    rec.looks = looks
    return rec


def _params(n=6):
    return [torch.nn.Parameter(torch.randn(40, 30)) for _ in range(n)]


def _new_grads(params, skip=()):
    for i, p in enumerate(params):
        p.grad = None if i in skip else torch.randn_like(p)


def test_quick_look_is_taken_and_finds_the_new_gradient_addresses(host):
    params = _params()
    opt = L.Lion(params)
    for step in range(4):
        _new_grads(params)
        opt.step()
        p_ptrs, g_ptrs, m_ptrs, numels = host.keys[-1]
        assert g_ptrs == [p.grad.data_ptr() for p in params] and p_ptrs == [p.data_ptr() for p in params]
        assert m_ptrs == [opt.state[p]["exp_avg"].data_ptr() for p in params] and numels == [1200] * 6
    assert host.looks == [0], "every tensor is looked at on the first step only"
    assert len(host.launches) == 4 and all(n == 6 for n, _, _ in host.launches)     # one chunk per 1200-element tensor


def test_no_gradient_is_kept_alive(host):
    params = _params()
    opt = L.Lion(params)
    _new_grads(params)
    refs = [weakref.ref(p.grad) for p in params]
    opt.step()
    opt.zero_grad()                       # torch's default: set_to_none=True
    gc.collect()
    assert all(r() is None for r in refs), "the optimizer still references a gradient after zero_grad()"


def test_same_addresses_mean_no_rebuild(host):
    params = _params()
    opt = L.Lion(params)
    bufs = [torch.randn_like(p) for p in params]
    for step in range(5):
        for p, b in zip(params, bufs):
            p.grad = b.view_as(b)         # a new tensor object over the same memory, as after zero_grad() + backward
        opt.step()
    assert opt.table_rebuilds == 1 and host.looks == [0]


def test_changes_are_noticed(host):
    params = _params()
    opt = L.Lion(params)
    _new_grads(params)
    opt.step()
    # another set of parameters has gradients
    _new_grads(params, skip=(2,))
    opt.step()
    assert host.looks == [0, 0] and len(host.keys[-1][0]) == 5 and params[2].data_ptr() not in host.keys[-1][0]
    _new_grads(params, skip=(2,))
    opt.step()
    assert host.looks == [0, 0]           # the same five again: quick look
    # a parameter's storage is replaced
    params[0].data = params[0].data.clone()
    _new_grads(params, skip=(2,))
    opt.step()
    assert host.looks == [0, 0, 0] and host.keys[-1][0][0] == params[0].data_ptr()
    # the caller replaces a momentum
    new_m = torch.zeros_like(params[1], dtype=torch.bfloat16)
    opt.state[params[1]]["exp_avg"] = new_m
    _new_grads(params, skip=(2,))
    opt.step()
    assert host.looks == [0, 0, 0, 0] and new_m.data_ptr() in host.keys[-1][2]
    # the group's list gets another parameter object at the same position
    extra = torch.nn.Parameter(torch.randn(40, 30))
    opt.param_groups[0]["params"][5] = extra
    _new_grads(params, skip=(2,))
    extra.grad = torch.randn_like(extra)
    opt.step()
    assert len(host.looks) == 5 and extra.data_ptr() in host.keys[-1][0]


def test_a_strided_or_sparse_gradient_still_raises_after_good_steps(host):
    params = _params(3)
    opt = L.Lion(params)
    for _ in range(2):
        _new_grads(params)
        opt.step()
    _new_grads(params)
    params[1].grad = torch.randn(30, 40).t()                     # right shape, other strides
    with pytest.raises(RuntimeError, match="contiguous"):
        opt.step()
    _new_grads(params)
    params[1].grad = torch.randn(40, 30).to_sparse()
    with pytest.raises(RuntimeError, match="sparse"):
        opt.step()
    _new_grads(params)
    opt.step()                                                    # good gradients again


def test_dtype_buckets_get_one_launch_each(host):
    a = [torch.nn.Parameter(torch.randn(100)) for _ in range(2)]
    b = [torch.nn.Parameter(torch.randn(100).to(torch.bfloat16)) for _ in range(3)]
    opt = L.Lion([a[0], b[0], a[1], b[1], b[2]])
    for _ in range(3):
        for p in a + b:
            p.grad = torch.randn(100).to(p.dtype)
        opt.step()
    per_step = host.launches[-2:]
    assert sorted(n for n, _, _ in per_step) == [2, 3]            # fp32 + bf16 momentum, and all-bf16
    assert host.looks == [0]
    assert [len(k[0]) for k in host.keys[-2:]] == [2, 3]


def test_chunk_table_of_columns_equals_the_per_tensor_table():
    ptrs = [(0x10000000, 0x20000000, 0x30000000, 8192 * 3 + 5), (0x40000000, 0x50000000, 0x60000000, 0), (0x70000000, 0x80000000, 0x90000000, 17)]
    t1 = L.build_chunk_table(ptrs)
    cols = list(zip(*ptrs))
    t2 = L._chunk_table_of_columns(list(cols[0]), list(cols[1]), list(cols[2]), list(cols[3]), 4, 2)
    assert np.array_equal(t1, t2) and int(t1["n"].sum()) == 8192 * 3 + 5 + 17 and t1.shape[0] == 5
