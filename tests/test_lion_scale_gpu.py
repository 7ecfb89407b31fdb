"""The fused Lion step at full size, through Lion.step() and the C ABI, against the CPU oracle:

* the 1.3 B-parameter benchmark configuration compared element for element (every parameter and every momentum value,
  after every step), as the reference's own test compares params and exp_avg after each step
  (tests/test_lion_optimizer.py:25-53) - with exact equality in place of allclose;
* one tensor of more than 2^31 elements (the reference's launcher holds numel in an int: lion_update.cu:130,143);
* torch's default training loop (backward, step, zero_grad()) over the GPT-2-small parameter set: results, the memory
  the optimizer keeps alive, and how often the chunk table is rebuilt (the reference keeps no tensor but
  state["exp_avg"]: lion_optimizer.py:57-76).
"""
import os
import time

import numpy as np
import pytest
import torch

from fast_ops.lion.lion_optimizer import Lion, lion_update
from oracle import lion_oracle as lo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HP = dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)
THREADS = min(16, os.cpu_count() or 1)


def _bits16(t):
    return t.detach().cpu().view(torch.int16).numpy().view(np.uint16).reshape(-1)


def _bits32(t):
    return t.detach().cpu().numpy().view(np.uint32).reshape(-1)


def test_config_5b_every_element_against_the_oracle():
    """78 tensors (39 x 2048x8192 + 39 x 8192x2048) = 1,308,622,848 fp32 parameters with bf16 momentum; parameters
    ~ N(0, 0.02) then momenta ~ N(0, 1e-3) from a CPU generator seeded 0, gradients ~ N(0, 1e-2) from seed 1000 + step;
    lr 1e-4, betas (0.9, 0.99), weight_decay 0.1; two steps through Lion.step(). After each step every parameter and
    every momentum value is compared bit for bit with the C oracle; one tensor also with the four torch statements run
    on the host; and after the first step the multi-tensor launch is compared with one launch per tensor."""
    shapes = [(2048, 8192)] * 39 + [(8192, 2048)] * 39
    t0 = time.perf_counter()
    gen = torch.Generator().manual_seed(0)
    host_p = [torch.randn(s, generator=gen) * 0.02 for s in shapes]
    params = [torch.nn.Parameter(t.to(DEV)) for t in host_p]
    opt = Lion(params, **HP)
    host_m = []
    for prm in params:
        m = (torch.randn(prm.shape, generator=gen) * 1e-3).to(torch.bfloat16)
        opt.state[prm]["exp_avg"] = m.to(DEV)
        host_m.append(m)
    total = sum(t.numel() for t in host_p)
    assert total == 1_308_622_848
    print(f"\n  inputs drawn and copied: {time.perf_counter() - t0:.1f} s", flush=True)
    bad_total = [0, 0]
    for step in range(2):
        ggen = torch.Generator().manual_seed(1000 + step)
        host_g = []
        for prm in params:
            g = torch.randn(prm.shape, generator=ggen) * 1e-2
            prm.grad = g.to(DEV)
            host_g.append(g)
        if step == 0:
            # the same step as one launch per tensor on copies (78 launches of the single-tensor entry point)
            single = [(prm.detach().clone(), opt.state[prm]["exp_avg"].clone()) for prm in params]
            for (p1, m1), prm in zip(single, params):
                lion_update(p1, prm.grad, m1, HP["lr"], *HP["betas"], HP["weight_decay"])
            # and one tensor through the four torch statements on the host
            pt, mt = host_p[40].clone(), host_m[40].clone()
            lo.lion_step_torch([pt], [host_g[40]], [mt], **HP)
        opt.step()
        for p, g, m in zip(host_p, host_g, host_m):         # the GPU runs its step meanwhile
            lo.lion_step_c(p.numpy().reshape(-1), g.numpy().reshape(-1), m.view(torch.int16).numpy().view(np.uint16).reshape(-1),
                           HP["lr"], HP["betas"], HP["weight_decay"], threads=THREADS)
        bad_p = bad_m = 0
        for prm, p, m in zip(params, host_p, host_m):
            bad_p += int(np.count_nonzero(_bits32(prm) != _bits32(p)))
            bad_m += int(np.count_nonzero(_bits16(opt.state[prm]["exp_avg"]) != _bits16(m)))
        print(f"  step {step}: vs C oracle {bad_p} parameter / {bad_m} momentum mismatches of {total} ({time.perf_counter() - t0:.1f} s)", flush=True)
        bad_total[0] += bad_p
        bad_total[1] += bad_m
        if step == 0:
            tp = int(np.count_nonzero(_bits32(params[40]) != _bits32(pt)))
            tm = int(np.count_nonzero(_bits16(opt.state[params[40]]["exp_avg"]) != _bits16(mt)))
            print(f"  step 0, tensor 40: vs the torch statements on the host {tp} parameter / {tm} momentum mismatches of {pt.numel()}", flush=True)
            assert tp == 0 and tm == 0
            for (p1, m1), prm in zip(single, params):
                assert torch.equal(p1.view(torch.int32), prm.detach().view(torch.int32)), "multi-tensor launch differs from per-tensor launches"
                assert torch.equal(m1.view(torch.int16), opt.state[prm]["exp_avg"].view(torch.int16))
            del single
        del host_g
    assert bad_total == [0, 0]
    assert opt.table_rebuilds <= 2


def test_one_tensor_of_more_than_2_to_31_elements():
    """n = 2^31 + 8192 + 5 fp32 parameters (262,146 chunk descriptors; byte offsets beyond 2^33), through the
    single-tensor entry point, through Lion.step() and as two tensors of fewer than 2^31 elements each: the three must
    agree on every element, windows at the start, around elements 2^29 (byte 2^31), 2^30 (byte 2^32) and 2^31 and the
    tail must equal the oracle, and the guard elements around the tensors must be untouched."""
    n = (1 << 31) + 8192 + 5
    guard = 4096
    gen = torch.Generator(device=DEV).manual_seed(5)

    def guarded(dtype, fill):
        buf = torch.empty(n + 2 * guard, dtype=dtype, device=DEV)
        buf[:guard] = fill
        buf[-guard:] = fill
        return buf, buf[guard:guard + n]

    p_buf, p = guarded(torch.float32, 7.0)
    m_buf, m = guarded(torch.bfloat16, 7.0)
    g_buf, g = guarded(torch.float32, 7.0)
    piece = 1 << 28
    for lo_ in range(0, n, piece):                       # drawn in pieces: the temporaries stay small
        hi = min(n, lo_ + piece)
        p[lo_:hi] = torch.randn(hi - lo_, device=DEV, generator=gen) * 0.02
        g[lo_:hi] = torch.randn(hi - lo_, device=DEV, generator=gen) * 1e-2
        m[lo_:hi] = (torch.randn(hi - lo_, device=DEV, generator=gen) * 1e-3).to(torch.bfloat16)
    w = 20000
    windows = [(0, w), ((1 << 29) - w, (1 << 29) + w), ((1 << 30) - w, (1 << 30) + w), ((1 << 31) - w, (1 << 31) + w), (n - w, n)]
    expect = []
    for a, b in windows:
        pc, gc, mc = p[a:b].cpu().numpy().copy(), g[a:b].cpu().numpy().copy(), _bits16(m[a:b]).copy()
        lo.lion_step_c(pc, gc, mc, HP["lr"], HP["betas"], HP["weight_decay"])
        expect.append((pc, mc))
    # copies for the other two routes
    p2, m2 = torch.nn.Parameter(p.clone()), m.clone()
    p3, m3 = p.clone(), m.clone()
    print(f"\n  single tensor entry point, n = {n}", flush=True)
    lion_update(p, g, m, HP["lr"], *HP["betas"], HP["weight_decay"])
    torch.cuda.synchronize()
    for (a, b), (pc, mc) in zip(windows, expect):
        assert np.array_equal(_bits32(p[a:b]), pc.view(np.uint32)), f"parameters differ from the oracle in [{a}, {b})"
        assert np.array_equal(_bits16(m[a:b]), mc), f"momentum differs from the oracle in [{a}, {b})"
    for buf in (p_buf, m_buf, g_buf):
        assert bool((buf[:guard] == 7.0).all()) and bool((buf[-guard:] == 7.0).all()), "written outside the tensor"
    print("  Lion.step()", flush=True)
    opt = Lion([p2], **HP)
    opt.state[p2]["exp_avg"] = m2
    p2.grad = g
    opt.step()
    torch.cuda.synchronize()
    assert torch.equal(p2.detach().view(torch.int32), p.view(torch.int32)) and torch.equal(m2.view(torch.int16), m.view(torch.int16))
    print("  two tensors below 2^31 elements", flush=True)
    cut = (1 << 30) + 8192 * 3 + 24
    for a, b in ((0, cut), (cut, n)):
        lion_update(p3[a:b], g[a:b], m3[a:b], HP["lr"], *HP["betas"], HP["weight_decay"])
    torch.cuda.synchronize()
    assert torch.equal(p3.view(torch.int32), p.view(torch.int32)) and torch.equal(m3.view(torch.int16), m.view(torch.int16))
    assert bool((g_buf[:guard] == 7.0).all()) and bool((g_buf[-guard:] == 7.0).all())


def _gpt2_small_shapes():
    shapes = [(50257, 768), (1024, 768)]
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,), (768,), (768,), (768, 3072), (3072,), (3072, 768), (768,)]
    return shapes + [(768,), (768,)]


def test_default_training_loop_frees_gradients_and_keeps_the_chunk_table():
    """backward -> step() -> zero_grad() with torch's default set_to_none=True, eight steps over the 148 GPT-2-small
    tensors, gradients made by autograd (new tensors every step). Every step equals the oracle bit for bit; after
    zero_grad() no gradient set is resident (the optimizer holds no reference to a gradient); and once the allocator's
    pattern has settled the gradients come back at the addresses of the step before, so the chunk table is not rebuilt."""
    shapes = _gpt2_small_shapes()
    sizes = [int(np.prod(s)) for s in shapes]
    total = sum(sizes)
    gen = torch.Generator().manual_seed(0)
    flat_p = torch.randn(total, generator=gen) * 0.02
    flat_m = (torch.randn(total, generator=gen) * 1e-3).to(torch.bfloat16)
    offs = np.concatenate([[0], np.cumsum(sizes)[:-1]]).tolist()
    params = [torch.nn.Parameter(flat_p[o:o + n].view(s).to(DEV)) for s, n, o in zip(shapes, sizes, offs)]
    opt = Lion(params, **HP)
    for prm, o, n in zip(params, offs, sizes):
        opt.state[prm]["exp_avg"] = flat_m[o:o + n].view(prm.shape).to(DEV)
    pc, mc = flat_p.numpy().copy(), _bits16(flat_m).copy()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    base = torch.cuda.memory_allocated()
    rebuilds, host_us = [], []
    for step in range(8):
        g = torch.randn(total, generator=torch.Generator().manual_seed(1000 + step)) * 1e-2
        w = g.to(DEV)
        # a loss whose gradient with respect to parameter i is w's slice i, produced by autograd as a new tensor
        loss = sum((prm * w[o:o + n].view(prm.shape)).sum() for prm, o, n in zip(params, offs, sizes))
        loss.backward()
        del loss, w
        assert all(prm.grad is not None for prm in params)
        torch.cuda.synchronize()
        before = opt.table_rebuilds
        t0 = time.perf_counter()
        opt.step()
        host_us.append((time.perf_counter() - t0) * 1e6)
        rebuilds.append(opt.table_rebuilds - before)
        opt.zero_grad()
        torch.cuda.synchronize()
        # parameters + momenta + the chunk tables (two generations of 15,263 descriptors of 32 bytes) and nothing else
        held = torch.cuda.memory_allocated() - base
        assert held < 4 * 1024 * 1024, f"step {step}: {held} bytes beyond parameters and momenta are still allocated after zero_grad()"
        lo.lion_step_c(pc, g.numpy(), mc, HP["lr"], HP["betas"], HP["weight_decay"], threads=THREADS)
        got_p = torch.cat([prm.detach().reshape(-1) for prm in params])
        got_m = torch.cat([opt.state[prm]["exp_avg"].reshape(-1) for prm in params])
        bad_p = int(np.count_nonzero(_bits32(got_p) != pc.view(np.uint32)))
        bad_m = int(np.count_nonzero(_bits16(got_m) != mc))
        assert bad_p == 0 and bad_m == 0, f"step {step}: {bad_p} parameter and {bad_m} momentum mismatches"
        del got_p, got_m
    print(f"\n  chunk table rebuilds per step: {rebuilds}; host time of step() in us: {[round(u) for u in host_us]}", flush=True)
    assert rebuilds[0] == 1 and sum(rebuilds[2:]) <= 1, f"the chunk table keeps being rebuilt: {rebuilds}"
