"""The boundary's promise about threads and streams: the library keeps no mutable state per call, so calls from several
host threads on different streams, and calls on several streams from one thread, may overlap. The reference launches on
whatever stream is current, under the GIL, with no host synchronisation (lion_update.cu:150, flash_attention_fwd.cu:173);
ctypes releases the GIL for the duration of a call, so here the calls of different threads really run concurrently.

Each worker runs a small training loop of its own - attention forward, backward (which allocates its own workspace),
a gradient for its parameters made from the attention gradients, a Lion step - on its own tensors and its own stream
of the default priority. Every worker's final tensors must equal, bit for bit, those of the same loop run alone on the
default stream (all kernels are deterministic: no atomics anywhere)."""
import threading

import pytest
import torch

from fast_ops.flash_attention.flash_attention import multi_head_attention
from fast_ops.lion.lion_optimizer import Lion

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# (B, H, S, D, dtype, causal): four different kernels - 128-row head_dim 128 causal, 128-row head_dim 64, the 256-row
# kernel (512 workgroups of 256 rows), a head_dim that is neither 64 nor 128
WORKLOADS = [
    (2, 4, 1024, 128, torch.bfloat16, True),
    (3, 5, 700, 64, torch.float16, False),
    (4, 32, 2048, 128, torch.bfloat16, True),
    (2, 3, 515, 40, torch.bfloat16, True),
]
PARAM_SIZES = [(257, 129), (8192,), (40000,), (3,)]


def _loop_steps(worker: int, iters: int):
    """The worker's loop on whatever stream is current when it is advanced: yields None after the set-up and after every
    iteration, and its final tensors at the end."""
    B, H, S, D, dtype, causal = WORKLOADS[worker]
    gen = torch.Generator().manual_seed(100 + worker)
    q, k, v, go = (torch.randn(B, H, S, D, generator=gen).to(dtype).to(DEV) for _ in range(4))
    params = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(DEV)) for s in PARAM_SIZES]
    opt = Lion(params, lr=1e-3, betas=(0.9, 0.99), weight_decay=0.1)
    yield None
    for it in range(iters):
        qr, kr, vr = (t.detach().requires_grad_(True) for t in (q, k, v))
        o = multi_head_attention(qr, kr, vr, causal=causal)
        dq, dk, dv = torch.autograd.grad(o, (qr, kr, vr), go)
        flat = torch.cat([dq.flatten(), dk.flatten(), dv.flatten()]).float()
        at = 0
        for p in params:
            p.grad = flat[at:at + p.numel()].view(p.shape).clone() * (1.0 + 0.01 * it)
            at += p.numel()
        opt.step()
        # feed the parameters back into the next iteration's queries so that every iteration depends on the one before
        q = (q.float() + params[1].detach()[:D] * 1e-2).to(dtype)
        opt.zero_grad()
        yield None
    out = [o.detach(), dq, dk, dv] + [p.detach() for p in params] + [opt.state[p]["exp_avg"] for p in params]
    yield [t.clone() for t in out]


def _loop(worker: int, iters: int):
    for res in _loop_steps(worker, iters):
        pass
    return res


def _same(a, b):
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.view(torch.uint8), b.view(torch.uint8))


def test_four_host_threads_on_their_own_streams():
    iters = 50
    alone = []
    for w in range(4):
        alone.append(_loop(w, iters))
    torch.cuda.synchronize()
    results, errors = [None] * 4, []
    start = threading.Barrier(4)

    def work(w):
        try:
            s = torch.cuda.Stream(device=DEV)          # default priority
            with torch.cuda.stream(s):
                start.wait()
                results[w] = _loop(w, iters)
            s.synchronize()
        except BaseException as e:                      # noqa: BLE001 - reported by the main thread
            errors.append((w, repr(e)))

    threads = [threading.Thread(target=work, args=(w,)) for w in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=300)
    assert not errors, errors
    assert all(not t.is_alive() for t in threads)
    torch.cuda.synchronize()
    for w in range(4):
        assert len(results[w]) == len(alone[w])
        for i, (a, b) in enumerate(zip(results[w], alone[w])):
            assert _same(a, b), f"worker {w}, tensor {i}: differs from the single-threaded run"


def test_two_streams_from_one_thread():
    """Two loops interleaved iteration by iteration on two streams of one thread, nothing synchronised in between."""
    iters = 20
    alone = [_loop(w, iters) for w in (0, 1)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=DEV) for _ in range(2)]
    # the same loops, each advanced one iteration at a time on its own stream
    gens = [_loop_steps(w, iters) for w in (0, 1)]
    results = [None, None]
    for _ in range(iters + 2):
        for w in (0, 1):
            with torch.cuda.stream(streams[w]):
                results[w] = next(gens[w])
    torch.cuda.synchronize()
    for w in (0, 1):
        for i, (a, b) in enumerate(zip(results[w], alone[w])):
            assert _same(a, b), f"loop {w}, tensor {i}: differs from the run on one stream"
