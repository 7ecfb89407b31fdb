"""A whole training step - attention forward, its backward, the fused Lion update - captured once into a HIP graph and
replayed: every replay must leave exactly the parameters and momenta that the same steps leave when launched eagerly.
The C ABI takes the stream it launches on as an argument and allocates nothing, so capture needs no special path; this
test pins that (and that nothing in the step depends on work a replay does not repeat). Between the replays the
program does eager work and synchronises, and every replay is checked, not only the first."""
import pytest
import torch

from fast_ops.flash_attention.flash_attention import multi_head_attention
from fast_ops.lion.lion_optimizer import Lion

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _step(params, opt, go, causal):
    q, k, v = params
    o = multi_head_attention(q, k, v, causal=causal)
    grads = torch.autograd.grad(o, params, go)
    for p, g in zip(params, grads):
        p.grad.copy_(g)             # static gradient buffers: the optimizer's chunk table keeps its addresses
    opt.step()


@pytest.mark.parametrize("shape,causal", [((2, 4, 512, 64), True), ((1, 8, 1024, 128), False)])
def test_training_step_replayed_from_a_graph_equals_eager_steps(shape, causal):
    B, H, S, D = shape
    gen = torch.Generator().manual_seed(S + D)
    init = [(torch.randn(B, H, S, D, generator=gen) * 0.5).to(torch.bfloat16).to(DEV) for _ in range(3)]
    go = torch.randn(B, H, S, D, generator=gen).to(torch.bfloat16).to(DEV)
    n_steps = 4

    def fresh():
        params = [torch.nn.Parameter(t.clone()) for t in init]
        for p in params:
            p.grad = torch.zeros_like(p)
        return params, Lion(params, lr=1e-3, betas=(0.9, 0.99), weight_decay=0.1)

    # eager trajectory: parameters and momenta after each step
    params, opt = fresh()
    want = []
    for _ in range(n_steps):
        _step(params, opt, go, causal)
        torch.cuda.synchronize()
        want.append([p.detach().clone() for p in params] + [opt.state[p]["exp_avg"].clone() for p in params])

    # graph: warm up on a side stream (creates the momenta and the chunk table), put the start values back, capture one
    # step, replay it n_steps times
    params, opt = fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            _step(params, opt, go, causal)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.no_grad():
        for p, t in zip(params, init):
            p.copy_(t)
            opt.state[p]["exp_avg"].zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _step(params, opt, go, causal)
    with torch.no_grad():               # the capture itself ran nothing, but be explicit about the start state
        for p, t in zip(params, init):
            p.copy_(t)
            opt.state[p]["exp_avg"].zero_()
    scratch = torch.zeros(1 << 20, device=DEV)
    for i in range(n_steps):
        graph.replay()
        scratch.add_(1.0).mul_(0.5)     # eager work of the program's own between the replays
        torch.cuda.synchronize()
        got = [p.detach() for p in params] + [opt.state[p]["exp_avg"] for p in params]
        for j, (a, b) in enumerate(zip(got, want[i])):
            assert torch.equal(a, b), f"replay {i}: tensor {j} differs from the eager step ({(a.float() - b.float()).abs().max().item():.3e})"
