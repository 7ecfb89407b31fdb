"""Parity of the fused Lion kernel (through the C ABI) with the CPU oracle: parameters bit-exact, bf16 momentum
identical. Mirrors the reference's own test (tests/test_lion_optimizer.py:11-53: same gradients to both optimizers,
several steps, compare parameters and exp_avg after every step) with exact equality in place of allclose."""
import ctypes
import os

import numpy as np
import pytest
import torch

from fast_ops.lion.lion_optimizer import Lion, lion_update
from fast_ops_amd import _lib
from oracle import lion_oracle as lo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HP = dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "lion_small.npz")


def _bits16(t):
    return t.detach().cpu().view(torch.int16).numpy().view(np.uint16).copy()


def _bits32(t):
    return t.detach().cpu().numpy().view(np.uint32)


def _seeded(n, seed):
    g = torch.Generator().manual_seed(seed)
    p = torch.randn(n, generator=g) * 0.02
    m = (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16)
    gr = torch.randn(n, generator=g) * 1e-2
    return p, gr, m


def _oracle(p, gr, m, hp, threads=8):
    pc, mc = p.numpy().copy(), _bits16(m)
    lo.lion_step_c(pc, gr.numpy().copy(), mc, hp["lr"], hp["betas"], hp["weight_decay"], threads=threads)
    return pc, mc


@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 1024, 8191, 8192, 8193, 3 * 8192 + 1021, (1 << 20) + 13])
def test_single_tensor_bit_exact(n):
    p, gr, m = _seeded(n, seed=n)
    pc, mc = _oracle(p, gr, m, HP)
    pd, gd, md = p.to(DEV), gr.to(DEV), m.to(DEV)
    lion_update(pd, gd, md, HP["lr"], *HP["betas"], HP["weight_decay"])
    torch.cuda.synchronize()
    assert np.array_equal(_bits32(pd), pc.view(np.uint32)), "parameters differ from the oracle"
    assert np.array_equal(_bits16(md), mc), "momentum differs from the oracle"
    assert torch.equal(gd.cpu(), gr), "gradient must not be written"


@pytest.mark.parametrize("variant", list(range(32)))
def test_every_kernel_variant_bit_exact(variant):
    n = 5 * 8192 + 77
    p, gr, m = _seeded(n, seed=100 + variant)
    pc, mc = _oracle(p, gr, m, HP)
    pd, gd, md = p.to(DEV), gr.to(DEV), m.to(DEV)
    _lib.tune_set("lion.variant", variant)
    try:
        lion_update(pd, gd, md, HP["lr"], *HP["betas"], HP["weight_decay"])
        torch.cuda.synchronize()
    finally:
        _lib.tune_set("lion.variant", -1)
    assert np.array_equal(_bits32(pd), pc.view(np.uint32)) and np.array_equal(_bits16(md), mc)


def test_adversarial_values():
    n = 8192 + 512
    p, gr, m = _seeded(n, seed=7)
    special = torch.tensor([0.0, -0.0, 1e-45, -1e-45, 1e-38, 3e38, -3e38, float("inf"), -float("inf"), float("nan")])
    k = special.numel()
    p[:k] = special
    gr[k:2 * k] = special
    m[2 * k:3 * k] = special.to(torch.bfloat16)
    p[3 * k:4 * k] = special
    gr[3 * k:4 * k] = special.flip(0)
    gr[4 * k:5 * k] = 0.0
    m[4 * k:5 * k] = 0.0
    pc, mc = _oracle(p, gr, m, HP)
    pd, gd, md = p.to(DEV), gr.to(DEV), m.to(DEV)
    lion_update(pd, gd, md, HP["lr"], *HP["betas"], HP["weight_decay"])
    got_p, got_m = pd.cpu().numpy(), _bits16(md)
    nan = np.isnan(pc)
    assert np.array_equal(np.isnan(got_p), nan)
    assert np.array_equal(got_p.view(np.uint32)[~nan], pc.view(np.uint32)[~nan])
    # NaN momentum: only NaN-ness is defined (torch's own scalar and vector conversions write different payloads)
    m_nan = (mc & 0x7FFF) > 0x7F80
    assert np.array_equal((got_m & 0x7FFF) > 0x7F80, m_nan)
    assert np.array_equal(got_m[~m_nan], mc[~m_nan])


def test_unaligned_views_take_the_scalar_path():
    n = 3 * 8192 + 5
    p, gr, m = _seeded(n + 3, seed=11)
    pc, mc = _oracle(p[1:n + 1].contiguous(), gr[3:n + 3].contiguous(), m[1:n + 1].contiguous(), HP)
    pd, gd, md = p.to(DEV), gr.to(DEV), m.to(DEV)
    pv, gv, mv = pd[1:n + 1], gd[3:n + 3], md[1:n + 1]
    lion_update(pv, gv, mv, HP["lr"], *HP["betas"], HP["weight_decay"])
    assert np.array_equal(_bits32(pv), pc.view(np.uint32)) and np.array_equal(_bits16(mv), mc)
    # elements outside the views are untouched
    assert torch.equal(pd[:1].cpu(), p[:1]) and torch.equal(pd[n + 1:].cpu(), p[n + 1:])
    assert torch.equal(md[:1].cpu(), m[:1]) and torch.equal(md[n + 1:].cpu(), m[n + 1:])


def test_golden_fixture_through_the_kernel():
    z = np.load(GOLDEN)
    p = torch.from_numpy(z["p"].copy()).to(DEV)
    m = torch.from_numpy(z["m_bits"].view(np.int16).copy()).view(torch.bfloat16).to(DEV)
    for step in range(int(z["steps"])):
        g = torch.from_numpy(z["g"][step].copy()).to(DEV)
        lion_update(p, g, m, float(z["lr"]), float(z["beta1"]), float(z["beta2"]), float(z["weight_decay"]))
    assert np.array_equal(_bits32(p), z["p_out"].view(np.uint32))
    assert np.array_equal(_bits16(m), z["m_bits_out"])


def gpt2_small_shapes():
    shapes = [(50257, 768), (1024, 768)]
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,), (768,), (768,), (768, 3072), (3072,), (3072, 768), (768,)]
    shapes += [(768,), (768,)]
    return shapes


def test_gpt2_small_ten_steps_multi_tensor():
    """The GPT-2-small parameter set: 148 tensors, 124,439,808 parameters, 10 steps with fresh seeded gradients;
    parameters and momentum are compared bit for bit with the oracle after every step."""
    shapes = gpt2_small_shapes()
    sizes = [int(np.prod(s)) for s in shapes]
    total = sum(sizes)
    assert len(shapes) == 148 and total == 124_439_808
    gen = torch.Generator().manual_seed(0)
    flat_p = torch.randn(total, generator=gen) * 0.02
    flat_m = (torch.randn(total, generator=gen) * 1e-3).to(torch.bfloat16)
    params, offs, o = [], [], 0
    for s, n in zip(shapes, sizes):
        params.append(torch.nn.Parameter(flat_p[o:o + n].view(s).to(DEV)))
        offs.append(o)
        o += n
    opt = Lion(params, **HP)
    for prm, o_, n in zip(params, offs, sizes):
        opt.state[prm]["exp_avg"] = flat_m[o_:o_ + n].view(prm.shape).to(DEV)   # pre-seeded bf16 momentum
    pc, mc = flat_p.numpy().copy(), _bits16(flat_m)
    for step in range(10):
        g = torch.randn(total, generator=torch.Generator().manual_seed(1000 + step)) * 1e-2
        for prm, o_, n in zip(params, offs, sizes):
            prm.grad = g[o_:o_ + n].view(prm.shape).to(DEV)
        opt.step()
        lo.lion_step_c(pc, g.numpy(), mc, HP["lr"], HP["betas"], HP["weight_decay"], threads=8)
        got_p = torch.cat([prm.detach().reshape(-1) for prm in params]).cpu().numpy()
        got_m = torch.cat([opt.state[prm]["exp_avg"].reshape(-1) for prm in params])
        bad_p = int((got_p.view(np.uint32) != pc.view(np.uint32)).sum())
        bad_m = int((_bits16(got_m) != mc).sum())
        assert bad_p == 0 and bad_m == 0, f"step {step}: {bad_p} parameter and {bad_m} momentum mismatches"


def test_matches_torch_restatement_and_reports_counts():
    """Second checker: the four reference statements run by torch on the CPU (whatever its dispatch does on this
    host). Mismatch counts are reported for it separately from the C oracle's."""
    n = (1 << 22) + 5
    p, gr, m = _seeded(n, seed=21)
    pt, mt = p.clone(), m.clone()
    lo.lion_step_torch([pt], [gr], [mt], **HP)
    pd, gd, md = p.to(DEV), gr.to(DEV), m.to(DEV)
    lion_update(pd, gd, md, HP["lr"], *HP["betas"], HP["weight_decay"])
    bad_p = int((_bits32(pd) != _bits32(pt)).sum())
    bad_m = int((_bits16(md) != _bits16(mt)).sum())
    print(f"vs torch CPU restatement: {bad_p} parameter / {bad_m} momentum mismatches of {n}")
    assert bad_p == 0 and bad_m == 0


def test_optimizer_semantics():
    # lazily created state is bf16 zeros under the key "exp_avg" (lion_optimizer.py:68-73); params without grad are skipped
    a = torch.nn.Parameter(torch.randn(1000, device=DEV))
    b = torch.nn.Parameter(torch.randn(10, 10, device=DEV))
    b0 = b.detach().clone()
    opt = Lion([a, b], lr=1e-3, weight_decay=0.5)
    a.grad = torch.randn_like(a)
    a0, g0 = a.detach().cpu().clone(), a.grad.cpu().clone()
    opt.step()
    assert torch.equal(b.detach(), b0) and "exp_avg" not in opt.state[b]
    st = opt.state[a]["exp_avg"]
    assert st.dtype == torch.bfloat16 and st.shape == a.shape
    pc, mc = a0.numpy().copy(), np.zeros(1000, np.uint16)
    lo.lion_step_c(pc, g0.numpy().copy(), mc, 1e-3, (0.9, 0.99), 0.5)
    assert np.array_equal(_bits32(a), pc.view(np.uint32)) and np.array_equal(_bits16(st), mc)
    # state_dict round trip keeps the key and the values
    sd = opt.state_dict()
    assert "exp_avg" in sd["state"][0]
    opt2 = Lion([a, b], lr=1e-3, weight_decay=0.5)
    opt2.load_state_dict(sd)
    assert torch.equal(opt2.state[a]["exp_avg"], st)
    # a second step after the gradient tensor was replaced (new pointer) rebuilds the table and still matches
    a.grad = torch.randn_like(a)
    g1 = a.grad.cpu().clone()
    opt.step()
    lo.lion_step_c(pc, g1.numpy().copy(), mc, 1e-3, (0.9, 0.99), 0.5)
    assert np.array_equal(_bits32(a), pc.view(np.uint32)) and np.array_equal(_bits16(opt.state[a]["exp_avg"]), mc)


def test_param_groups_use_their_own_hyperparameters():
    a = torch.nn.Parameter(torch.randn(9000, device=DEV))
    b = torch.nn.Parameter(torch.randn(9000, device=DEV))
    opt = Lion([{"params": [a], "lr": 1e-3, "weight_decay": 0.0}, {"params": [b], "betas": (0.95, 0.98)}], lr=1e-4, weight_decay=0.1)
    a.grad, b.grad = torch.randn_like(a), torch.randn_like(b)
    ref = {}
    for name, t, hp in (("a", a, (1e-3, (0.9, 0.99), 0.0)), ("b", b, (1e-4, (0.95, 0.98), 0.1))):
        pc, mc = t.detach().cpu().numpy().copy(), np.zeros(9000, np.uint16)
        lo.lion_step_c(pc, t.grad.cpu().numpy().copy(), mc, *hp)
        ref[name] = (pc, mc)
    opt.step()
    for name, t in (("a", a), ("b", b)):
        assert np.array_equal(_bits32(t), ref[name][0].view(np.uint32))
        assert np.array_equal(_bits16(opt.state[t]["exp_avg"]), ref[name][1])


def test_wrong_dtypes_and_layouts_raise():
    a = torch.nn.Parameter(torch.randn(64, device=DEV, dtype=torch.float64))
    opt = Lion([a])
    a.grad = torch.randn_like(a)
    with pytest.raises(RuntimeError, match="unsupported dtypes"):
        opt.step()
    b = torch.nn.Parameter(torch.randn(64, device=DEV, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="unsupported dtypes"):   # gradient dtype must be the parameter's (lion_update.cu:132)
        lion_update(b.detach(), torch.randn(64, device=DEV), torch.zeros(64, device=DEV, dtype=torch.float16), 1e-4, 0.9, 0.99, 0.0)
    with pytest.raises(RuntimeError, match="exp_avg_dtype"):
        Lion([b], exp_avg_dtype=torch.float64)
    p = torch.randn(8, 8, device=DEV)
    with pytest.raises(RuntimeError, match="expected tensor to be contiguous"):
        lion_update(p, torch.randn(8, 8, device=DEV).t(), torch.zeros(8, 8, device=DEV, dtype=torch.bfloat16), 1e-4, 0.9, 0.99, 0.0)


def test_full_size_properties_1p3b():
    """1,308,622,848 parameters (39 x 2048x8192 + 39 x 8192x2048): too big for the CPU oracle in a test, so the
    size-independent properties are checked: (1) the multi-tensor launch equals per-tensor launches bit for bit on a
    sampled subset, (2) with weight_decay = 0 every parameter moves by exactly f32(lr) up to one rounding,
    (3) a sampled slice of every tensor matches the oracle bit for bit."""
    shapes = [(2048, 8192)] * 39 + [(8192, 2048)] * 39
    n_each = 2048 * 8192
    gen = torch.Generator(device=DEV).manual_seed(0)
    params = [torch.nn.Parameter(torch.randn(s, device=DEV, generator=gen) * 0.02) for s in shapes]
    opt = Lion(params, lr=1e-4, betas=(0.9, 0.99), weight_decay=0.0)
    sample = slice(12345, 12345 + 70001)
    before = []
    for prm in params:
        prm.grad = torch.randn(prm.shape, device=DEV, generator=gen) * 1e-2
        opt.state[prm]["exp_avg"] = (torch.randn(prm.shape, device=DEV, generator=gen) * 1e-3).to(torch.bfloat16)
        before.append((prm.detach().reshape(-1)[sample].cpu(), prm.grad.reshape(-1)[sample].cpu(), opt.state[prm]["exp_avg"].reshape(-1)[sample].cpu()))
    p_first = params[0].detach().clone()
    opt.step()
    torch.cuda.synchronize()
    # (2)
    delta = (params[0].detach().double() - p_first.double()).abs()
    tol = torch.maximum(params[0].detach().abs(), p_first.abs()).float()
    tol = (torch.nextafter(tol, torch.full_like(tol, float("inf"))) - tol).double()
    assert bool(((delta - float(np.float32(1e-4))).abs() <= tol).all())
    # (3) and (1)
    for prm, (p0, g0, m0) in zip(params, before):
        pc, mc = p0.numpy().copy(), _bits16(m0)
        lo.lion_step_c(pc, g0.numpy().copy(), mc, 1e-4, (0.9, 0.99), 0.0)
        assert np.array_equal(_bits32(prm.detach().reshape(-1)[sample]), pc.view(np.uint32))
        assert np.array_equal(_bits16(opt.state[prm]["exp_avg"].reshape(-1)[sample]), mc)
    assert sum(p.numel() for p in params) == 1_308_622_848 and n_each * 78 == 1_308_622_848


# ---------------------------------------------------------------------------------------------------------------
# every (parameter, momentum) dtype combination; fp32 + bf16 above is the tuned path, the other eight share one
# generic kernel. Oracle: lion_step_explicit_typed (pinned on the CPU against the literal torch statements).
# ---------------------------------------------------------------------------------------------------------------
_DTS = [torch.float32, torch.float16, torch.bfloat16]


def _same_bits(a, b):
    a, b = a.detach().cpu(), b.detach().cpu()
    view = torch.int32 if a.dtype == torch.float32 else torch.int16
    nan = a.isnan() & b.isnan()        # a NaN stays a NaN; its payload bits are unspecified
    return bool(torch.equal(a.view(view)[~nan], b.view(view)[~nan]) and torch.equal(a.isnan(), b.isnan()))


def _typed_inputs(n, p_dtype, m_dtype, seed):
    g = torch.Generator().manual_seed(seed)
    p = (torch.randn(n, generator=g) * 0.02).to(p_dtype)
    m = (torch.randn(n, generator=g) * 1e-3).to(m_dtype)
    gr = (torch.randn(n, generator=g) * 1e-2).to(p_dtype)
    return p, gr, m


@pytest.mark.parametrize("n", [1, 7, 8, 511, 512, 8191, 8192, 8193, 5 * 8192 + 77, (1 << 18) + 5])
@pytest.mark.parametrize("m_dtype", _DTS, ids=str)
@pytest.mark.parametrize("p_dtype", _DTS, ids=str)
def test_typed_single_tensor_bit_exact(p_dtype, m_dtype, n):
    p, gr, m = _typed_inputs(n, p_dtype, m_dtype, seed=n)
    if n >= 8:
        p[:8] = torch.tensor([0.0, -0.0, 1.0, -1.0, 60000.0, 6e-8, 1e-30, float("nan")]).to(p_dtype)
        m[:3] = 0.0
        gr[:3] = 0.0                               # u == 0 exactly: sign 0, the parameter only decays
    pe, me = lo.lion_step_explicit_typed(p, gr, m, **HP)
    pd, gd, md = p.to(DEV), gr.to(DEV), m.to(DEV)
    lion_update(pd, gd, md, HP["lr"], *HP["betas"], HP["weight_decay"])
    torch.cuda.synchronize()
    assert _same_bits(pd, pe), "parameters differ from the oracle"
    assert _same_bits(md, me), "momentum differs from the oracle"
    assert _same_bits(gd, gr), "gradient must not be written"


@pytest.mark.parametrize("weight_decay", [0.0, 0.5])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_reference_test_matrix_all_half(weight_decay, dtype):
    # tests/test_lion_optimizer.py:11-53 at a reduced size (3 x 1024 x 1024 instead of 3 x 8192 x 8192): all tensors in
    # one half dtype, lr 1e-3, betas (0.9, 0.99), five steps, momentum created by the optimizer as zeros_like(param);
    # compared after every step with the reference's allclose tolerances against the torch statements AND bit for bit
    # against the explicit formula
    hp = dict(lr=1e-3, betas=(0.9, 0.99), weight_decay=weight_decay)
    g = torch.Generator().manual_seed(0)
    masters = [torch.randn(1024 * 1024, generator=g).to(dtype) for _ in range(3)]
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in masters]
    ref_p = [t.clone() for t in masters]
    ref_m = [torch.zeros_like(t) for t in masters]
    exp_p = [t.clone() for t in masters]
    exp_m = [torch.zeros_like(t) for t in masters]
    opt = Lion(params, **hp)
    for it in range(5):
        grads = [torch.randn(1024 * 1024, generator=g).to(dtype) for _ in range(3)]
        for prm, gr in zip(params, grads):
            prm.grad = gr.to(DEV)
        opt.step()
        lo.lion_step_torch(ref_p, grads, ref_m, **hp)
        torch.cuda.synchronize()
        for i in range(3):
            exp_p[i], exp_m[i] = lo.lion_step_explicit_typed(exp_p[i], grads[i], exp_m[i], **hp)
            st = opt.state[params[i]]["exp_avg"]
            assert st.dtype == dtype                      # zeros_like(param), lion_optimizer.py:68-73
            assert torch.allclose(params[i].detach().cpu(), ref_p[i], rtol=1e-5, atol=1e-2), f"param {i}, iter {it}"
            assert torch.allclose(st.cpu(), ref_m[i], rtol=1e-5, atol=1e-2), f"exp_avg {i}, iter {it}"
            assert _same_bits(params[i], exp_p[i]) and _same_bits(st, exp_m[i]), f"bits differ: tensor {i}, iter {it}"


def test_typed_mixed_dtypes_in_one_optimizer_and_state_dict():
    # one parameter group holding fp32, fp16 and bf16 parameters: one launch per (parameter, momentum) dtype pair;
    # exp_avg_dtype overrides the momentum dtype of new state; state_dict round trip keeps key, dtype and values
    shapes = [(300, 70), (8192,), (5, 4099)]
    dts = [torch.float32, torch.float16, torch.bfloat16]
    g = torch.Generator().manual_seed(3)
    host_p = [(torch.randn(s, generator=g) * 0.05).to(dt) for s, dt in zip(shapes, dts)]
    params = [torch.nn.Parameter(t.clone().to(DEV)) for t in host_p]
    opt = Lion(params, lr=3e-4, betas=(0.95, 0.98), weight_decay=0.01, exp_avg_dtype=torch.float32)
    exp_p = [t.clone().flatten() for t in host_p]
    exp_m = [torch.zeros(t.numel(), dtype=torch.float32) for t in host_p]
    for it in range(3):
        grads = [(torch.randn(s, generator=g) * 0.01).to(dt) for s, dt in zip(shapes, dts)]
        for prm, gr in zip(params, grads):
            prm.grad = gr.to(DEV)
        opt.step()
        for i in range(3):
            exp_p[i], exp_m[i] = lo.lion_step_explicit_typed(exp_p[i], grads[i].flatten(), exp_m[i], 3e-4, (0.95, 0.98), 0.01)
    torch.cuda.synchronize()
    for i in range(3):
        st = opt.state[params[i]]["exp_avg"]
        assert st.dtype == torch.float32 and st.shape == params[i].shape
        assert _same_bits(params[i].detach().flatten(), exp_p[i]) and _same_bits(st.flatten(), exp_m[i])
    sd = opt.state_dict()
    assert all("exp_avg" in s for s in sd["state"].values())
    # torch.optim.Optimizer.load_state_dict casts floating-point state to the parameter's dtype; this class restores the
    # dtype each momentum was saved with, so a resumed run continues on the same rounding points
    opt2 = Lion(params, lr=3e-4, betas=(0.95, 0.98), weight_decay=0.01)
    opt2.load_state_dict(sd)
    grads = [(torch.randn(s, generator=g) * 0.01).to(dt) for s, dt in zip(shapes, dts)]
    for i, prm in enumerate(params):
        st2 = opt2.state[prm]["exp_avg"]
        assert st2.dtype == torch.float32 and torch.equal(st2, opt.state[prm]["exp_avg"])
        prm.grad = grads[i].to(DEV)
    opt2.step()
    torch.cuda.synchronize()
    for i, prm in enumerate(params):
        pe, me = lo.lion_step_explicit_typed(exp_p[i], grads[i].flatten(), exp_m[i], 3e-4, (0.95, 0.98), 0.01)
        assert _same_bits(prm.detach().flatten(), pe) and _same_bits(opt2.state[prm]["exp_avg"].flatten(), me)


def test_resume_from_a_checkpoint_continues_bit_identically():
    # fp32 parameters with the default bf16 momentum: 3 steps, checkpoint (through torch.save / torch.load, as a training
    # script would), 3 more steps on a fresh optimizer - against 6 uninterrupted steps
    import io

    shapes = [(300, 70), (8192,), (5,)]
    g = torch.Generator().manual_seed(21)
    host_p = [torch.randn(s, generator=g) * 0.02 for s in shapes]
    grads = [[torch.randn(s, generator=g) * 0.01 for s in shapes] for _ in range(6)]
    hp = dict(lr=1e-3, betas=(0.9, 0.99), weight_decay=0.1)

    def run(params, opt, steps):
        for it in steps:
            for prm, gr in zip(params, grads[it]):
                prm.grad = gr.to(DEV)
            opt.step()

    straight = [torch.nn.Parameter(t.clone().to(DEV)) for t in host_p]
    opt_s = Lion(straight, **hp)
    run(straight, opt_s, range(6))
    first = [torch.nn.Parameter(t.clone().to(DEV)) for t in host_p]
    opt_a = Lion(first, **hp)
    run(first, opt_a, range(3))
    buf = io.BytesIO()
    torch.save({"params": [p.detach() for p in first], "opt": opt_a.state_dict()}, buf)
    buf.seek(0)
    ckpt = torch.load(buf, weights_only=True)
    resumed = [torch.nn.Parameter(t.clone()) for t in ckpt["params"]]
    opt_b = Lion(resumed, **hp)
    opt_b.load_state_dict(ckpt["opt"])
    assert all(opt_b.state[p]["exp_avg"].dtype == torch.bfloat16 for p in resumed)
    run(resumed, opt_b, range(3, 6))
    torch.cuda.synchronize()
    for a, b in zip(straight, resumed):
        assert _same_bits(a.detach().flatten().cpu(), b.detach().flatten().cpu())
        assert _same_bits(opt_s.state[a]["exp_avg"].flatten().cpu(), opt_b.state[b]["exp_avg"].flatten().cpu())


def test_gradients_accumulated_in_place_and_replaced_between_steps():
    # the step keeps what it learnt about a parameter while its gradient and momentum are the same objects; in-place
    # changes of the gradient must be seen, a replaced gradient or momentum must be picked up
    n = 20000
    g = torch.Generator().manual_seed(4)
    p0 = torch.randn(n, generator=g) * 0.02
    gs = [torch.randn(n, generator=g) * 0.01 for _ in range(4)]
    prm = torch.nn.Parameter(p0.clone().to(DEV))
    opt = Lion([prm], **HP)
    pc, mc = p0.numpy().copy(), np.zeros(n, np.uint16)
    prm.grad = gs[0].to(DEV)
    opt.step()
    lo.lion_step_c(pc, gs[0].numpy().copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    prm.grad.copy_(gs[1].to(DEV))                      # same tensor object, new values
    opt.step()
    lo.lion_step_c(pc, gs[1].numpy().copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    prm.grad = None                                     # zero_grad(set_to_none=True), then a new gradient tensor
    keep_alive = torch.empty(n, device=DEV)             # so that the allocator hands out another address
    prm.grad = gs[2].to(DEV)
    opt.step()
    lo.lion_step_c(pc, gs[2].numpy().copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    new_m = (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16)
    opt.state[prm]["exp_avg"] = new_m.to(DEV)           # momentum replaced by the caller
    mc = new_m.view(torch.int16).numpy().view(np.uint16).copy()
    prm.grad.copy_(gs[3].to(DEV))
    opt.step()
    lo.lion_step_c(pc, gs[3].numpy().copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    old_storage = prm.data
    prm.data = prm.data.clone()                          # the parameter moved to other memory; gradient and momentum objects stay
    opt.step()
    lo.lion_step_c(pc, gs[3].numpy().copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    torch.cuda.synchronize()
    assert np.array_equal(_bits32(prm), pc.view(np.uint32)) and np.array_equal(_bits16(opt.state[prm]["exp_avg"]), mc)
    assert not torch.equal(old_storage, prm.data)       # the step went to the new memory, not to the old one
    del keep_alive


def test_a_bad_gradient_after_good_steps_still_raises():
    # after the first step only a new gradient tensor is looked at again (torch's zero_grad makes one every step): that
    # look must still refuse what the full check refuses, and a good one at a new address or as a new object over the
    # same memory must be used
    g = torch.Generator().manual_seed(9)
    p0 = torch.randn(64, 48, generator=g) * 0.02
    g1, g2, g3 = (torch.randn(64, 48, generator=g) * 0.01 for _ in range(3))
    prm = torch.nn.Parameter(p0.clone().to(DEV))
    opt = Lion([prm], **HP)
    pc, mc = p0.numpy().reshape(-1).copy(), np.zeros(p0.numel(), np.uint16)
    prm.grad = g1.to(DEV)
    opt.step()
    lo.lion_step_c(pc, g1.numpy().reshape(-1).copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    # (a gradient of another dtype never gets this far: torch refuses the assignment)
    prm.grad = g2.to(DEV).t().contiguous().t()          # right shape, other strides
    with pytest.raises(RuntimeError, match="contiguous"):
        opt.step()
    prm.grad = g2.to(DEV)                                # a good one again, another tensor at another address
    opt.step()
    lo.lion_step_c(pc, g2.numpy().reshape(-1).copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    buf = g3.to(DEV)
    prm.grad = buf.view_as(buf)                          # a new tensor object over memory ...
    opt.step()
    lo.lion_step_c(pc, g3.numpy().reshape(-1).copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    buf.copy_(g1.to(DEV))
    prm.grad = buf.view_as(buf)                          # ... and another one over the same memory with new values
    opt.step()
    lo.lion_step_c(pc, g1.numpy().reshape(-1).copy(), mc, HP["lr"], HP["betas"], HP["weight_decay"])
    torch.cuda.synchronize()
    assert np.array_equal(_bits32(prm).reshape(-1), pc.view(np.uint32))
    assert np.array_equal(_bits16(opt.state[prm]["exp_avg"]).reshape(-1), mc)


def test_typed_unaligned_views_and_multi_tensor_equivalence():
    # views at odd element offsets take the element-wise path; a multi-tensor launch equals per-tensor launches
    for p_dtype, m_dtype in ((torch.float16, torch.float16), (torch.bfloat16, torch.float32), (torch.float32, torch.float32)):
        n = 20000
        p, gr, m = _typed_inputs(n + 3, p_dtype, m_dtype, seed=9)
        pe, me = lo.lion_step_explicit_typed(p[3:], gr[3:], m[1:n + 1], **HP)
        pd, gd, md = p.to(DEV), gr.to(DEV), m.to(DEV)
        lion_update(pd[3:], gd[3:], md[1:n + 1], HP["lr"], *HP["betas"], HP["weight_decay"])
        torch.cuda.synchronize()
        assert _same_bits(pd[3:], pe) and _same_bits(md[1:n + 1], me)
        assert _same_bits(pd[:3], p[:3]) and _same_bits(md[:1], m[:1]) and _same_bits(md[n + 1:], m[n + 1:])
