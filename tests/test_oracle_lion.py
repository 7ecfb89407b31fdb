"""Pins the Lion oracle (oracle/lion_oracle.py, oracle/lion_oracle.c) on the CPU.

The reference's tests hold no golden vectors for this path (tests/test_lion_optimizer.py:25-53 is a run-time
differential test), so the oracle is pinned against (a) the individual torch ops the reference formula calls
(lion_optimizer_ref.py:51,64,65,67), (b) three independent restatements agreeing bit for bit, (c) closed-form
special cases, and (d) the committed fixture tests/golden/lion_small.npz.
"""
import os

import numpy as np
import pytest
import torch

from oracle import lion_oracle as lo

HP = dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "lion_small.npz")


def _inputs(n, seed=0, adversarial=False):
    g = torch.Generator().manual_seed(seed)
    p = torch.randn(n, generator=g) * 0.02
    m = (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16)
    gr = torch.randn(n, generator=g) * 1e-2
    if adversarial:
        # zeros, signed zeros, denormals, huge, inf, nan, and u landing exactly on zero
        special = torch.tensor([0.0, -0.0, 1e-45, -1e-45, 1e-38, 3e38, -3e38, float("inf"), -float("inf"), float("nan")])
        k = special.numel()
        p[:k] = special
        gr[k:2 * k] = special
        m[2 * k:3 * k] = special.to(torch.bfloat16)
        p[3 * k:4 * k] = special
        gr[3 * k:4 * k] = special.flip(0)
        gr[4 * k:5 * k] = 0.0
        m[4 * k:5 * k] = 0.0
    return p, gr, m


def _bits(t):
    return t.view(torch.int16).numpy().view(np.uint16).copy()


def _run_all(p, gr, m, hp, exact_fma=False):
    # torch restatement
    pt, mt = p.clone(), m.clone()
    lo.lion_step_torch([pt], [gr], [mt], hp["lr"], hp["betas"], hp["weight_decay"])
    # numpy restatement
    pn, mn = lo.lion_step_numpy(p.numpy(), gr.numpy(), _bits(m), hp["lr"], hp["betas"], hp["weight_decay"], exact_fma=exact_fma)
    # C restatement
    pc, mc = p.numpy().copy(), _bits(m)
    lo.lion_step_c(pc, gr.numpy().copy(), mc, hp["lr"], hp["betas"], hp["weight_decay"])
    return (pt.numpy(), _bits(mt)), (pn, mn), (pc, mc)


def _same_bits_f32(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("hp", [HP, dict(lr=1e-3, betas=(0.9, 0.99), weight_decay=0.0), dict(lr=1e-3, betas=(0.95, 0.98), weight_decay=0.5)])
def test_three_restatements_agree_bitwise(hp):
    p, gr, m = _inputs(1 << 20, seed=1)
    (pt, mt), (pn, mn), (pc, mc) = _run_all(p, gr, m, hp)
    assert _same_bits_f32(pt, pc) and np.array_equal(mt, mc)
    assert _same_bits_f32(pn, pc) and np.array_equal(mn, mc)


def test_adversarial_values_agree_bitwise():
    p, gr, m = _inputs(4096, seed=2, adversarial=True)
    (pt, mt), (pn, mn), (pc, mc) = _run_all(p, gr, m, HP, exact_fma=True)
    # NaN payloads may differ between libraries; compare NaN-ness and all non-NaN bit patterns
    for a, b in ((pt, pc), (pn, pc)):
        assert np.array_equal(np.isnan(a), np.isnan(b))
        ok = ~np.isnan(a)
        assert np.array_equal(a.view(np.uint32)[ok], b.view(np.uint32)[ok])
    # torch's vectorised fp32->bf16 conversion writes 0xFFFF for NaN where its scalar one writes 0x7FC0: for NaN
    # momentum only NaN-ness is defined, every other pattern must match
    def bf16_nan(b):
        return (b & 0x7FFF) > 0x7F80
    assert np.array_equal(bf16_nan(mt), bf16_nan(mc))
    ok = ~bf16_nan(mc)
    assert np.array_equal(mt[ok], mc[ok]) and np.array_equal(mn, mc)


def test_each_statement_against_the_torch_op_it_restates():
    """A dropped rounding, an fp32 scalar rounded to bf16, or an unfused add would each fail one line here."""
    p, gr, m = _inputs(1 << 20, seed=3)
    lr, (b1, b2), wd = HP["lr"], HP["betas"], HP["weight_decay"]
    c_wd, c_b1, c_1b1, c_nlr, c_b2, c_1b2 = (torch.tensor(float(c), dtype=torch.float32) for c in lo.lion_consts(lr, (b1, b2), wd))
    mf = m.float()
    # :51
    assert torch.equal(p.clone().mul_(1 - lr * wd), p * c_wd)
    # :64 exp_avg * beta1 is bf16, computed with the scalar kept in fp32 (not rounded to bf16 first)
    t1 = m * b1
    assert t1.dtype == torch.bfloat16
    assert torch.equal(t1, (mf * c_b1).to(torch.bfloat16))
    assert not torch.equal(t1, (mf * c_b1.to(torch.bfloat16).float()).to(torch.bfloat16))
    # :64 sum is fp32
    upd = m * b1 + gr * (1 - b1)
    assert upd.dtype == torch.float32
    assert torch.equal(upd, t1.float() + gr * c_1b1)
    # :65 sign(0) == 0, sign(nan) == 0
    assert torch.equal(torch.sign(torch.tensor([0.0, -0.0, float("nan"), 2.0, -3.0])), torch.tensor([0.0, 0.0, 0.0, 1.0, -1.0]))
    # :67 mul_ rounds to bf16, then add_ with alpha is a single-rounding fma
    m1 = m.clone().mul_(b2)
    assert torch.equal(m1, (mf * c_b2).to(torch.bfloat16))
    m2 = m1.clone().add_(gr, alpha=1 - b2)
    fused = (c_1b2.double() * gr.double() + m1.double()).float().to(torch.bfloat16)
    unfused = (c_1b2 * gr + m1.float()).to(torch.bfloat16)
    assert torch.equal(m2, fused)
    assert (m2.view(torch.int16) != unfused.view(torch.int16)).sum().item() > 0, "inputs do not discriminate fused from unfused"


def test_fp64_fma_emulation_matches_exact_fma_on_sample():
    p, gr, m = _inputs(3000, seed=4)
    a = lo.lion_step_numpy(p.numpy(), gr.numpy(), _bits(m), **HP, exact_fma=True)
    b = lo.lion_step_numpy(p.numpy(), gr.numpy(), _bits(m), **HP, exact_fma=False)
    assert _same_bits_f32(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_bf16_rne_against_torch():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1 << 18, generator=g) * torch.logspace(-40, 38, 1 << 18)
    x[:6] = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 1.00390625])  # last: exact tie
    mine, theirs = lo.bf16_rne_bits(x.numpy()), _bits(x.to(torch.bfloat16))
    nan = np.isnan(x.numpy())
    assert np.array_equal(mine[~nan], theirs[~nan])
    assert np.all((mine[nan] & 0x7FFF) > 0x7F80) and np.all((theirs[nan] & 0x7FFF) > 0x7F80)


def test_closed_form_special_cases():
    n = 1 << 14
    p, gr, m = _inputs(n, seed=6)
    pn, gn, mb = p.numpy(), gr.numpy(), _bits(m)
    f32 = np.float32
    # wd = 0 => the decay factor is exactly 1 and |delta p| == f32(lr) wherever the update is non-zero
    p2, _ = lo.lion_step_numpy(pn, gn, mb, 1e-4, (0.9, 0.99), 0.0)
    d = np.abs(p2.astype(np.float64) - pn.astype(np.float64))
    assert np.all(np.abs(d - float(f32(1e-4))) <= np.spacing(np.maximum(np.abs(pn), np.abs(p2))).astype(np.float64))
    # beta1 = 0 => the step direction is sign(g)
    p2, _ = lo.lion_step_numpy(pn, gn, mb, 1e-4, (0.0, 0.99), 0.0)
    assert np.array_equal(np.sign(pn.astype(np.float64) - p2.astype(np.float64)), np.sign(gn).astype(np.float64))
    # beta2 = 0 => momentum becomes bf16(g)  (1 - 0 = 1 exactly, m*0 = 0)
    _, m2 = lo.lion_step_numpy(pn, gn, mb, 1e-4, (0.9, 0.0), 0.0)
    assert np.array_equal(m2, lo.bf16_rne_bits(gn))
    # beta2 = 1 => momentum unchanged (g * 0 added)
    _, m2 = lo.lion_step_numpy(pn, gn, mb, 1e-4, (0.9, 1.0), 0.0)
    assert np.array_equal(m2, mb)
    # g = 0 and m = 0 => sign is 0: p only decays, m stays 0
    z = np.zeros(n, f32)
    p2, m2 = lo.lion_step_numpy(pn, z, np.zeros(n, np.uint16), 1e-4, (0.9, 0.99), 0.1)
    assert _same_bits_f32(p2, (pn * f32(1 - 1e-4 * 0.1)).astype(f32)) and not m2.any()


def test_c_oracle_multithreaded_equals_scalar():
    p, gr, m = _inputs((1 << 20) + 13, seed=7)
    a_p, a_m = p.numpy().copy(), _bits(m)
    b_p, b_m = p.numpy().copy(), _bits(m)
    lo.lion_step_c(a_p, gr.numpy().copy(), a_m, **HP)
    lo.lion_step_c(b_p, gr.numpy().copy(), b_m, **HP, threads=5)
    assert _same_bits_f32(a_p, b_p) and np.array_equal(a_m, b_m)


def test_ten_step_trajectory_torch_vs_c():
    """Fresh seeded gradients each step (seed 1000 + step), as the benchmark configuration prescribes."""
    n = 200_003
    g0 = torch.Generator().manual_seed(0)
    p = torch.randn(n, generator=g0) * 0.02
    m = (torch.randn(n, generator=g0) * 1e-3).to(torch.bfloat16)
    pc, mc = p.numpy().copy(), _bits(m)
    for step in range(10):
        gr = torch.randn(n, generator=torch.Generator().manual_seed(1000 + step)) * 1e-2
        lo.lion_step_torch([p], [gr], [m], **HP)
        lo.lion_step_c(pc, gr.numpy().copy(), mc, **HP)
        assert _same_bits_f32(p.numpy(), pc) and np.array_equal(_bits(m), mc), f"diverged at step {step}"


def test_golden_fixture():
    """tests/golden/lion_small.npz was written by tests/golden/make_golden.py from the torch restatement."""
    z = np.load(GOLDEN)
    hp = dict(lr=float(z["lr"]), betas=(float(z["beta1"]), float(z["beta2"])), weight_decay=float(z["weight_decay"]))
    pc, mc = z["p"].copy(), z["m_bits"].copy()
    for step in range(int(z["steps"])):
        lo.lion_step_c(pc, z["g"][step].copy(), mc, **hp)
    assert _same_bits_f32(pc, z["p_out"]) and np.array_equal(mc, z["m_bits_out"])


_DTS = [torch.float32, torch.float16, torch.bfloat16]


@pytest.mark.parametrize("m_dtype", _DTS, ids=str)
@pytest.mark.parametrize("p_dtype", _DTS, ids=str)
@pytest.mark.parametrize("hp", [dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1), dict(lr=1e-3, betas=(0.95, 0.98), weight_decay=0.0)],
                         ids=["north-star", "ref-test"])
def test_explicit_typed_formula_equals_the_torch_statements(p_dtype, m_dtype, hp):
    # the spelled-out rounding sequence (what the typed kernel implements) against the literal reference statements
    # executed by torch on the CPU, for all nine dtype combinations, three steps in a row, bit for bit
    # (n is a power of two on purpose: for two tensors of one half dtype, torch's CPU add_(other, alpha) runs its
    # vectorised fp32 path on whole vectors and a scalar path - which rounds alpha * other to the half type first - on
    # the few leftover elements at the end of each thread's range; the vectorised behaviour is the one restated)
    g0 = torch.Generator().manual_seed(11)
    n = 1 << 18
    p = (torch.randn(n, generator=g0) * 0.02).to(p_dtype)
    m = (torch.randn(n, generator=g0) * 1e-3).to(m_dtype)
    # adversarial entries: zeros (sign(0) = 0), values that make u cancel exactly, large and tiny magnitudes
    p[:8] = torch.tensor([0.0, -0.0, 1.0, -1.0, 65504.0, 6e-8, 1e-30, -3.0]).to(p_dtype)
    m[:4] = 0.0
    pe, me = p.clone(), m.clone()
    for step in range(3):
        gr = (torch.randn(n, generator=g0) * 1e-2).to(p_dtype)
        gr[:4] = 0.0
        gr[8] = 0.0
        pe, me = lo.lion_step_explicit_typed(pe, gr, me, hp["lr"], hp["betas"], hp["weight_decay"])
        lo.lion_step_torch([p], [gr], [m], hp["lr"], hp["betas"], hp["weight_decay"])
        assert torch.equal(pe.view(torch.int16 if p_dtype != torch.float32 else torch.int32), p.view(torch.int16 if p_dtype != torch.float32 else torch.int32)), f"params differ at step {step}"
        assert torch.equal(me.view(torch.int16 if m_dtype != torch.float32 else torch.int32), m.view(torch.int16 if m_dtype != torch.float32 else torch.int32)), f"momentum differs at step {step}"
