"""CPU oracle for the fused Lion step (TEST INFRASTRUCTURE ONLY - never imported by the product).

Three independent restatements of ``fast_ops/lion/lion_optimizer_ref.py:41-67`` for fp32 parameters, fp32
gradients and bf16 momentum:

* ``lion_step_torch``  - the four reference statements (:51, :64, :65, :67) written with the same torch tensor
  ops on CPU tensors. Its rounding points are whatever torch's type promotion does, which is what "bit-exact to
  the reference formula" means. It is also the CPU baseline that bench.py times.
* ``lion_step_numpy``  - every rounding point spelled out with numpy float32 arithmetic and integer
  round-to-nearest-even bf16 packing; the fused multiply-add of statement :67 is emulated exactly with Python
  fractions for small inputs or with float64 (``exact_fma=False``; double rounding is possible in principle).
* ``lion_step_c``      - ``oracle/lion_oracle.c`` (scalar C, ``fmaf`` from libm), loaded with ctypes. Exact FMA,
  fast enough for 10^8 elements, independent of torch's CPU dispatch.

The per-element sequence, with the six scalars computed in Python double and rounded once to fp32
(``lion_consts``)::

    p1 = f32(p * c_wd)                                  # :51  p.data.mul_(1 - lr*wd)
    t1 = bf16(f32(f32(m) * c_b1))                       # :64  exp_avg * beta1 is a bf16 tensor
    t2 = f32(g * c_1b1)                                 # :64  grad * (1 - beta1)
    u  = f32(f32(t1) + t2)                              # :64  bf16 + fp32 -> fp32
    s  = (u > 0) - (u < 0)                              # :65  torch.sign: 0 for +-0 and for NaN
    p2 = f32(p1 + c_nlr * s)                            # :65  add_(sign, alpha=-lr); the product is exact
    m1 = bf16(f32(f32(m) * c_b2))                       # :67  in-place mul_ rounds to bf16
    m2 = bf16(fma32(c_1b2, g, f32(m1)))                 # :67  add_(grad, alpha=1-beta2) is a fused multiply-add

``lion_step_torch`` takes any dtypes; for the other eight (parameter, momentum) dtype combinations the rounding
points are spelled out in ``lion_step_explicit_typed``.

Pinned by tests/test_oracle_lion.py: the three restatements agree bit-for-bit on random and adversarial inputs,
each statement is compared against the single torch op it restates, and the closed-form special cases hold
(wd = 0, beta1 = 0, beta2 = 0, beta2 = 1, g = m = 0, |delta p| = f32(lr) exactly).
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from fractions import Fraction
from typing import Sequence, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))


def lion_consts(lr: float, betas: Tuple[float, float], weight_decay: float) -> Tuple[np.float32, ...]:
    """(c_wd, c_b1, c_1b1, c_nlr, c_b2, c_1b2): Python-double expressions of the reference, rounded once to fp32."""
    b1, b2 = betas
    return (
        np.float32(1 - lr * weight_decay),   # :51
        np.float32(b1),                      # :64
        np.float32(1 - b1),                  # :64
        np.float32(-lr),                     # :65
        np.float32(b2),                      # :67
        np.float32(1 - b2),                  # :67
    )


# ---------------------------------------------------------------------------------------------------------------
# 1. torch restatement (the reference's own ops)
# ---------------------------------------------------------------------------------------------------------------
@torch.no_grad()
def lion_step_torch(
    params: Sequence[torch.Tensor],
    grads: Sequence[torch.Tensor],
    exp_avgs: Sequence[torch.Tensor],
    lr: float,
    betas: Tuple[float, float],
    weight_decay: float,
) -> None:
    """In-place Lion step over lists of CPU tensors; statement for statement lion_optimizer_ref.py:51,64,65,67."""
    beta1, beta2 = betas
    for p, grad, exp_avg in zip(params, grads, exp_avgs):
        p.mul_(1 - lr * weight_decay)                               # :51
        update = exp_avg * beta1 + grad * (1 - beta1)                # :64
        p.add_(torch.sign(update), alpha=-lr)                        # :65
        exp_avg.mul_(beta2).add_(grad, alpha=1 - beta2)              # :67


@torch.no_grad()
def lion_step_explicit_typed(p: torch.Tensor, g: torch.Tensor, m: torch.Tensor, lr: float, betas: Tuple[float, float],
                             weight_decay: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """One step for ANY combination of parameter/gradient dtype P and momentum dtype M in {fp32, fp16, bf16}, with
    every rounding point spelled out: fp32 arithmetic, each tensor-valued intermediate of lion_optimizer_ref.py
    :51,:64,:65,:67 rounded to the dtype PyTorch's type promotion gives it. Returns (p_new, m_new); inputs untouched.

        p1 = rP(p * c_wd)                         t1 = rM(m * c_b1)      t2 = rP(g * c_1b1)
        u  = rR(t1 + t2),  R = P if P == M else fp32                     s = sign(u) (0 for 0 and NaN)
        p2 = rP(p1 + a_nlr * s)                   m2 = rM(fma(a_1b2, g, rM(m * c_b2)))

    a_nlr, a_1b2 are -lr and 1 - beta2 in fp32, except when P == M is a half type: torch converts the ``alpha`` of an
    add_ between two tensors of one half dtype to that dtype first. The fused multiply-add is emulated in float64
    (the product of two fp32 values is exact there; a double rounding of the sum is possible in principle).
    Pinned by tests/test_oracle_lion.py against lion_step_torch (the literal torch statements) for all nine (P, M)."""
    P, M = p.dtype, m.dtype
    assert g.dtype == P
    c_wd, c_b1, c_1b1, c_nlr, c_b2, c_1b2 = (torch.tensor(float(c), dtype=torch.float32) for c in lion_consts(lr, betas, weight_decay))
    R = P if P == M else torch.float32
    if P == M and P != torch.float32:
        c_nlr = c_nlr.to(P).float()
        c_1b2 = c_1b2.to(P).float()
    r = lambda x, dt: x.to(dt).float()
    pf, gf, mf = p.float(), g.float(), m.float()
    p1 = r(pf * c_wd, P)
    t1 = r(mf * c_b1, M)
    t2 = r(gf * c_1b1, P)
    u = r(t1 + t2, R)
    s = torch.sign(u)
    p2 = (p1 + c_nlr * s).to(P)
    m1 = r(mf * c_b2, M)
    m2 = (c_1b2.double() * gf.double() + m1.double()).float().to(M)
    return p2, m2


# ---------------------------------------------------------------------------------------------------------------
# 2. numpy restatement with explicit rounding
# ---------------------------------------------------------------------------------------------------------------
def bf16_rne_bits(x: np.ndarray) -> np.ndarray:
    """fp32 array -> uint16 bf16 bit patterns, round-to-nearest-even, NaN -> 0x7FC0 (c10::BFloat16 semantics)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    bias = ((u >> 16) & 1) + 0x7FFF
    r = ((u + bias) >> 16).astype(np.uint16)
    r[np.isnan(x)] = 0x7FC0
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _fma32_exact(a: np.float32, b: np.ndarray, c: np.ndarray) -> np.ndarray:
    """Exact single-rounding fma in fp32 via rational arithmetic (slow; small inputs only)."""
    out = np.empty(b.shape, np.float32)
    fa = Fraction(float(a))
    for i in range(b.size):
        bi, ci = float(b.flat[i]), float(c.flat[i])
        if not (np.isfinite(bi) and np.isfinite(ci)):
            out.flat[i] = np.float32(np.float64(a) * np.float64(bi) + np.float64(ci))
            continue
        exact = fa * Fraction(bi) + Fraction(ci)
        if exact == 0:
            # sign of an exact zero sum under round-to-nearest: +0 unless both addends are -0
            prod_neg = (np.signbit(a) != np.signbit(b.flat[i]))
            out.flat[i] = np.float32(-0.0) if (prod_neg and np.signbit(c.flat[i])) else np.float32(0.0)
            continue
        # float(Fraction) is correctly rounded to double; pick the nearest fp32 among its neighbours (ties to even)
        cand = np.float32(float(exact))
        lo = np.nextafter(cand, np.float32(-np.inf))
        hi = np.nextafter(cand, np.float32(np.inf))
        best = min((lo, cand, hi), key=lambda t: (abs(Fraction(float(t)) - exact), int(np.float32(t).view(np.uint32)) & 1))
        out.flat[i] = best
    return out


def lion_step_numpy(
    p: np.ndarray, g: np.ndarray, m_bits: np.ndarray, lr: float, betas: Tuple[float, float], weight_decay: float,
    exact_fma: bool = False,
) -> Tuple[np.ndarray, np.ndarray]:
    """One step on flat arrays. p, g float32; m_bits uint16 (bf16 patterns). Returns (p_new float32, m_new uint16)."""
    c_wd, c_b1, c_1b1, c_nlr, c_b2, c_1b2 = lion_consts(lr, betas, weight_decay)
    p = np.ascontiguousarray(p, np.float32)
    g = np.ascontiguousarray(g, np.float32)
    with np.errstate(all="ignore"):
        mf = bf16_bits_to_f32(m_bits)
        p1 = (p * c_wd).astype(np.float32)
        t1 = bf16_bits_to_f32(bf16_rne_bits((mf * c_b1).astype(np.float32)))
        t2 = (g * c_1b1).astype(np.float32)
        u = (t1 + t2).astype(np.float32)
        s = (u > 0).astype(np.float32) - (u < 0).astype(np.float32)
        p2 = (p1 + (c_nlr * s).astype(np.float32)).astype(np.float32)
        m1 = bf16_bits_to_f32(bf16_rne_bits((mf * c_b2).astype(np.float32)))
        if exact_fma:
            f = _fma32_exact(c_1b2, g, m1)
        else:
            f = (np.float64(c_1b2) * g.astype(np.float64) + m1.astype(np.float64)).astype(np.float32)
        m2 = bf16_rne_bits(f)
    return p2, m2


# ---------------------------------------------------------------------------------------------------------------
# 3. C restatement (oracle/lion_oracle.c)
# ---------------------------------------------------------------------------------------------------------------
_C_LIB = None


def build_c_oracle(force: bool = False) -> str:
    """Compile oracle/lion_oracle.c with gcc into oracle/liblion_oracle.so (a checker, not the product)."""
    so = os.path.join(_HERE, "liblion_oracle.so")
    src = os.path.join(_HERE, "lion_oracle.c")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-C", _HERE, "liblion_oracle.so"] + (["-B"] if force else []))
    return so


def _c_lib() -> ctypes.CDLL:
    global _C_LIB
    if _C_LIB is None:
        so = os.path.join(_HERE, "liblion_oracle.so")
        if not os.path.exists(so):
            build_c_oracle()
        lib = ctypes.CDLL(so)
        lib.lion_oracle_step.restype = None
        lib.lion_oracle_step.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64] + [ctypes.c_float] * 6
        lib.lion_oracle_step_mt.restype = None
        lib.lion_oracle_step_mt.argtypes = lib.lion_oracle_step.argtypes + [ctypes.c_int]
        _C_LIB = lib
    return _C_LIB


def lion_step_c(p: np.ndarray, g: np.ndarray, m_bits: np.ndarray, lr: float, betas: Tuple[float, float],
                weight_decay: float, threads: int = 1) -> None:
    """In-place step on flat C-contiguous arrays (p float32, g float32, m_bits uint16)."""
    assert p.dtype == np.float32 and g.dtype == np.float32 and m_bits.dtype == np.uint16
    assert p.flags.c_contiguous and g.flags.c_contiguous and m_bits.flags.c_contiguous
    assert p.size == g.size == m_bits.size
    c = [ctypes.c_float(float(x)) for x in lion_consts(lr, betas, weight_decay)]
    lib = _c_lib()
    if threads > 1:
        lib.lion_oracle_step_mt(p.ctypes.data, g.ctypes.data, m_bits.ctypes.data, p.size, *c, threads)
    else:
        lib.lion_oracle_step(p.ctypes.data, g.ctypes.data, m_bits.ctypes.data, p.size, *c)
