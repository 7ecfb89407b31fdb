"""CPU oracle for the attention forward pass (TEST INFRASTRUCTURE ONLY - never imported by the product).

Restates, with torch CPU ops in fp32, what the reference defines:

* output: ``fast_ops/flash_attention/attention_ref.py:41-49,54-59,67`` - upcast q/k/v to fp32, scores =
  (q * scale) . k^T, causal mask = strict upper triangle (top-left aligned) set to -inf, softmax over keys, times v.
  The reference divides q by sqrt(d); the Triton surface takes an arbitrary ``softmax_scale``
  (``flash_attention_triton.py:750``), so the scale is a parameter here and defaults to 1/sqrt(d).
* logsumexp: ``fast_ops/flash_attention/flash_attention_triton.py:201-203,241-243,255`` - natural-log
  logsumexp of the *scaled* scores over the unmasked keys, one fp32 value per query row.
* the tile recurrence itself (``flash_attention_triton.py:128-129,149,169-175,200-213,237-250``) is restated in
  ``online_softmax_tiles`` so that tests can show recurrence == closed form, including the running reference
  being ``lse_i`` rather than ``m_i``.

* backward: ``attention_bwd_oracle`` - the closed-form gradients of the same expression
  (``flash_attention_triton.py:273-315,497-578``).

Layout is the drop-in surface's: Q [B,H,M,D], K/V [B,H,N,D] (``flash_attention.py:30-37``).

Pinned by tests/test_oracle_attention.py against: torch.nn.functional.scaled_dot_product_attention (independent
library routine), torch.logsumexp, a float64 triple-loop brute force on tiny inputs, and closed-form invariants
(V == 1, Q == 0, causal row 0, key permutation, one-hot selection).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch


def dropout_keep_mask(dropout_p: float, seed: int, rng_offset: int, B: int, H: int, M: int, N: int) -> np.ndarray:
    """The reference's dropout mask (flash_attention_triton.py:38-50 hash, :125,:216-217 / :682-691 indices): bool
    [B, H, M, N], True = kept. Index of (b, h, m, n) = rng_offset + (b*H + h)*M*N + m*N + n in 32-bit arithmetic;
    a = index ^ seed;  a ^= a >> 4;  a = (a ^ 0xDEADBEEF) + (a << 5);  a ^= a >> 11;  keep = a > uint32(fp32(p) * fp32(2^32 - 1)).
    Pinned by tests/test_oracle_attention.py: a pure-Python-integer restatement on small shapes, hand-computed hashes,
    the kept fraction, and independence of offset-shifted masks.
    PARITY UNPINNED for one step: the threshold. The reference computes it inside a Triton kernel as
    ``(dropout_p * 4294967295).to(tl.uint32)`` (flash_attention_triton.py:50); that the product is taken in fp32 (so
    that the constant becomes 2^32 and the threshold is trunc(fp32(p) * 2^32)) is an inference about the promotion
    rules of triton 2.0.0.dev20221202, which is not available here, and the reference holds no mask vectors. A double
    or integer product would move the threshold by at most 2^32 * 2^-24 = 256 of 2^32 hash values: one element in 16
    million would flip."""
    idx = (np.arange(B * H * M * N, dtype=np.uint64) + np.uint64(rng_offset % (1 << 32))).astype(np.uint32)
    a = idx ^ np.uint32(seed & 0xFFFFFFFF)
    a = a ^ (a >> np.uint32(4))
    a = ((a ^ np.uint32(0xDEADBEEF)).astype(np.uint64) + (a.astype(np.uint64) << np.uint64(5))).astype(np.uint32)
    a = a ^ (a >> np.uint32(11))
    thr = np.uint32(int(np.float32(dropout_p) * np.float32(4294967295)))
    return (a > thr).reshape(B, H, M, N)


def attention_fwd_oracle(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    causal: bool = False,
    softmax_scale: Optional[float] = None,
    q_chunk: int = 1024,
    dropout: Optional[Tuple[float, int, int]] = None,
    bias: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 softmax(scale * Q K^T + bias + mask) V and its logsumexp. Returns (O fp32 [B,H,M,D], LSE fp32 [B,H,M]).
    ``bias`` broadcasts to [B,H,M,N] and is added to the scaled scores in fp32 (attention_ref.py:50-51,
    flash_attention_triton.py:176-198); the logsumexp includes it.

    Works one (batch, head) slice and ``q_chunk`` query rows at a time so that S = 8192 does not materialise
    the full [B,H,M,N] score tensor (attention_ref.py does; same arithmetic per row).
    """
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4
    B, H, M, D = q.shape
    N = k.shape[2]
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    qf, kf, vf = q.float().cpu(), k.float().cpu(), v.float().cpu()   # attention_ref.py:41-43
    out = torch.empty(B, H, M, D, dtype=torch.float32)
    lse = torch.empty(B, H, M, dtype=torch.float32)
    keep = None
    bias_f = None if bias is None else bias.float().cpu().expand(B, H, M, N)
    if dropout is not None and dropout[0] > 0.0:
        # dropout of the probabilities after the row sums are taken (flash_attention_triton.py:203,216-219): LSE is that
        # of the undropped scores, kept probabilities are scaled by 1 / (1 - p) computed in fp32
        keep = torch.from_numpy(dropout_keep_mask(dropout[0], dropout[1], dropout[2], B, H, M, N))
        keep_scale = float(np.float32(1.0) / (np.float32(1.0) - np.float32(dropout[0])))
    for b in range(B):
        for h in range(H):
            kt = kf[b, h].t()
            for m0 in range(0, M, q_chunk):
                m1 = min(M, m0 + q_chunk)
                scores = (qf[b, h, m0:m1] * scale) @ kt                      # attention_ref.py:46-47
                if bias_f is not None:
                    scores = scores + bias_f[b, h, m0:m1]                     # attention_ref.py:50-51
                if causal:
                    rows = torch.arange(m0, m1).unsqueeze(1)
                    cols = torch.arange(N).unsqueeze(0)
                    scores = scores.masked_fill(cols > rows, float("-inf"))  # attention_ref.py:54-58 (triu, diagonal=1)
                lse[b, h, m0:m1] = torch.logsumexp(scores, dim=-1)
                attn = torch.softmax(scores, dim=-1)                          # attention_ref.py:59
                if keep is not None:
                    attn = torch.where(keep[b, h, m0:m1], attn * keep_scale, torch.zeros_like(attn))
                out[b, h, m0:m1] = attn @ vf[b, h]                            # attention_ref.py:67
    return out, lse


def attention_bwd_oracle(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    d_o: torch.Tensor,
    causal: bool = False,
    softmax_scale: Optional[float] = None,
    dtype: torch.dtype = torch.float32,
    dropout: Optional[Tuple[float, int, int]] = None,
    bias: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Gradients of sum(O * dO) with respect to Q, K, V, in closed form, one (batch, head) at a time:

        P = softmax(scale * Q K^T + mask)        dV = P^T dO           dP = dO V^T
        delta_i = sum_d dO_id O_id               dS = P * (dP - delta) dQ = scale * dS K        dK = scale * dS^T Q

    which is what the reference's backward computes tile by tile (flash_attention_triton.py:273-315 delta pre-pass,
    :497-578 per-tile dv / dp / ds / dk / dq) and what autograd gives for attention_ref.py:41-67. ``dtype`` is the
    arithmetic type (fp32 for the oracle proper, float64 to pin it). With dropout (mask Z = keep / (1 - p), :524-532,
    :551,:599): O = (P * Z) V, dV = (P * Z)^T dO, dP = (dO V^T) * Z, the rest unchanged. A ``bias`` (broadcast to
    [B,H,M,N]) is added to the scaled scores before the softmax (:497-509) and gets no gradient.
    Returns (dQ, dK, dV) in ``dtype`` on the CPU.
    Pinned by tests/test_oracle_attention.py against torch.autograd on the forward expression in float64."""
    B, H, M, D = q.shape
    N = k.shape[2]
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    qf, kf, vf, gf = (t.to(dtype).cpu() for t in (q, k, v, d_o))
    dq, dk, dv = torch.zeros_like(qf), torch.zeros_like(kf), torch.zeros_like(vf)
    z = None
    bias_f = None if bias is None else bias.to(dtype).cpu().expand(B, H, M, N)
    if dropout is not None and dropout[0] > 0.0:
        keep = torch.from_numpy(dropout_keep_mask(dropout[0], dropout[1], dropout[2], B, H, M, N))
        z = keep.to(dtype) * float(np.float32(1.0) / (np.float32(1.0) - np.float32(dropout[0])))
    for b in range(B):
        for h in range(H):
            s = (qf[b, h] * scale) @ kf[b, h].t()
            if bias_f is not None:
                s = s + bias_f[b, h]
            if causal:
                rows = torch.arange(M).unsqueeze(1)
                cols = torch.arange(N).unsqueeze(0)
                s = s.masked_fill(cols > rows, float("-inf"))
            p = torch.softmax(s, dim=-1)
            pz = p if z is None else p * z[b, h]
            o = pz @ vf[b, h]
            dv[b, h] = pz.t() @ gf[b, h]
            dp = gf[b, h] @ vf[b, h].t()
            if z is not None:
                dp = dp * z[b, h]
            delta = (gf[b, h] * o).sum(dim=-1, keepdim=True)
            ds = p * (dp - delta)
            dq[b, h] = (ds @ kf[b, h]) * scale
            dk[b, h] = (ds.t() @ qf[b, h]) * scale
    return dq, dk, dv


def online_softmax_tiles(
    q: np.ndarray, k: np.ndarray, v: np.ndarray, causal: bool, scale: float, block_m: int = 128, block_n: int = 128
) -> Tuple[np.ndarray, np.ndarray]:
    """The reference's tile recurrence for one (batch, head): q [M,D], k/v [N,D] float32 -> (O [M,D], LSE [M]).

    Follows flash_attention_triton.py: state init :128-130, causal loop bound :149, qk :169-170, causal -inf :174-175,
    m_ij / p / l_ij :200-203, accumulator rescale :206-213, PV :237-238, state update :241-243, epilogue :245-250,255.
    P is *not* rounded to half here (this function pins the recurrence, not the operand rounding).
    """
    M, D = q.shape
    N = k.shape[0]
    out = np.zeros((M, D), np.float32)
    lse_out = np.zeros((M,), np.float32)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        for start_m in range(0, M, block_m):
            rows = np.arange(start_m, min(M, start_m + block_m))
            qi = q[rows]
            lse_i = np.full(len(rows), -np.inf, np.float32)
            m_i = np.full(len(rows), -np.inf, np.float32)
            acc = np.zeros((len(rows), D), np.float32)
            end_n = N if not causal else min(start_m + block_m, N)
            for start_n in range(0, end_n, block_n):
                cols = np.arange(start_n, min(N, start_n + block_n))
                qk = (qi @ k[cols].T).astype(np.float32)
                if causal:
                    qk = qk + np.where(rows[:, None] >= cols[None, :], 0.0, -np.inf).astype(np.float32)
                m_ij = np.maximum(qk.max(axis=1) * np.float32(scale), lse_i)
                p = np.exp(qk * np.float32(scale) - m_ij[:, None]).astype(np.float32)
                l_ij = p.sum(axis=1, dtype=np.float32)
                acc = acc * np.exp(m_i - m_ij)[:, None]
                acc = acc + p @ v[cols]
                m_i = m_ij
                lse_i = (m_ij + np.log(np.exp(lse_i - m_ij) + l_ij)).astype(np.float32)
            acc = acc * np.exp(m_i - lse_i)[:, None]
            out[rows] = acc
            lse_out[rows] = lse_i
    return out, lse_out
