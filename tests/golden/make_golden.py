"""Writes the committed fixtures in this directory. Run from the repo root: ``python tests/golden/make_golden.py``.

The reference's tests hold no stored vectors for either path (they are run-time differential tests), and no
reference file is imported here. The vectors come from library routines that are independent of the oracle they
pin:

* ``lion_small.npz``  - three steps of the four reference statements (lion_optimizer_ref.py:51,64,65,67) executed
  with torch CPU tensor ops on seeded inputs, including values that land on rounding ties and zeros.
* ``attn_small.npz``  - torch.nn.functional.scaled_dot_product_attention (fp32, CPU) and torch.logsumexp on seeded
  fp16-rounded inputs, causal and non-causal, in the [B,H,S,D] layout of flash_attention.py:30-37.
"""
import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def make_lion():
    n, steps = 4099, 3
    lr, (b1, b2), wd = 1e-4, (0.9, 0.99), 0.1
    gen = torch.Generator().manual_seed(0)
    p = torch.randn(n, generator=gen) * 0.02
    m = (torch.randn(n, generator=gen) * 1e-3).to(torch.bfloat16)
    g = torch.stack([torch.randn(n, generator=torch.Generator().manual_seed(1000 + s)) * 1e-2 for s in range(steps)])
    # a few special values: zero gradient with zero momentum, signed zeros, a huge and a tiny value
    g[:, :4] = 0.0
    m[:4] = 0.0
    p[4:8] = torch.tensor([0.0, -0.0, 3e38, 1e-42])
    p0, m0 = p.clone(), m.clone()
    with torch.no_grad():
        for s in range(steps):
            p.mul_(1 - lr * wd)
            update = m * b1 + g[s] * (1 - b1)
            p.add_(torch.sign(update), alpha=-lr)
            m.mul_(b2).add_(g[s], alpha=1 - b2)
    np.savez_compressed(
        os.path.join(HERE, "lion_small.npz"),
        p=p0.numpy(), g=g.numpy(), m_bits=m0.view(torch.int16).numpy().view(np.uint16),
        p_out=p.numpy(), m_bits_out=m.view(torch.int16).numpy().view(np.uint16),
        lr=lr, beta1=b1, beta2=b2, weight_decay=wd, steps=steps,
    )


def make_attn():
    B, H, S, D = 1, 2, 128, 64
    gen = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(B, H, S, D, generator=gen).to(torch.float16) for _ in range(3))
    scale = 1.0 / math.sqrt(D)
    out = {}
    for causal in (False, True):
        o = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal, scale=scale)
        s = (q.float() @ k.float().transpose(-1, -2)) * scale
        if causal:
            s = s.masked_fill(torch.ones(S, S, dtype=torch.bool).triu(1), float("-inf"))
        tag = "causal" if causal else "full"
        out[f"o_{tag}"] = o.numpy()
        out[f"lse_{tag}"] = torch.logsumexp(s, dim=-1).numpy()
    np.savez_compressed(
        os.path.join(HERE, "attn_small.npz"),
        q=q.view(torch.int16).numpy().view(np.uint16), k=k.view(torch.int16).numpy().view(np.uint16),
        v=v.view(torch.int16).numpy().view(np.uint16), scale=scale, **out,
    )


if __name__ == "__main__":
    make_lion()
    make_attn()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
