"""Seeded random shapes for the attention backward, against the CPU oracle with the criterion of
test_attention_bwd_gpu.py (the reference's: error within twice that of a half-precision PyTorch evaluation,
tests/test_flash_attention_triton.py:137-141): head dims on and off the two the kernels are laid out for, ragged and
unequal sequence lengths on both sides of the 64-query tiles and 128-key blocks, one to a few dozen (batch, head) pairs,
both dtypes, causal and not. The pipelined dK/dV kernel sees every mix of masked, whole and ragged tiles this way."""
import random

import pytest
import torch

from test_attention_bwd_gpu import _run

pytestmark = pytest.mark.gpu


def _cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        D = rng.choice([64, 128, 128, 64, 96, 40])
        causal = rng.random() < 0.5
        Sq = rng.choice([rng.randint(1, 300), rng.randint(300, 1500), rng.choice([256, 512, 1024, 1088, 2048])])
        Sk = Sq if rng.random() < 0.6 else rng.randint(1, 1500)
        out.append((rng.randint(1, 3), rng.randint(1, 9), Sq, Sk, D, rng.choice([torch.bfloat16, torch.float16]), causal, i))
    return out


@pytest.mark.parametrize("case", _cases(40, 2024), ids=lambda c: f"B{c[0]}H{c[1]}q{c[2]}k{c[3]}d{c[4]}{'c' if c[6] else 'f'}{str(c[5])[6:]}")
def test_random_shape(case):
    B, H, Sq, Sk, D, dtype, causal, seed = case
    _run(B, H, Sq, Sk, D, dtype, causal, seed=seed)
