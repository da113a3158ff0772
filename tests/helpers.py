"""Shared test helpers: seeded inputs (CPU generator, so every machine sees the same values) and
torch <-> numpy conversions for bfloat16."""

import numpy as np
import torch

from oracle import quant_oracle as qo

SEED = 1234  # the reference's default seed (inference_generate.py:539)


def gen(seed=SEED):
    return torch.Generator(device="cpu").manual_seed(seed)


def randn_bf16(shape, std=1.0, seed=SEED):
    return (torch.randn(shape, generator=gen(seed), dtype=torch.float32) * std).to(torch.bfloat16)


def bf16_to_np(t):
    """bfloat16 tensor -> float32 numpy array (exact)."""
    return t.detach().cpu().to(torch.float32).numpy()


def np_to_bf16(a):
    """float32 numpy array holding bf16-exact values -> bfloat16 tensor."""
    assert qo.is_bf16_exact(a)
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16)


def weight_with_edge_rows(n, k, g, std=0.02, seed=SEED):
    """bf16 [n, k] ~ N(0, std) with rows/groups that exercise the quantizers' edge cases."""
    w = randn_bf16((n, k), std=std, seed=seed).clone()
    if n >= 8:
        w[0].zero_()                        # all-zero row: scale clamps (int8 eps, int4 1e-6)
        w[1].fill_(0.0123)                  # constant row: max == min
        w[2, :g] = -0.5                     # constant negative group
        w[3, 5] = 3.0                       # single positive outlier
        w[4, 7] = -3.0                      # single negative outlier
        w[5, :g:2] = 0.25                   # two-valued group: exact ties at the ends
        w[5, 1:g:2] = -0.25
        w[6, :k] = torch.linspace(-1, 1, k).to(torch.bfloat16)  # ramp: many .5 rounding ties
    return w
