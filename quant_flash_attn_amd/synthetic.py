"""Synthetic q, k, v, dO of the benchmark configurations (seeded, generated on the CPU in fp32, then cast).

Shared by bench.py, the parity tests and __graft_entry__.smoke(): a data generator, not part of the product path
and not part of the oracle."""
from __future__ import annotations

import math

import torch


def make_inputs(config: str, B: int, H: int, N: int, D: int, seed: int = 0, dtype=torch.bfloat16):
    """Synthetic q, k, v, dO with the distributions of the benchmark configurations:
       'normal'  q,k,v ~ N(0,1)                                            (plumbing case)
       'offset'  N(0,1) + per-token mean ~ N(0,0.5)   (nonzero zero-points; headline config)
       'outlier' q,k ~ N(0,1) with ceil(0.01*D) channels per head scaled 20x; v ~ N(0,1)
       'uniform' q,k ~ U(-3,5); v ~ N(0,1)
    """
    g = torch.Generator().manual_seed(seed)
    shape = (B, H, N, D)

    def randn(*s):
        return torch.randn(*s, generator=g, dtype=torch.float32)

    if config == "normal":
        q, k, v = randn(*shape), randn(*shape), randn(*shape)
    elif config == "offset":
        q = randn(*shape) + 0.5 * randn(B, H, N, 1)
        k = randn(*shape) + 0.5 * randn(B, H, N, 1)
        v = randn(*shape) + 0.5 * randn(B, H, N, 1)
    elif config == "outlier":
        q, k, v = randn(*shape), randn(*shape), randn(*shape)
        n_out = max(1, math.ceil(0.01 * D))
        for h in range(H):
            idx = torch.randperm(D, generator=g)[:n_out]
            q[:, h, :, idx] *= 20.0
            k[:, h, :, idx] *= 20.0
    elif config == "uniform":
        q = torch.rand(*shape, generator=g) * 8.0 - 3.0
        k = torch.rand(*shape, generator=g) * 8.0 - 3.0
        v = randn(*shape)
    else:
        raise ValueError(config)
    do = randn(*shape)
    return tuple(t.to(dtype) for t in (q, k, v, do))
