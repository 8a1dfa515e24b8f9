"""Seeded synthetic inputs shared by the tests (CPU tensors; GPU tests move them over)."""

from __future__ import annotations

import math

import numpy as np
import torch


def single_inputs(M, K, N, r, p=0.1, seed=0, dtype=torch.bfloat16, bias=False):
    """X~N(0,1), W~N(0,0.02), A kaiming-uniform(a=sqrt 5), B~N(0,0.01), dY~N(0,1), Bernoulli keep-mask."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    bound = 1.0 / math.sqrt(K)  # kaiming_uniform_(a=sqrt(5)) on [r, K]
    a = ((torch.rand(r, K, generator=g) * 2 - 1) * bound).to(dtype)
    b = (torch.randn(N, r, generator=g) * 0.01).to(dtype)
    dy = torch.randn(M, N, generator=g).to(dtype)
    gm = torch.Generator().manual_seed(seed + 1)
    mask = torch.rand(M, K, generator=gm) >= p if p > 0 else None
    bias_t = (torch.randn(N, generator=g) * 0.1).to(dtype) if bias else None
    return dict(x=x, w=w, a=a, b=b, dy=dy, mask=mask, bias=bias_t)


def lognormal_segments(total_tokens, n_adapters, seed=0, mu=6.5, sigma=0.8, lo=64, hi=4096):
    """Lengths ~ lognormal clipped to [lo, hi], drawn until they sum to total_tokens (last one
    truncated), dealt round-robin to the adapters; returns tokens per adapter."""
    rng = np.random.default_rng(seed)
    lens, tot = [], 0
    while tot < total_tokens:
        n = int(np.clip(rng.lognormal(mu, sigma), lo, hi))
        n = min(n, total_tokens - tot)
        lens.append(n)
        tot += n
    per = [0] * n_adapters
    for i, n in enumerate(lens):
        per[i % n_adapters] += n
    return [p for p in per if p > 0]


def multi_inputs(seq_len_list, K, N, ranks, p_list, seed=0, dtype=torch.bfloat16, block=128, bias=False):
    g = torch.Generator().manual_seed(seed)
    padded = [((n - 1) // block + 1) * block for n in seq_len_list]
    Mp = sum(padded)
    x = torch.randn(Mp, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    dy = torch.randn(Mp, N, generator=g).to(dtype)
    a_list, b_list = [], []
    for i, r in enumerate(ranks):
        ga = torch.Generator().manual_seed(seed + 10 + i)
        a_list.append(((torch.rand(r, K, generator=ga) * 2 - 1) / math.sqrt(K)).to(dtype))
        b_list.append((torch.randn(N, r, generator=ga) * 0.01).to(dtype))
    gm = torch.Generator().manual_seed(seed + 1)
    u = torch.rand(Mp, K, generator=gm)
    row_p = torch.cat([torch.full((pl,), float(p)) for pl, p in zip(padded, p_list)])
    mask = u >= row_p[:, None] if any(p > 0 for p in p_list) else None
    bias_t = (torch.randn(N, generator=g) * 0.1).to(dtype) if bias else None
    return dict(x=x, w=w, dy=dy, a_list=a_list, b_list=b_list, mask=mask, padded=padded, bias=bias_t)


def golden(name: str):
    """A fixture of tests/golden (JSON data)."""
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)) as f:
        return json.load(f)
