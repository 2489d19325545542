"""Seeded synthetic inputs shared by the parity tests and the benchmark."""
from __future__ import annotations

import math

import torch


def make_inputs(N, H, V, dtype, seed, ignore_frac=0.0, ignore_index=-1, zipf=False, w_dtype=None,
                w_std=None, device="cpu"):
    """x ~ N(0,1); W ~ truncated normal(std 1/sqrt(H), +-3 std); labels uniform or Zipf(1.1)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, H, generator=g, dtype=torch.float32)
    std = w_std if w_std is not None else 1.0 / math.sqrt(H)
    w = torch.empty(H, V, dtype=torch.float32)
    torch.nn.init.trunc_normal_(w, mean=0.0, std=std, a=-3 * std, b=3 * std, generator=g)
    if zipf:
        p = (torch.arange(1, V + 1, dtype=torch.float64)) ** -1.1
        cdf = torch.cumsum(p, 0) / p.sum()
        u = torch.rand(N, generator=g, dtype=torch.float64)
        y = torch.searchsorted(cdf, u).clamp_(max=V - 1).to(torch.int64)
    else:
        y = torch.randint(0, V, (N,), generator=g, dtype=torch.int64)
    if ignore_frac > 0:
        drop = torch.rand(N, generator=g) < ignore_frac
        y[drop] = ignore_index
    x = x.to(dtype)
    w = w.to(w_dtype if w_dtype is not None else dtype)
    return x.to(device), y.to(device), w.to(device)


def rel_errors(got, ref):
    """(max_abs(diff)/max_abs(ref), ||diff||_2/||ref||_2) in float64."""
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    d = got - ref
    return (d.abs().max() / ref.abs().max()).item(), (d.norm() / ref.norm()).item()
