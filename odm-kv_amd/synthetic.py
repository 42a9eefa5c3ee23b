"""Seeded synthetic workloads of the ODM-KV hot path (no datasets, no checkpoints).

Every tensor is drawn in fp32 from ``torch.Generator(device="cpu")`` and cast afterwards, so a
(config, seed) pair names the same numbers on every machine.  Shapes follow the benchmark
configurations: one layer of K/V per call, ``[Hkv, T, 128]``, sink tokens with 8x norm, a
64-query observation window whose mean is the expected query, and one decode query per head.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

LEVELS = (0, 2, 3, 4, 8, 16)
N_SINK = 4
WINDOW = 128            # trailing tokens kept exact (decode buffer size)
SCORE_EPS = 1e-2
EVICTION_COST = 0.5


@dataclass
class Layer:
    keys: torch.Tensor      # [Hkv, T, d]
    values: torch.Tensor    # [Hkv, T, d]
    mu: torch.Tensor        # [Hq, d] expected query (mean of the observation window)
    query: torch.Tensor     # [Hq, d] decode query
    n_q_heads: int


def gaussian_layer(seed: int, n_kv: int, n_q: int, T: int, d: int = 128, dtype=torch.float16,
                   sink_scale: float = 8.0, window_queries: int = 64) -> Layer:
    """K, V ~ N(0,1) with the first four tokens scaled by 8; mu = mean of 64 N(0,1) queries."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    k = torch.randn(n_kv, T, d, generator=g)
    v = torch.randn(n_kv, T, d, generator=g)
    k[:, :N_SINK] *= sink_scale
    v[:, :N_SINK] *= sink_scale
    qwin = torch.randn(n_q, window_queries, d, generator=g)
    q = torch.randn(n_q, d, generator=g).half().float()      # queries arrive in the model dtype
    return Layer(k.to(dtype), v.to(dtype), qwin.mean(dim=1), q, n_q)


def heavy_tail_layer(seed: int, n_kv: int = 4, n_q: int = 28, T: int = 32768, d: int = 128,
                     dtype=torch.float16) -> Layer:
    """V ~ Student-t(3) and four K channels scaled 20x (stress for the score range)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    k = torch.randn(n_kv, T, d, generator=g)
    z = torch.randn(n_kv, T, d, generator=g)
    chi = torch.randn(3, n_kv, T, d, generator=g).pow(2).sum(0) / 3.0
    v = z / chi.sqrt()
    ch = torch.randperm(d, generator=g)[:4]
    k[..., ch] *= 20.0
    k[:, :N_SINK] *= 8.0
    v[:, :N_SINK] *= 8.0
    qwin = torch.randn(n_q, 64, d, generator=g)
    q = torch.randn(n_q, d, generator=g).half().float()      # queries arrive in the model dtype
    return Layer(k.to(dtype), v.to(dtype), qwin.mean(dim=1), q, n_q)


def lognormal_norm_layer(seed: int, n_kv: int = 8, n_q: int = 32, T: int = 131072, d: int = 128,
                         sigma: float = 1.0, dtype=torch.float16) -> Layer:
    """Gaussian directions with log-normal per-token norms: a wide score range, so that a 2-bit
    budget evicts a large share of the tokens."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    k = torch.randn(n_kv, T, d, generator=g)
    v = torch.randn(n_kv, T, d, generator=g)
    scale = torch.exp(sigma * torch.randn(n_kv, T, 1, generator=g))
    k *= scale
    v *= scale
    k[:, :N_SINK] *= 8.0
    v[:, :N_SINK] *= 8.0
    qwin = torch.randn(n_q, 64, d, generator=g)
    q = torch.randn(n_q, d, generator=g).half().float()      # queries arrive in the model dtype
    return Layer(k.to(dtype), v.to(dtype), qwin.mean(dim=1), q, n_q)


def config(name: str, layer: int = 0, seq: int = 0, T: int | None = None) -> Layer:
    """The layer tensors of one of the five benchmark configurations."""
    if name == "c1":
        return gaussian_layer(1001, 8, 32, T or 4096)
    if name == "c2":
        return gaussian_layer(2002 + layer, 8, 32, T or 32768)
    if name == "c3":
        return gaussian_layer(3003 + seq, 8, 32, T or 8192)
    if name == "c4":
        return lognormal_norm_layer(4004, 8, 32, T or 131072)
    if name == "c5":
        return heavy_tail_layer(5005 + layer, 4, 28, T or 32768)
    raise ValueError(name)


C3_TARGETS = (1.5, 2.0, 3.0)
