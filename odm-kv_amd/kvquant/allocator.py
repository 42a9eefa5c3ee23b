"""Score -> bit-level mapping on the GPU.

Same functions and signatures as the reference's kvquant/allocator.py: ``optimal_scores_to_bits``
(:459-663) runs in libodmkv (batched bisection on the Lagrange multiplier, integer histograms,
exact repair); ``calibrate_epsilon`` (:352-452) measures the round-trip error of the GPU
quantiser on the reference's seeded sample; ``effective_bits`` (:333-342); the two small helpers
the decode-time flush uses, ``ratio_scores_to_bits`` (:46-148) and ``scores_to_bits`` (:11-43),
stay PyTorch (they see at most a few thousand tokens).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import lib

DEFAULT_BIT_LEVELS: tuple[int, ...] = (0, 1, 2, 4, 8)


def scores_to_bits(scores: torch.Tensor, bit_levels: tuple[int, ...] = DEFAULT_BIT_LEVELS) -> torch.Tensor:
    """Uniform partition of [0, 1] into len(bit_levels) intervals."""
    assert len(bit_levels) >= 1
    levels = torch.tensor(sorted(bit_levels), dtype=torch.int32, device=scores.device)
    if len(bit_levels) == 1:
        return levels[0].expand_as(scores).clone()
    n = len(bit_levels)
    cuts = torch.linspace(0.0, 1.0, n + 1)[1:-1].to(scores.device)
    return levels[torch.bucketize(scores.float(), cuts)]


def ratio_scores_to_bits(scores: torch.Tensor, bit_levels: tuple[int, ...], ratios: tuple[float, ...],
                         sink_mask: Optional[torch.Tensor] = None, sink_bits: int = 16,
                         per_head: bool = True) -> torch.Tensor:
    """Rank-based tiers: the lowest ``ratios[0]`` share of the non-sink tokens gets the lowest
    level and so on; ties keep index order."""
    assert len(bit_levels) == len(ratios), (
        f"bit_levels ({len(bit_levels)}) and ratios ({len(ratios)}) must have the same length")
    shape = scores.shape
    if per_head and scores.dim() >= 2:
        rows = scores.reshape(-1, shape[-1])
        masks = sink_mask.reshape(-1, shape[-1]) if sink_mask is not None else None
        out = torch.empty(rows.shape, dtype=torch.int32, device=scores.device)
        for r in range(rows.shape[0]):
            out[r] = ratio_scores_to_bits(rows[r], bit_levels, ratios,
                                          None if masks is None else masks[r], sink_bits, per_head=False)
        return out.reshape(shape)
    flat = scores.flatten()
    result = torch.zeros(flat.shape[0], dtype=torch.int32, device=scores.device)
    if sink_mask is not None:
        sinks = sink_mask.flatten().bool()
        result[sinks] = sink_bits
        active = (~sinks).nonzero(as_tuple=True)[0]
    else:
        active = torch.arange(flat.shape[0], device=scores.device)
    n_active = int(active.shape[0])
    if n_active == 0:
        return result.reshape(shape)
    share = torch.tensor(ratios, dtype=torch.float64)
    share = (share / share.sum()).tolist()
    order = torch.argsort(flat[active], stable=True)
    bits = torch.empty(n_active, dtype=torch.int32, device=scores.device)
    tiers = sorted(zip(bit_levels, share), key=lambda t: t[0])
    cursor = 0
    for i, (b, frac) in enumerate(tiers):
        count = n_active - cursor if i == len(tiers) - 1 else min(int(round(frac * n_active)), n_active - cursor)
        bits[order[cursor:cursor + count]] = b
        cursor += count
    result[active] = bits
    return result.reshape(shape)


def effective_bits(b: int, n_outlier: int = 0, d: int = 128, outlier_min_bits: int = 4) -> float:
    if b == 0 or b >= 16 or n_outlier <= 0:
        return float(b)
    return b + n_outlier * max(0, max(b, outlier_min_bits) - b) / d


_epsilon_cache: dict[tuple, dict[int, float]] = {}


@torch.no_grad()
def calibrate_epsilon(d: int, bit_levels: Sequence[int], *, n_samples: int = 4096, seed: int = 42,
                      device="cuda", value_group_size: int = 32, n_outlier: int = 0,
                      outlier_min_bits: int = 4, value_quantizer: str = "minmax") -> dict[int, float]:
    """Relative round-trip MSE per level: mean of the key quantiser (rotation seed ``seed``) and the
    value quantiser (rotation seed ``seed + 2000``) on a seeded 4096 x d fp16 Gaussian sample;
    eps[0] = 1, eps[>=16] = 0.  Memoised on every argument that changes the result."""
    from .tq_backend import TurboQuantMSE, normalize_value_quantizer
    if n_outlier > 0:
        raise NotImplementedError("outlier-channel separation is not built (n_outlier must be 0)")
    if normalize_value_quantizer(value_quantizer) != "mse" and any(b not in (0, 1, 16) for b in bit_levels):
        raise NotImplementedError("only value_quantizer='mse' is built")
    device = torch.device(device)
    key = (d, tuple(sorted(bit_levels)), seed, value_group_size, n_outlier, outlier_min_bits, "mse", n_samples)
    if key in _epsilon_cache:
        return _epsilon_cache[key]
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    x = torch.randn(n_samples, d, generator=gen).to(device=device, dtype=torch.float16)
    xf = x.float()
    x_norm_sq = xf.pow(2).sum(-1).mean().item()
    eps: dict[int, float] = {}
    for b in sorted(set(int(v) for v in bit_levels)):
        if b == 0:
            eps[0] = 1.0
            continue
        if b >= 16:
            eps[b] = 0.0
            continue
        errs = []
        for s in (seed, seed + 2000):
            q = TurboQuantMSE(d, b, device=device, dtype=torch.float16, seed=s)
            rec = q.dequantize(q.quantize(x))
            errs.append((xf - rec.float()).pow(2).sum(-1).mean().item() / max(x_norm_sq, 1e-12))
        eps[b] = (errs[0] + errs[1]) / 2.0
    _epsilon_cache[key] = eps
    return eps


def _eps_table(levels, target_avg_bits, epsilon, eviction_cost, above_target_alpha):
    """Host-side shaping of the error table (allocator.py:549-569)."""
    eps_raw = [epsilon.get(b, 0.0) for b in levels]
    if eviction_cost != 1.0 and levels[0] == 0:
        eps_raw[0] *= eviction_cost
    if above_target_alpha < 1.0:
        below = [b for b in levels if b <= target_avg_bits and b != 0]
        at_target = epsilon.get(int(target_avg_bits), None)
        if at_target is None and below:
            at_target = epsilon.get(below[-1], 0.0)
        if at_target is not None and at_target > 1e-12:
            for k, b in enumerate(levels):
                if b > target_avg_bits:
                    eps_raw[k] = (1.0 - above_target_alpha) * at_target + above_target_alpha * eps_raw[k]
    return eps_raw


_TARGETS: dict = {}        # (device, budgets) -> the budgets as an fp64 device tensor


def _targets_on(dev: torch.device, tgt: torch.Tensor) -> torch.Tensor:
    """The per-row budgets on the device.  A model asks for the same few budgets layer after layer; uploading eight
    bytes from pageable memory costs a staging copy and a small kernel every call, so the uploaded tensors are kept
    (they are never written again; the upload is waited for once, so that any stream may read them)."""
    key = (dev.type, dev.index if dev.index is not None else torch.cuda.current_device(), tuple(tgt.tolist()))
    hit = _TARGETS.get(key)
    if hit is None:
        if len(_TARGETS) >= 256:
            _TARGETS.clear()
        hit = _TARGETS[key] = tgt.to(dev)
        torch.cuda.current_stream(dev).synchronize()
    return hit


def optimal_scores_to_bits_batched(scores: torch.Tensor, bit_levels, targets, epsilon: dict,
                                   *, n_sink: int = 0, period: Optional[int] = None,
                                   sink_mask: Optional[torch.Tensor] = None, sink_bits: int = 16,
                                   eviction_cost: float = 5.0, above_target_alpha: float = 1.0,
                                   return_stats: bool = False):
    """Rows of independent problems in one go: scores [rows, n] fp32 on the GPU, one budget per row.

    Sinks are either the first ``n_sink`` tokens of every ``period`` tokens (the [Hkv, T] layout
    flattened) or an explicit bool mask.  Returns int32 bits [rows, n] (and, on request, the level
    histogram [rows, K] and the multipliers [rows])."""
    _lib.require_gpu(scores, "scores")
    levels = sorted(set(int(b) for b in bit_levels))
    rows, n = scores.shape
    dev = scores.device
    s = scores.float().contiguous()
    if isinstance(targets, (int, float)):
        targets = [float(targets)] * rows
    tgt = torch.as_tensor(targets, dtype=torch.float64).reshape(rows)
    # every row shares one error table, shaped for its own budget only when alpha < 1
    if above_target_alpha < 1.0 and len(set(tgt.tolist())) > 1:
        raise ValueError("above_target_alpha < 1 needs one common target per call")
    eps_raw = _eps_table(levels, float(tgt[0]), epsilon, eviction_cost, above_target_alpha)
    bits = torch.empty(rows, n, dtype=torch.int32, device=dev)
    counts = torch.empty(rows, len(levels), dtype=torch.int32, device=dev) if return_stats else None
    lam = torch.empty(rows, dtype=torch.float64, device=dev) if return_stats else None
    mask = None
    if sink_mask is not None:
        mask = sink_mask.reshape(rows, n).to(device=dev, dtype=torch.uint8).contiguous()
    ws_bytes = lib.odmkv_allocate_workspace_bytes(rows, n)
    ws = _lib.workspace(dev, ws_bytes, "allocate")
    lv = (C.c_int32 * len(levels))(*levels)
    ep = (C.c_double * len(levels))(*eps_raw)
    tgt_dev = _targets_on(dev, tgt)
    _lib.check(lib.odmkv_allocate(
        s.data_ptr(), rows, n, _lib.ptr(mask), int(period or n), int(n_sink), int(sink_bits),
        lv, len(levels), ep, tgt_dev.data_ptr(), bits.data_ptr(), _lib.ptr(counts), _lib.ptr(lam),
        ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev)))
    return (bits, counts, lam) if return_stats else bits


def optimal_scores_to_bits(scores: torch.Tensor, bit_levels: tuple[int, ...], target_avg_bits: float,
                           epsilon: dict[int, float], sink_mask: Optional[torch.Tensor] = None,
                           sink_bits: int = 16, eviction_cost: float = 5.0, n_outlier: int = 0,
                           head_dim: int = 128, outlier_min_bits: int = 4,
                           above_target_alpha: float = 1.0) -> torch.Tensor:
    """Lagrangian-optimal per-token bit allocation under an average-bit budget: every non-sink token
    takes argmin_b s * eps'(b) + lambda * b, lambda chosen by bisection so the mean meets the
    budget, then the gap is closed by moving the lowest (highest) scores one level."""
    if n_outlier > 0:
        raise NotImplementedError("outlier-channel separation is not built (n_outlier must be 0)")
    shape = scores.shape
    if scores.numel() == 0:
        return torch.empty(shape, dtype=torch.int32, device=scores.device)
    flat = scores.reshape(1, -1)
    mask = None if sink_mask is None else sink_mask.reshape(1, -1)
    bits = optimal_scores_to_bits_batched(flat, bit_levels, [float(target_avg_bits)], epsilon,
                                          sink_mask=mask, sink_bits=sink_bits,
                                          eviction_cost=eviction_cost,
                                          above_target_alpha=above_target_alpha)
    return bits.reshape(shape)
