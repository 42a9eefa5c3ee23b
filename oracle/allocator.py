"""Oracle: Lagrangian bit allocation under an average-bit budget.

Follows /root/reference/kvquant/allocator.py
  effective_bits           :333-342
  calibrate_epsilon        :352-452   (key/value both TurboQuant-MSE, n_outlier = 0)
  optimal_scores_to_bits   :459-663
  ratio_scores_to_bits     :46-148
  scores_to_bits           :11-43

Arithmetic the restatement has to reproduce (torch CPU semantics of the reference):
  * cost[k, i] = fl32( fl32(s_i * eps_k) + fl32( fl32(lam) * b_k ) ): the Python float lam
    is rounded to fp32 before the multiply; two rounded products, one rounded add, no fma;
  * argmin over k keeps the first (lowest-bit) level on a tie;
  * avg = fl32(sum of chosen bits) / fl32(n), the sum being an exact integer;
  * lo, hi, mid and the budget gap are Python floats (fp64).
numpy does each of these the same way when the operands are float32 arrays/scalars.

One thing is left open by the reference: ``s.argsort()`` is not stable, so *which* of
several equal-score tokens is moved by the repair step is implementation-defined.
Here ties keep index order (stable sort).
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np
import torch


def effective_bits(b: int, n_outlier: int = 0, d: int = 128, outlier_min_bits: int = 4) -> float:
    if b == 0 or b >= 16 or n_outlier <= 0:
        return float(b)
    return b + n_outlier * max(0, max(b, outlier_min_bits) - b) / d


def prepare_tables(bit_levels: Sequence[int], target_avg_bits: float, epsilon: dict,
                   eviction_cost: float = 5.0, n_outlier: int = 0, head_dim: int = 128,
                   outlier_min_bits: int = 4, above_target_alpha: float = 1.0):
    """levels, fp32 eps table, fp32 bit-cost table, clamped target (allocator.py:512-577)."""
    levels = sorted(set(int(b) for b in bit_levels))
    target = max(float(levels[0]), min(float(levels[-1]), target_avg_bits))
    eps_raw = [epsilon.get(b, 0.0) for b in levels]
    if eviction_cost != 1.0 and levels[0] == 0:
        eps_raw[0] *= eviction_cost
    if above_target_alpha < 1.0:
        below = [b for b in levels if b <= target_avg_bits and b != 0]
        eps_at_target = epsilon.get(int(target_avg_bits), None)
        if eps_at_target is None and below:
            eps_at_target = epsilon.get(below[-1], 0.0)
        if eps_at_target is not None and eps_at_target > 1e-12:
            for k, b in enumerate(levels):
                if b > target_avg_bits:
                    eps_raw[k] = (1.0 - above_target_alpha) * eps_at_target + above_target_alpha * eps_raw[k]
    eff = [effective_bits(b, n_outlier, head_dim, outlier_min_bits) for b in levels]
    return levels, np.asarray(eps_raw, np.float32), np.asarray(eff, np.float32), eff, target


def sanitise(s: np.ndarray) -> np.ndarray:
    """allocator.py:543-547: negatives -> 0; if some but not all finite, non-finite -> max finite;
    then nan -> 0 (and any remaining inf -> largest fp32)."""
    s = np.maximum(s, np.float32(0.0))
    finite = np.isfinite(s)
    if finite.any() and not finite.all():
        s = np.where(finite, s, s[finite].max())
    return np.nan_to_num(s, nan=0.0).astype(np.float32)


def assign(s: np.ndarray, eps_t: np.ndarray, bits_t: np.ndarray, lam: float):
    """allocator.py:579-584 -> (chosen level index [n], avg as Python float)."""
    lam32 = np.float32(lam)
    cost = s[None, :] * eps_t[:, None] + (lam32 * bits_t)[:, None]
    chosen = cost.argmin(axis=0)
    total = bits_t[chosen].sum(dtype=np.float64)
    avg = float(np.float32(total) / np.float32(len(s)))
    return chosen, avg


def optimal_scores_to_bits(scores, bit_levels, target_avg_bits, epsilon, sink_mask=None,
                           sink_bits: int = 16, eviction_cost: float = 5.0, n_outlier: int = 0,
                           head_dim: int = 128, outlier_min_bits: int = 4,
                           above_target_alpha: float = 1.0, info: Optional[dict] = None):
    """scores (array or tensor, any shape) -> int32 bits of the same shape (allocator.py:459-663)."""
    is_tensor = isinstance(scores, torch.Tensor)
    arr = scores.detach().cpu().float().numpy() if is_tensor else np.asarray(scores, np.float32)
    shape = arr.shape
    flat = arr.reshape(-1).astype(np.float32)
    n = flat.shape[0]
    result = np.zeros(n, np.int32)
    if sink_mask is not None:
        sm = sink_mask.detach().cpu().numpy() if isinstance(sink_mask, torch.Tensor) else np.asarray(sink_mask)
        sm = sm.reshape(-1).astype(bool)
        result[sm] = sink_bits
        active = np.nonzero(~sm)[0]
    else:
        active = np.arange(n)

    def done():
        out = result.reshape(shape)
        return torch.from_numpy(out) if is_tensor else out

    n_active = active.shape[0]
    if n_active == 0:
        return done()
    levels, eps_t, bits_t, eff, target = prepare_tables(
        bit_levels, target_avg_bits, epsilon, eviction_cost, n_outlier, head_dim,
        outlier_min_bits, above_target_alpha)
    K = len(levels)
    if K == 1:
        result[active] = levels[0]
        return done()
    s = sanitise(flat[active])

    lo, hi = 0.0, 1.0
    _, avg_hi = assign(s, eps_t, bits_t, hi)
    n_widen = 0
    while avg_hi > target and hi < 1e8:
        hi *= 10.0
        _, avg_hi = assign(s, eps_t, bits_t, hi)
        n_widen += 1
    for _ in range(64):
        mid = (lo + hi) * 0.5
        _, avg = assign(s, eps_t, bits_t, mid)
        if avg > target:
            lo = mid
        else:
            hi = mid
    lam = (lo + hi) * 0.5
    chosen, avg = assign(s, eps_t, bits_t, lam)

    nominal = np.asarray(levels, np.int32)
    eff_assigned = bits_t[chosen].copy()
    nom_assigned = nominal[chosen].copy()
    gap = (avg - target) * n_active
    moved = 0
    if info is not None:
        info.update(lam=lam, avg=avg, gap=gap, n_widen=n_widen,
                    pre_repair=nom_assigned.copy(), active=active)
    if abs(gap) > 0.5:
        order = np.argsort(s, kind="stable")
        eff_o = eff_assigned[order]
        nom_o = nom_assigned[order]
        if gap > 0:                                    # over budget: demote lowest scores
            for i in range(K - 1):
                delta = float(eff[i + 1]) - float(eff[i])
                if delta <= 0:
                    continue
                at_hi = eff_o == np.float32(eff[i + 1])
                n_dem = min(int(at_hi.sum()), int(gap / delta + 0.5))
                if n_dem <= 0:
                    continue
                pick = np.nonzero(at_hi)[0][:n_dem]
                eff_o[pick] = np.float32(eff[i])
                nom_o[pick] = levels[i]
                moved += n_dem
                gap -= n_dem * delta
                if gap <= 0.5:
                    break
        else:                                          # under budget: promote highest scores
            gap = -gap
            for i in range(K - 2, -1, -1):
                delta = float(eff[i + 1]) - float(eff[i])
                if delta <= 0:
                    continue
                at_lo = eff_o == np.float32(eff[i])
                n_pro = min(int(at_lo.sum()), int(gap / delta + 0.5))
                if n_pro <= 0:
                    continue
                pick = np.nonzero(at_lo)[0][-n_pro:]
                eff_o[pick] = np.float32(eff[i + 1])
                nom_o[pick] = levels[i + 1]
                moved += n_pro
                gap -= n_pro * delta
                if gap <= 0.5:
                    break
        nom_assigned = np.empty_like(nom_o)
        nom_assigned[order] = nom_o
    if info is not None:
        info.update(moved=moved, sanitised=s)
    result[active] = nom_assigned
    return done()


def calibrate_epsilon(d: int, bit_levels: Sequence[int], *, n_samples: int = 4096, seed: int = 42,
                      order: str = "blas") -> dict:
    """Relative round-trip MSE per level with key and value both TurboQuant-MSE
    (allocator.py:352-452 with value_quantizer="mse", n_outlier=0): key rotation seed ``seed``,
    value rotation seed ``seed + 2000``, eps[b] = mean of the two; eps[0] = 1, eps[>=16] = 0."""
    from .quantizer import dequantize, quantize, random_rotation
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    x = torch.randn(n_samples, d, generator=gen).to(torch.float16)
    x_norm_sq = x.float().pow(2).sum(-1).mean().item()
    out: dict[int, float] = {}
    for b in sorted(set(int(v) for v in bit_levels)):
        if b == 0:
            out[0] = 1.0
            continue
        if b >= 16:
            out[b] = 0.0
            continue
        errs = []
        for s in (seed, seed + 2000):
            pi = random_rotation(d, s)
            rec = dequantize(quantize(x, pi, b, order=order), pi)
            errs.append((x.float() - rec.float()).pow(2).sum(-1).mean().item() / max(x_norm_sq, 1e-12))
        out[b] = (errs[0] + errs[1]) / 2.0
    return out


def scores_to_bits(scores: torch.Tensor, bit_levels: Sequence[int]) -> torch.Tensor:
    """Uniform partition of [0, 1] into len(levels) intervals (allocator.py:11-43)."""
    levels = torch.tensor(sorted(bit_levels), dtype=torch.int32)
    if len(bit_levels) == 1:
        return levels[0].expand_as(scores).clone()
    n = len(bit_levels)
    thresholds = torch.linspace(0.0, 1.0, n + 1)[1:-1]
    return levels[torch.bucketize(scores.float(), thresholds)]


def ratio_scores_to_bits(scores: torch.Tensor, bit_levels: Sequence[int], ratios: Sequence[float],
                         sink_mask: Optional[torch.Tensor] = None, sink_bits: int = 16,
                         per_head: bool = True) -> torch.Tensor:
    """Rank-based tiers: the lowest ratios[0] fraction gets levels[0], and so on
    (allocator.py:46-148).  Ties keep index order (stable sort), as above."""
    assert len(bit_levels) == len(ratios)
    shape = scores.shape
    if per_head and scores.dim() >= 2:
        rows = scores.reshape(-1, shape[-1])
        sm = sink_mask.reshape(-1, shape[-1]) if sink_mask is not None else None
        out = torch.empty(rows.shape, dtype=torch.int32)
        for i in range(rows.shape[0]):
            out[i] = ratio_scores_to_bits(rows[i], bit_levels, ratios,
                                          None if sm is None else sm[i], sink_bits, per_head=False)
        return out.reshape(shape)
    flat = scores.flatten()
    n = flat.shape[0]
    result = torch.zeros(n, dtype=torch.int32)
    if sink_mask is not None:
        fs = sink_mask.flatten().bool()
        result[fs] = sink_bits
        idx = (~fs).nonzero(as_tuple=True)[0]
    else:
        idx = torch.arange(n)
    n_active = idx.shape[0]
    if n_active == 0:
        return result.reshape(shape)
    r = torch.tensor(ratios, dtype=torch.float64)
    r = (r / r.sum()).tolist()
    order = torch.argsort(flat[idx], stable=True)
    bits = torch.empty(n_active, dtype=torch.int32)
    tiers = sorted(zip(bit_levels, r), key=lambda t: t[0])
    cursor = 0
    for i, (b, frac) in enumerate(tiers):
        if i == len(tiers) - 1:
            count = n_active - cursor
        else:
            count = min(int(round(frac * n_active)), n_active - cursor)
        bits[order[cursor:cursor + count]] = b
        cursor += count
    result[idx] = bits
    return result.reshape(shape)
