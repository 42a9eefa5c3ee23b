"""Oracle: decode-time compression of the 128-token buffer (TEST INFRASTRUCTURE ONLY).

Follows /root/reference/kvquant/adaptive_backend_press.py
  _record_observed_ratios          :243-290   level shares per (layer, kv-head) seen at prefill
  _allocate_bits_via_cached_ratios :198-241   rank tiers per kv-head with those shares
  _flush_decode_buffer             :464-595   score -> min-max normalise -> allocate
  _flush_attention                 :601-665   current query (GQA mean) against the buffered keys
and uses ``oracle.scorer.risk_score_with_attn`` (scorer.py:406-416) and
``oracle.allocator.ratio_scores_to_bits`` (allocator.py:46-148), both pinned by the reference's
own output vectors in tests/golden.

The loops over (batch, head) with boolean masks are kept as the reference writes them; the product
batches them.  Pins (tests/test_oracle_flush.py): the attention weights against an independent fp64
softmax per (batch, head) on shuffled flat inputs, row sums of one, the GQA mean against a loop
over the group; the recorded shares against a hand count; the cached-ratio levels against the
golden ``ratio_scores_to_bits`` vectors (one head = the plain routine) and against the
renormalisation worked out by hand.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import numpy as np
import torch

from .allocator import ratio_scores_to_bits
from .scorer import risk_score_with_attn


def flush_attention(q_last: torch.Tensor, buf_keys: torch.Tensor, positions: np.ndarray,
                    num_kv_heads: int) -> torch.Tensor:
    """Weights [N] of the current query over the buffered keys (adaptive_backend_press.py:636-665).

    q_last [B, Hq, d] is the (RoPE'd) query of the newest position; buf_keys [N, d] with
    positions [N, 3] = (batch, kv-head, token), any order.  The G query heads of a kv-head are
    averaged BEFORE the dot product; softmax runs over the entries of each (batch, head)."""
    B, Hq, d = q_last.shape
    G = Hq // num_kv_heads
    q_kv = q_last.reshape(B, num_kv_heads, G, d).mean(dim=2)
    bi = torch.from_numpy(np.asarray(positions[:, 0], np.int64))
    hi = torch.from_numpy(np.asarray(positions[:, 1], np.int64))
    q_per_entry = q_kv[bi, hi]
    logits = (q_per_entry * buf_keys).sum(-1) / math.sqrt(d)
    attn = torch.zeros_like(logits)
    for b in range(B):
        for h in range(num_kv_heads):
            m = (bi == b) & (hi == h)
            if m.any():
                attn[m] = torch.softmax(logits[m], dim=0)
    return attn


def flush_scores(buf_keys: torch.Tensor, buf_values: torch.Tensor, attn: Optional[torch.Tensor],
                 positions: np.ndarray, num_kv_heads: int, *, epsilon: float = 1e-2,
                 use_scorer: bool = True) -> torch.Tensor:
    """Min-max normalised scores [N] fp32 of the buffered tokens (adaptive_backend_press.py:497-536)."""
    if attn is not None and use_scorer:
        bi = torch.from_numpy(np.asarray(positions[:, 0], np.int64))
        hi = torch.from_numpy(np.asarray(positions[:, 1], np.int64))
        B = int(bi.max().item()) + 1 if positions.size else 1
        scores = torch.zeros_like(attn, dtype=torch.float32)
        for b in range(B):
            for h in range(num_kv_heads):
                m = (bi == b) & (hi == h)
                if not m.any():
                    continue
                s = risk_score_with_attn(buf_keys[m].unsqueeze(0), buf_values[m].unsqueeze(0),
                                         attn[m].unsqueeze(0), epsilon)
                scores[m] = s.squeeze(0).float()
    elif attn is not None:
        scores = attn.pow(2) * buf_values.pow(2).sum(-1)
    else:
        scores = buf_keys.pow(2).sum(-1) + buf_values.pow(2).sum(-1)
    return minmax(scores)


def minmax(scores: torch.Tensor) -> torch.Tensor:
    """adaptive_backend_press.py:531-536.  Scores that are not finite go through torch's own rules: a NaN makes
    min() and max() NaN, the comparison below fails and every score becomes 0.5; an infinite score makes the range
    infinite, itself NaN and every finite score 0.  The stable sort of the ranking puts NaN behind every number."""
    lo, hi = scores.min(), scores.max()
    if hi - lo > 1e-8:
        return (scores - lo) / (hi - lo)
    return torch.full_like(scores, 0.5)


def record_observed_ratios(bits: torch.Tensor, sink_tokens: int, buffer_size: int) -> dict:
    """{kv-head: ((level, share), ...)} over the bulk of a prefill allocation [B, Hkv, T]: sink
    prefix and the protected tail cut off; the last batch row wins (adaptive_backend_press.py:243-290)."""
    out = {}
    if bits.dim() != 3 or bits.shape[-1] == 0:
        return out
    B, H, T = bits.shape
    start = min(int(sink_tokens), T) if sink_tokens > 0 else 0
    end = T - min(int(buffer_size), T) if buffer_size > 0 else T
    if end <= start:
        start, end = 0, T
    bulk = bits[..., start:end]
    if bulk.shape[-1] == 0:
        return out
    flat = bulk.reshape(B * H, -1)
    for row in range(B * H):
        uniq, counts = torch.unique(flat[row], return_counts=True)
        total = counts.sum().item()
        if total == 0:
            continue
        fracs = (counts.float() / total).tolist()
        out[row % H] = tuple(sorted(zip(uniq.tolist(), fracs)))
    return out


def cached_ratio_bits(scores: torch.Tensor, positions: np.ndarray, num_kv_heads: int,
                      observed: dict, allowed_levels: Sequence[int]) -> Optional[torch.Tensor]:
    """Levels [N] int32 from the shares recorded at prefill, or None when a head has none
    (adaptive_backend_press.py:198-241).  Levels outside `allowed_levels` (0 bits, when decode-time
    eviction is off) are dropped and the rest renormalised; all batch rows of a kv-head are ranked
    together."""
    allowed = set(int(b) for b in allowed_levels)
    if not all(h in observed for h in range(num_kv_heads)):
        return None
    bits = torch.empty(scores.shape, dtype=torch.int32)
    hi = torch.from_numpy(np.asarray(positions[:, 1], np.int64))
    for h in range(num_kv_heads):
        kept = [(b, r) for b, r in observed[h] if b in allowed and r > 0]
        if not kept:
            return None
        total = sum(r for _, r in kept)
        levels, ratios = zip(*[(b, r / total) for b, r in kept])
        m = hi == h
        if not m.any():
            continue
        bits[m] = ratio_scores_to_bits(scores[m], tuple(levels), tuple(ratios)).to(torch.int32)
    return bits


def flush_levels(q_last: Optional[torch.Tensor], buf_keys: torch.Tensor, buf_values: torch.Tensor,
                 positions: np.ndarray, num_kv_heads: int, observed: dict,
                 allowed_levels: Sequence[int], *, epsilon: float = 1e-2):
    """(attention weights, normalised scores, levels) of one flush with cached shares."""
    attn = None if q_last is None else flush_attention(q_last, buf_keys, positions, num_kv_heads)
    scores = flush_scores(buf_keys, buf_values, attn, positions, num_kv_heads, epsilon=epsilon)
    return attn, scores, cached_ratio_bits(scores, positions, num_kv_heads, observed, allowed_levels)
