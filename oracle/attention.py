"""Oracle: one-token decode attention over a (materialised) mixed-precision cache.

What the reference executes (/root/reference/kvquant/attention_patch.py:30-55 wrapping the HF
attention function, on the tensors written by ``materialize``/``materialize_quantized_into``,
/root/reference/kvquant/tq_adaptive_backend.py:439-464): softmax(q K^T * scaling) V with GQA
head sharing, where evicted keys are overwritten by a "fake key" whose weight underflows to
zero (attention_patch.py:13-27, 45-48).  The arithmetic itself lives in torch SDPA / flash
attention, which the reference does not pin; the oracle is the textbook formula in fp64 with
evicted positions removed from the softmax.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def decode_attention(q: torch.Tensor, keys: torch.Tensor, values: torch.Tensor,
                     visible: Optional[torch.Tensor] = None,
                     scaling: Optional[float] = None) -> torch.Tensor:
    """q [B, Hq, d]; keys/values [B, Hkv, T, d]; visible bool [B, Hkv, T] -> fp64 [B, Hq, d]."""
    B, Hq, d = q.shape
    Hkv = keys.shape[1]
    G = Hq // Hkv
    scale = 1.0 / math.sqrt(d) if scaling is None else scaling
    k = keys.double()[:, :, None].expand(B, Hkv, G, keys.shape[2], d).reshape(B, Hq, -1, d)
    v = values.double()[:, :, None].expand(B, Hkv, G, keys.shape[2], d).reshape(B, Hq, -1, d)
    logits = torch.einsum("bhd,bhtd->bht", q.double(), k) * scale
    if visible is not None:
        vis = visible[:, :, None].expand(B, Hkv, G, keys.shape[2]).reshape(B, Hq, -1)
        logits = logits.masked_fill(~vis, float("-inf"))
    w = torch.softmax(logits, dim=-1)
    return torch.einsum("bht,bhtd->bhd", w, v)


def decode_attention_state(q: torch.Tensor, state, scaling: Optional[float] = None) -> torch.Tensor:
    """Attention of q over ``state.materialize()`` with the state's evicted positions removed."""
    k, v = state.materialize()
    return decode_attention(q, k, v, state.visible_mask(), scaling)
