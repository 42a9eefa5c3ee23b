"""Query / RoPE / GQA helpers the scorer and the press share (host-side PyTorch, tiny tensors).

Same helper names as the reference's kvquant/attention_utils.py:19-157.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn


def _repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[b, Hkv, t, d] -> [b, Hkv * n_rep, t, d]; query head q reads kv-head q // n_rep."""
    if n_rep == 1:
        return hidden_states
    b, h, t, d = hidden_states.shape
    return hidden_states[:, :, None, :, :].expand(b, h, n_rep, t, d).reshape(b, h * n_rep, t, d)


def _head_geometry(module: nn.Module, hidden_size: int) -> tuple[int, int]:
    cfg = getattr(module, "config", None)
    n_heads = getattr(module, "num_heads", None)
    if n_heads is None and cfg is not None:
        n_heads = getattr(cfg, "num_attention_heads", None)
    if n_heads is None:
        raise AttributeError(f"Cannot determine num_heads from {module.__class__.__name__}")
    head_dim = getattr(module, "head_dim", None)
    if head_dim is None and cfg is not None:
        head_dim = getattr(cfg, "head_dim", None)
    if head_dim is None:
        head_dim = hidden_size // n_heads
    return int(n_heads), int(head_dim)


def _get_query_states(module: nn.Module, hidden_states: torch.Tensor) -> torch.Tensor:
    """Pre-RoPE queries [b, Hq, t, d] of an HF attention module (q_proj or fused qkv_proj, then
    q_norm if the module has one)."""
    b, t, hidden = hidden_states.shape
    n_heads, head_dim = _head_geometry(module, hidden)
    if hasattr(module, "qkv_proj"):
        q = module.qkv_proj(hidden_states)[..., : n_heads * head_dim]
    elif hasattr(module, "q_proj"):
        q = module.q_proj(hidden_states)
    else:
        raise NotImplementedError(f"ExpectedAttentionScorer does not support {module.__class__.__name__}.")
    q = q.view(b, t, n_heads, head_dim).transpose(1, 2)
    if hasattr(module, "q_norm"):
        q = module.q_norm(q)
    return q


def _mean_query_states(module: nn.Module, hidden_states: torch.Tensor) -> torch.Tensor:
    """mean over positions of ``_get_query_states`` -> [b, Hq, d].

    Without a ``q_norm`` the projection is affine, so the mean of the projected rows equals the
    projection of the mean row: one GEMV instead of a [T, hidden] x [hidden, Hq*d] GEMM."""
    if hasattr(module, "q_norm"):
        return _get_query_states(module, hidden_states).mean(dim=2)
    b, t, hidden = hidden_states.shape
    n_heads, head_dim = _head_geometry(module, hidden)
    mean_h = hidden_states.float().mean(dim=1, keepdim=True).to(hidden_states.dtype)
    if hasattr(module, "qkv_proj"):
        q = module.qkv_proj(mean_h)[..., : n_heads * head_dim]
    elif hasattr(module, "q_proj"):
        q = module.q_proj(mean_h)
    else:
        raise NotImplementedError(f"ExpectedAttentionScorer does not support {module.__class__.__name__}.")
    return q.view(b, n_heads, head_dim)


def _aligned_rotary_outputs(rotary_emb, x: torch.Tensor, position_ids: torch.Tensor):
    """RoPE cos/sin on the caller's device and dtype (the root rotary module may live elsewhere)."""
    cos, sin = rotary_emb(x, position_ids)
    return cos.to(device=x.device, dtype=x.dtype), sin.to(device=x.device, dtype=x.dtype)


def _rotate_half(x: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def _apply_rotary_pos_emb_q(q: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    if cos.dim() == 2:
        cos, sin = cos.unsqueeze(0), sin.unsqueeze(0)
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    return (q * cos) + (_rotate_half(q) * sin)


def _apply_avg_rope(module: nn.Module, mu: torch.Tensor, cov: Optional[torch.Tensor], q_len: int,
                    n_future_positions: int, n_samples: int = 8):
    """mu -> R_avg mu and cov -> R_avg cov R_avg^T, R_avg = mean RoPE matrix over positions
    [q_len, q_len + n_future).

    Averaging the rotation matrices element-wise leaves diag(mean cos) + diag(mean sin) P with P
    the half-rotation, i.e. R_avg x = mean(cos) * x + mean(sin) * rotate_half(x): high-frequency
    pairs average towards zero (a low-pass on the query), low-frequency pairs survive.  The
    covariance takes the same map on its rows and then on its columns."""
    rotary_emb = getattr(module, "rotary_emb", None)
    if rotary_emb is None or n_future_positions <= 0:
        return mu, cov
    pos = torch.arange(q_len, q_len + n_future_positions, device=mu.device).unsqueeze(0)
    cos, sin = _aligned_rotary_outputs(rotary_emb, mu, pos)
    c_bar, s_bar = cos[0].mean(dim=0), sin[0].mean(dim=0)

    def r_avg(x):
        return c_bar * x + s_bar * _rotate_half(x)

    mu_out = r_avg(mu)
    if cov is None:
        return mu_out, None
    half = r_avg(cov)                                     # cov R^T  (the map acts on the last axis)
    return mu_out, r_avg(half.transpose(-1, -2)).transpose(-1, -2)
