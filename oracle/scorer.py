"""Oracle: the ODM risk score  s = (p + eps)^2 * (|v|^2 + |k|^2/d * |v - o|^2).

Follows /root/reference/kvquant/scorer.py
  ExpectedAttentionScorer._query_statistics   :184-202
  _expected_core_internals                    :285-318
  _pad_sinks_and_normalize                    :321-325  (grain "global" = identity, :118-119)
  RiskScorer.score_prefill                    :385-404
  RiskScorer.score_with_attn                  :406-416
  ExpectedAttentionScorer.score_prefill       :204-257  (expected_attention_score below)
window_attention / window_risk_score have no counterpart in the reference (it scores with the mean
query only): they restate the textbook definition, causal softmax attention of each of the last W
queries averaged over queries and GQA group, and are pinned by brute force and special cases only.
  _NormFallback.score_prefill                 :145-147 (+ _normalize_scores "layer" :130-134)
and /root/reference/kvquant/attention_utils.py
  _repeat_kv :19-26, _get_query_states :29-54, _apply_avg_rope :57-115.

Like the reference the code is dtype-generic: whatever dtype the caller passes is
the dtype the attention estimate is computed in.  Parity tests pass fp32 tensors.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[b, Hkv, t, d] -> [b, Hkv*n_rep, t, d]; q-head q reads kv-head q // n_rep."""
    if n_rep == 1:
        return x
    b, h, t, d = x.shape
    return x[:, :, None].expand(b, h, n_rep, t, d).reshape(b, h * n_rep, t, d)


def _num_heads(module) -> Optional[int]:
    n = getattr(module, "num_heads", None)
    cfg = getattr(module, "config", None)
    if n is None and cfg is not None:
        n = getattr(cfg, "num_attention_heads", None)
    return n


def query_states(module, hidden: torch.Tensor) -> torch.Tensor:
    """Pre-RoPE queries [b, Hq, T, d] of an HF attention module (attention_utils.py:29-54)."""
    b, t, _ = hidden.shape
    n_heads = _num_heads(module)
    if n_heads is None:
        raise AttributeError("cannot determine num_heads")
    cfg = getattr(module, "config", None)
    head_dim = getattr(module, "head_dim", None)
    if head_dim is None and cfg is not None:
        head_dim = getattr(cfg, "head_dim", None)
    if head_dim is None:
        head_dim = hidden.shape[-1] // n_heads
    if hasattr(module, "qkv_proj"):
        q = module.qkv_proj(hidden)[..., : n_heads * head_dim]
    elif hasattr(module, "q_proj"):
        q = module.q_proj(hidden)
    else:
        raise NotImplementedError(type(module).__name__)
    q = q.view(b, t, n_heads, head_dim).transpose(1, 2)
    if hasattr(module, "q_norm"):
        q = module.q_norm(q)
    return q


def avg_rope(module, mu: torch.Tensor, q_len: int, n_future: int) -> torch.Tensor:
    """mu -> R_avg mu with R_avg the mean RoPE matrix over positions [q_len, q_len+n_future)
    (attention_utils.py:57-115).  Identity without ``rotary_emb`` or with n_future <= 0."""
    rotary = getattr(module, "rotary_emb", None)
    if rotary is None or n_future <= 0:
        return mu
    pos = torch.arange(q_len, q_len + n_future, device=mu.device).unsqueeze(0)
    cos, sin = rotary(mu, pos)
    cos = cos.to(device=mu.device, dtype=mu.dtype)[0]
    sin = sin.to(device=mu.device, dtype=mu.dtype)[0]
    d = mu.shape[-1]
    half = d // 2
    eye = torch.eye(d, dtype=mu.dtype, device=mu.device)
    perm = torch.zeros(d, d, dtype=mu.dtype, device=mu.device)
    perm[half:, :half] = torch.eye(half, dtype=mu.dtype, device=mu.device)
    perm[:half, half:] = -torch.eye(half, dtype=mu.dtype, device=mu.device)
    r_avg = (cos.unsqueeze(-1) * eye + sin.unsqueeze(-1) * perm).mean(dim=0)
    return torch.matmul(mu, r_avg.T)


def mean_query(module, hidden: torch.Tensor, n_sink: int, n_future: int) -> torch.Tensor:
    """[1, Hq, d]: mean over positions >= n_sink of the pre-RoPE queries, then averaged RoPE
    (scorer.py:184-202 with use_covariance=False)."""
    if hidden.dim() == 2:
        hidden = hidden.unsqueeze(0)
    q_len = hidden.shape[1]
    if q_len <= n_sink:
        raise ValueError("not enough tokens to estimate expected attention")
    q = query_states(module, hidden[:, n_sink:])
    return avg_rope(module, q.mean(dim=2), q_len, n_future)


def expected_attention(keys: torch.Tensor, mu: torch.Tensor, n_sink: int,
                       n_q_heads: int) -> torch.Tensor:
    """p [1, Hkv, T - n_sink]: softmax over core tokens of mu . k / sqrt(d) per q-head,
    then the mean over each GQA group (scorer.py:296-315)."""
    core = keys[:, n_sink:]
    h_kv, t_core, d = core.shape
    groups = n_q_heads // h_kv
    kt = repeat_kv(core.unsqueeze(0), groups).transpose(2, 3)          # [1, Hq, d, Tc]
    logits = torch.matmul(mu.unsqueeze(2), kt).squeeze(2) / math.sqrt(d)
    a = torch.softmax(logits, dim=-1)
    return a.reshape(1, h_kv, groups, t_core).mean(dim=2)


def risk_from_attention(p_raw: torch.Tensor, keys_core: torch.Tensor, values_core: torch.Tensor,
                        epsilon: float) -> torch.Tensor:
    """scorer.py:394-403: p_raw [1, H, Tc] in its own dtype, keys/values [H, Tc, d] -> [1, H, Tc]."""
    d = keys_core.shape[-1]
    p = p_raw[0].float()
    p_hat = p / p.sum(dim=-1, keepdim=True).clamp(min=1e-8)
    o_bar = torch.einsum("ht,htd->hd", p_hat, values_core.float())
    irrep = (values_core.float() - o_bar.unsqueeze(1)).pow(2).sum(dim=-1)
    kn2 = keys_core.unsqueeze(0).float().pow(2).sum(dim=-1)
    vn2 = values_core.unsqueeze(0).float().pow(2).sum(dim=-1)
    return (p_raw + epsilon).pow(2) * (vn2 + (kn2 / float(d)) * irrep.unsqueeze(0))


def pad_sinks(core_scores: torch.Tensor, n_sink: int) -> torch.Tensor:
    """Left-pad n_sink columns with the global maximum (scorer.py:321-325) -> [H, T]."""
    top = float(core_scores.max().item()) if core_scores.numel() else 1.0
    return torch.nn.functional.pad(core_scores, (n_sink, 0), value=top).squeeze(0)


def norm_fallback(keys: torch.Tensor, values: torch.Tensor) -> torch.Tensor:
    """|k| + |v|, min-max normalised over the layer (scorer.py:145-147 with :130-134).

    The fallback scorer is its own object (scorer.py:176) and keeps the class default
    ``normalize_grain = "layer"``; the factory sets "global" on the risk scorer only
    (press_factory.py:59), so this path does normalise."""
    raw = keys.norm(dim=-1) + values.norm(dim=-1)
    if raw.numel() == 0:
        return raw
    lo, hi = raw.min(), raw.max()
    if (hi - lo) < 1e-8:
        return torch.full_like(raw, 0.5)
    return (raw - lo) / (hi - lo)


def risk_score_from_mu(keys: torch.Tensor, values: torch.Tensor, mu: torch.Tensor,
                       n_q_heads: int, *, n_sink: int = 4, epsilon: float = 1e-2) -> torch.Tensor:
    """Scores [Hkv, T] given the (already RoPE-averaged) mean query mu [1, Hq, d]."""
    if keys.shape[1] <= n_sink:
        return torch.ones(keys.shape[:2], dtype=keys.dtype)
    p = expected_attention(keys, mu, n_sink, n_q_heads)
    s = risk_from_attention(p, keys[:, n_sink:], values[:, n_sink:], epsilon)
    return pad_sinks(s, n_sink)


def risk_score_prefill(keys: torch.Tensor, values: torch.Tensor, *, module=None,
                       hidden_states: Optional[torch.Tensor] = None, n_sink: int = 4,
                       epsilon: float = 1e-2, n_future: int = 512) -> torch.Tensor:
    """RiskScorer.score_prefill (scorer.py:385-404), keys/values [Hkv, T, d] -> [Hkv, T]."""
    if module is None or hidden_states is None:
        return norm_fallback(keys, values)
    if keys.shape[1] <= n_sink:
        return torch.ones(keys.shape[:2], dtype=keys.dtype)
    try:
        mu = mean_query(module, hidden_states, n_sink, n_future)
    except (AttributeError, NotImplementedError, ValueError):
        return norm_fallback(keys, values)
    n_q = _num_heads(module) or keys.shape[0]
    return risk_score_from_mu(keys, values, mu, n_q, n_sink=n_sink, epsilon=epsilon)


def risk_score_with_attn(keys: torch.Tensor, values: torch.Tensor, attn: torch.Tensor,
                         epsilon: float = 1e-2) -> torch.Tensor:
    """RiskScorer.score_with_attn (scorer.py:406-416): keys/values [H, T, d], attn [H, T]."""
    p = attn.float()
    p_hat = p / p.sum(dim=-1, keepdim=True).clamp(min=1e-8)
    o_bar = torch.einsum("ht,htd->hd", p_hat, values.float())
    irrep = (values.float() - o_bar.unsqueeze(1)).pow(2).sum(dim=-1)
    kn2 = keys.float().pow(2).sum(dim=-1)
    vn2 = values.float().pow(2).sum(dim=-1)
    return (p + epsilon).pow(2) * (vn2 + (kn2 / float(keys.shape[-1])) * irrep)


def avg_rope_matrix(module, like: torch.Tensor, q_len: int, n_future: int) -> Optional[torch.Tensor]:
    """R_avg [d, d]: element-wise mean over positions [q_len, q_len + n_future) of the RoPE matrices
    diag(cos_p) + diag(sin_p) P (attention_utils.py:83-105); None where the reference returns its
    inputs unchanged."""
    rotary = getattr(module, "rotary_emb", None)
    if rotary is None or n_future <= 0:
        return None
    pos = torch.arange(q_len, q_len + n_future, device=like.device).unsqueeze(0)
    cos, sin = rotary(like, pos)
    cos = cos.to(device=like.device, dtype=like.dtype)[0]
    sin = sin.to(device=like.device, dtype=like.dtype)[0]
    d = like.shape[-1]
    half = d // 2
    eye = torch.eye(d, dtype=like.dtype, device=like.device)
    perm = torch.zeros(d, d, dtype=like.dtype, device=like.device)
    perm[half:, :half] = torch.eye(half, dtype=like.dtype, device=like.device)
    perm[:half, half:] = -torch.eye(half, dtype=like.dtype, device=like.device)
    return (cos.unsqueeze(-1) * eye + sin.unsqueeze(-1) * perm).mean(dim=0)


def query_statistics(module, hidden: torch.Tensor, n_sink: int, n_future: int,
                     use_covariance: bool):
    """(mu [1, Hq, d], cov [1, Hq, d, d] or None) after the averaged RoPE: scorer.py:184-202 with
    attention_utils.py:107-115 (mu' = mu R^T, cov' = R cov R^T)."""
    if hidden.dim() == 2:
        hidden = hidden.unsqueeze(0)
    q_len = hidden.shape[1]
    if q_len <= n_sink:
        raise ValueError("not enough tokens to estimate expected attention")
    q_in = hidden[:, n_sink:]
    q = query_states(module, q_in)
    mu = q.mean(dim=2)
    cov = None
    if use_covariance:
        centered = q - mu.unsqueeze(2)
        cov = torch.einsum("bhsd,bhse->bhde", centered, centered) / q_in.shape[1]
    r = avg_rope_matrix(module, mu, q_len, n_future)
    if r is None:
        return mu, cov
    mu = torch.matmul(mu, r.T)
    if cov is not None:
        cov = torch.matmul(r, torch.matmul(cov, r.T))
    return mu, cov


def expected_attention_score(keys: torch.Tensor, values: torch.Tensor, mu: torch.Tensor,
                             cov: Optional[torch.Tensor], n_q_heads: int, *, n_sink: int = 4,
                             epsilon: float = 0.0, use_vnorm: bool = True) -> torch.Tensor:
    """ExpectedAttentionScorer.score_prefill after the query statistics (scorer.py:227-257),
    before the final normalisation: keys/values [Hkv, T, d], mu [1, Hq, d], cov [1, Hq, d, d] or
    None -> [Hkv, T]."""
    if keys.shape[1] <= n_sink:
        return torch.ones(keys.shape[:2], dtype=keys.dtype)
    k_core, v_core = keys[:, n_sink:], values[:, n_sink:]
    h_kv, t_core, d = k_core.shape
    groups = n_q_heads // h_kv
    kt = repeat_kv(k_core.unsqueeze(0), groups).transpose(2, 3)             # [1, Hq, d, Tc]
    raw = torch.matmul(mu.unsqueeze(2), kt).squeeze(2) / math.sqrt(d)
    if cov is not None:
        raw = raw + torch.einsum("bhdt,bhde,bhet->bht", kt, cov, kt) / d / 2
    raw = torch.softmax(raw, dim=-1)
    raw = raw.reshape(1, h_kv, groups, t_core).mean(dim=2)
    if use_vnorm:
        raw = (raw + epsilon) * v_core.unsqueeze(0).norm(dim=-1)
    return pad_sinks(raw, n_sink)


def window_attention(keys: torch.Tensor, queries: torch.Tensor, n_sink: int, q_pos0: int,
                     scaling: Optional[float] = None) -> torch.Tensor:
    """p [1, Hkv, T - n_sink]: mean over the W window queries and the GQA group of
    softmax_t(q . k_t * scaling) over core tokens, query w (at position q_pos0 + w) seeing keys at
    positions <= its own.  keys [Hkv, T, d], queries [Hq, W, d] (already rotated to their positions)."""
    core = keys[:, n_sink:]
    h_kv, t_core, d = core.shape
    h_q, w, _ = queries.shape
    groups = h_q // h_kv
    scale = d ** -0.5 if scaling is None else scaling
    kx = repeat_kv(core.unsqueeze(0), groups)[0]                                  # [Hq, Tc, d]
    logits = torch.einsum("qwd,qtd->qwt", queries, kx) * scale
    key_pos = n_sink + torch.arange(t_core)
    q_pos = q_pos0 + torch.arange(w)
    logits = logits.masked_fill(key_pos[None, None, :] > q_pos[None, :, None], float("-inf"))
    a = torch.softmax(logits, dim=-1)
    return a.reshape(h_kv, groups * w, t_core).mean(dim=1).unsqueeze(0)


def window_risk_score(keys: torch.Tensor, values: torch.Tensor, queries: torch.Tensor, q_pos0: int, *,
                      n_sink: int = 4, epsilon: float = 1e-2, scaling: Optional[float] = None) -> torch.Tensor:
    """The risk score with the window attention mass in place of the mean query's: [Hkv, T]."""
    p = window_attention(keys, queries, n_sink, q_pos0, scaling)
    return pad_sinks(risk_from_attention(p, keys[:, n_sink:], values[:, n_sink:], epsilon), n_sink)
