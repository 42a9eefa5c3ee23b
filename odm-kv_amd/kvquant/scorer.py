"""KV-unit scoring: the ODM risk score on the GPU.

Class names, constructor arguments and method signatures follow the reference's
kvquant/scorer.py (BaseScorer :29-97, ExpectedAttentionScorer :154-202, RiskScorer :363-416);
the per-token arithmetic runs in libodmkv:

    s_j = (p_j + eps)^2 * ( |v_j|^2 + |k_j|^2 / d * |v_j - o_bar|^2 )

with p the expected attention of the mean (RoPE-averaged) query, averaged over the GQA group.
"""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Optional

import torch
from torch import nn

from . import _lib
from ._lib import lib
from .attention_utils import (  # noqa: F401  (re-exported under the names callers import from here)
    _aligned_rotary_outputs,
    _apply_avg_rope,
    _apply_rotary_pos_emb_q,
    _get_query_states,
    _mean_query_states,
    _repeat_kv,
    _rotate_half,
)


def _normalize_scores(raw: torch.Tensor, *, grain: str = "layer") -> torch.Tensor:
    """Min-max normalisation: "layer" over the whole tensor, "head" per row, "global" none."""
    if raw.numel() == 0 or grain == "global":
        return raw
    if grain == "head" and raw.dim() >= 2:
        lo = raw.amin(dim=-1, keepdim=True)
        hi = raw.amax(dim=-1, keepdim=True)
        span = hi - lo
        out = (raw - lo) / torch.where(span < 1e-8, torch.ones_like(span), span)
        dead = span.squeeze(-1) < 1e-8
        if dead.any():
            out[dead] = 0.5
        return out
    lo, hi = raw.min(), raw.max()
    if (hi - lo) < 1e-8:
        return torch.full_like(raw, 0.5)
    return (raw - lo) / (hi - lo)


class BaseScorer(ABC):
    """Interface every scorer implements."""

    normalize_grain: str = "layer"

    def _maybe_normalize(self, raw: torch.Tensor) -> torch.Tensor:
        return _normalize_scores(raw, grain=self.normalize_grain)

    @abstractmethod
    def score_prefill(self, keys: torch.Tensor, values: torch.Tensor, layer_idx: int, *,
                      module: nn.Module | None = None,
                      hidden_states: torch.Tensor | None = None) -> torch.Tensor:
        """keys/values [H, T, d] -> scores [H, T]."""

    def score_decode(self, key: torch.Tensor, value: torch.Tensor, layer_idx: int, *,
                     module: nn.Module | None = None,
                     hidden_states: torch.Tensor | None = None) -> torch.Tensor:
        return torch.ones(key.shape[0], device=key.device)

    def score_with_attn(self, keys: torch.Tensor, values: torch.Tensor, attn_weights: torch.Tensor, *,
                        module: nn.Module | None = None) -> torch.Tensor:
        eps = float(getattr(self, "epsilon", 0.0) or 0.0)
        return (attn_weights + eps).pow(2) * values.float().pow(2).sum(dim=-1)


class _NormFallback(BaseScorer):
    """|k| + |v|, used when the query statistics cannot be formed."""

    def score_prefill(self, keys, values, layer_idx, *, module=None, hidden_states=None):
        return self._maybe_normalize(keys.norm(dim=-1) + values.norm(dim=-1))

    def score_decode(self, key, value, layer_idx, *, module=None, hidden_states=None):
        return self._maybe_normalize(key.norm(dim=-1) + value.norm(dim=-1))


class ExpectedAttentionScorer(BaseScorer):
    """Expected attention of future queries (kvquant/scorer.py:154-282 of the reference):

        softmax_t( E[q] . k_t / sqrt(d) + k_t^T Cov[q] k_t / (2 d) ) * |v_t|

    with E[q], Cov[q] the mean and covariance of the pre-RoPE queries over the prefill positions
    after the sinks, passed through the averaged future RoPE.  Also holds the query statistics
    shared with ``RiskScorer`` (which switches the covariance off)."""

    def __init__(self, *, n_future_positions: int = 512, n_sink: int = 4, use_covariance: bool = True,
                 use_vnorm: bool = True, epsilon: float = 0.0):
        self.n_future_positions = n_future_positions
        self.n_sink = n_sink
        self.use_covariance = use_covariance
        self.use_vnorm = use_vnorm
        self.epsilon = epsilon
        self._fallback = _NormFallback()

    def _query_statistics(self, module: nn.Module, hidden_states: torch.Tensor):
        q_len = hidden_states.shape[1]
        if q_len <= self.n_sink:
            raise ValueError("not enough tokens to estimate expected attention")
        query_input = hidden_states[:, self.n_sink:]
        if not self.use_covariance:
            mu = _mean_query_states(module, query_input)
            return _apply_avg_rope(module, mu, None, q_len, self.n_future_positions)
        # the covariance is accumulated in fp32 whatever the model's dtype: a 16-bit result of a sum
        # over tens of thousands of positions would overflow or lose the small eigen-directions
        q = _get_query_states(module, query_input).float()            # [b, Hq, t, d]
        mu = q.mean(dim=2)
        centered = q - mu.unsqueeze(2)
        cov = torch.matmul(centered.transpose(-1, -2), centered) / query_input.shape[1]
        return _apply_avg_rope(module, mu, cov, q_len, self.n_future_positions)

    def score_prefill(self, keys, values, layer_idx, *, module=None, hidden_states=None):
        if module is None or hidden_states is None:
            return self._fallback.score_prefill(keys, values, layer_idx)
        if hidden_states.dim() == 2:
            hidden_states = hidden_states.unsqueeze(0)
        if hidden_states.shape[0] != 1:
            raise ValueError("ExpectedAttentionScorer expects a single-sample hidden-state slice.")
        if keys.shape[1] <= self.n_sink:
            return torch.ones(keys.shape[:2], device=keys.device, dtype=keys.dtype)
        try:
            mu, cov = self._query_statistics(module, hidden_states)
        except (AttributeError, NotImplementedError, ValueError):
            return self._fallback.score_prefill(keys, values, layer_idx)
        scores = _launch_score_expected(keys, values, mu[0], None if cov is None else cov[0],
                                        mu.shape[1], self.n_sink, self.epsilon, self.use_vnorm)
        return self._maybe_normalize(scores)

    def score_decode(self, key, value, layer_idx, *, module=None, hidden_states=None):
        return self._fallback.score_decode(key, value, layer_idx, module=module, hidden_states=hidden_states)


def _kv_operands(keys: torch.Tensor, values: torch.Tensor):
    """keys/values as the kernels read them: rows contiguous and 16-byte aligned, equal strides."""
    _lib.require_gpu(keys, "keys")
    if keys.shape[-1] != _lib.HEAD_DIM:
        raise ValueError(f"the HIP kernels are written for head_dim {_lib.HEAD_DIM}, got {keys.shape[-1]}")
    align = 4 if keys.dtype == torch.float32 else 8
    def ok(t):
        return t.stride(-1) == 1 and t.stride(0) % align == 0 and t.stride(1) % align == 0 and t.data_ptr() % 16 == 0
    if not ok(keys) or not ok(values) or keys.stride() != values.stride():
        keys, values = keys.contiguous(), values.contiguous()
    return keys, values


def _launch_score_expected(keys: torch.Tensor, values: torch.Tensor, mu: torch.Tensor,
                           cov: Optional[torch.Tensor], n_q_heads: int, n_sink: int, eps: float,
                           use_vnorm: bool) -> torch.Tensor:
    keys, values = _kv_operands(keys, values)
    H, T, D = keys.shape
    dev = keys.device
    scores = torch.empty(H, T, dtype=torch.float32, device=dev)
    ws_bytes = lib.odmkv_score_workspace_bytes(H, n_q_heads, T)
    ws = _lib.workspace(dev, ws_bytes, "score")
    mu32 = mu.reshape(n_q_heads, D).float().contiguous()
    cov32 = None if cov is None else cov.reshape(n_q_heads, D, D).float().contiguous()
    _lib.check(lib.odmkv_score_expected(
        keys.data_ptr(), values.data_ptr(), _lib.dtype_code(keys), H, T, keys.stride(0), keys.stride(1),
        mu32.data_ptr(), _lib.ptr(cov32), n_q_heads, n_sink, float(eps), int(bool(use_vnorm)),
        scores.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev)))
    return scores


def _launch_score(keys: torch.Tensor, values: torch.Tensor, mu: Optional[torch.Tensor],
                  attn: Optional[torch.Tensor], n_q_heads: int, n_sink: int, eps: float,
                  round_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """round_dtype (float16 / bfloat16): round the logits, the softmax and the group mean as a model of that
    dtype does in the reference (kvquant/scorer.py:309-315, 403); None: fp32 throughout."""
    keys, values = _kv_operands(keys, values)
    H, T, D = keys.shape
    dev = keys.device
    scores = torch.empty(H, T, dtype=torch.float32, device=dev)
    ws_bytes = lib.odmkv_score_workspace_bytes(H, n_q_heads, T)
    ws = _lib.workspace(dev, ws_bytes, "score")
    mu32 = None if mu is None else mu.reshape(n_q_heads, D).float().contiguous()
    a32 = None if attn is None else attn.float().contiguous()
    rd = -1 if round_dtype is None else {torch.float16: 0, torch.bfloat16: 1}[round_dtype]
    _lib.check(lib.odmkv_score_model_dtype(
        keys.data_ptr(), values.data_ptr(), _lib.dtype_code(keys), H, T, keys.stride(0), keys.stride(1),
        _lib.ptr(mu32), n_q_heads, _lib.ptr(a32), n_sink, float(eps), rd, scores.data_ptr(),
        ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev)))
    return scores


class RiskScorer(ExpectedAttentionScorer):
    """s = (p + eps)^2 * [ |v|^2 + (|k|^2 / d) * |v - o|^2 ]: first-order joint error of the
    attention output under independent key and value quantisation noise."""

    def __init__(self, *, model_dtype_rounding: bool = False, **kw):
        """model_dtype_rounding (not in the reference's constructor; off by default): with keys in fp16 / bf16, round
        the attention estimate where the reference's tensors have the model's dtype (logits, softmax, group mean,
        (p + eps)^2: kvquant/scorer.py:309-315, 403), so that the scores are the ones the reference computes on such a model, not
        the fp32 ones."""
        kw["use_covariance"] = False
        super().__init__(**kw)
        self.model_dtype_rounding = bool(model_dtype_rounding)

    def score_prefill(self, keys, values, layer_idx, *, module=None, hidden_states=None):
        if module is None or hidden_states is None:
            return self._fallback.score_prefill(keys, values, layer_idx)
        if keys.shape[1] <= self.n_sink:
            return torch.ones(keys.shape[:2], device=keys.device, dtype=keys.dtype)
        if hidden_states.dim() == 2:
            hidden_states = hidden_states.unsqueeze(0)
        try:
            mu, _ = self._query_statistics(module, hidden_states)
        except (AttributeError, NotImplementedError, ValueError):
            return self._fallback.score_prefill(keys, values, layer_idx)
        n_q = mu.shape[1]
        rd = keys.dtype if self.model_dtype_rounding and keys.dtype in (torch.float16, torch.bfloat16) else None
        scores = _launch_score(keys, values, mu[0], None, n_q, self.n_sink, self.epsilon, round_dtype=rd)
        return self._maybe_normalize(scores)

    def score_with_attn(self, keys, values, attn_weights, *, module=None):
        H = keys.shape[0]
        return _launch_score(keys, values, None, attn_weights, H, 0, self.epsilon)


def _launch_window_attention(keys: torch.Tensor, queries: torch.Tensor, n_sink: int, q_pos0: int,
                             scaling: float) -> torch.Tensor:
    """p fp32 [Hkv, T - n_sink]: attention mass of the window queries [Hq, W, d] (rotated to positions
    q_pos0 .. q_pos0 + W - 1) over the core keys, per-query causal softmax, mean over queries and group."""
    _lib.require_gpu(keys, "keys")
    if keys.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"window attention runs on the 16-bit matrix cores: keys must be float16 or bfloat16, got {keys.dtype}")
    if keys.shape[-1] != _lib.HEAD_DIM:
        raise ValueError(f"the HIP kernels are written for head_dim {_lib.HEAD_DIM}, got {keys.shape[-1]}")
    if keys.stride(-1) != 1 or keys.stride(0) % 8 or keys.stride(1) % 8 or keys.data_ptr() % 16:
        keys = keys.contiguous()
    H, T, D = keys.shape
    Hq, W, _ = queries.shape
    q = queries.to(keys.dtype).contiguous()
    dev = keys.device
    p = torch.empty(H, T - n_sink, dtype=torch.float32, device=dev)
    ws_bytes = lib.odmkv_window_attention_workspace_bytes(H, Hq, W, T)
    ws = _lib.workspace(dev, ws_bytes, "window")
    _lib.check(lib.odmkv_window_attention(
        keys.data_ptr(), _lib.dtype_code(keys), H, T, keys.stride(0), keys.stride(1), q.data_ptr(), Hq, W,
        int(q_pos0), int(n_sink), float(scaling), p.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev)))
    return p


class WindowRiskScorer(RiskScorer):
    """The risk score with the attention estimate taken from the prompt's last `window` queries, each
    with its own causal softmax, instead of from the one mean query (not in the reference; opt-in).

        p_j = mean over window queries and GQA group of softmax_j(q . k_j / sqrt(d)),   s_j as in RiskScorer

    The queries are the module's own (q_proj / q_norm, RoPE at their positions); keys must be 16-bit."""

    def __init__(self, *, window: int = 64, **kw):
        super().__init__(**kw)
        if window < 1:
            raise ValueError("window must be at least 1")
        self.window = int(window)

    def _window_queries(self, module: nn.Module, hidden_states: torch.Tensor, w: int) -> torch.Tensor:
        q_len = hidden_states.shape[1]
        q = _get_query_states(module, hidden_states[:, q_len - w:])              # [1, Hq, w, d], pre-RoPE
        rotary_emb = getattr(module, "rotary_emb", None)
        if rotary_emb is not None:
            pos = torch.arange(q_len - w, q_len, device=q.device).unsqueeze(0)
            cos, sin = _aligned_rotary_outputs(rotary_emb, q, pos)
            q = _apply_rotary_pos_emb_q(q, cos, sin)
        return q[0]

    def score_prefill(self, keys, values, layer_idx, *, module=None, hidden_states=None):
        if module is None or hidden_states is None:
            return self._fallback.score_prefill(keys, values, layer_idx)
        if keys.shape[1] <= self.n_sink:
            return torch.ones(keys.shape[:2], device=keys.device, dtype=keys.dtype)
        if hidden_states.dim() == 2:
            hidden_states = hidden_states.unsqueeze(0)
        H, T, D = keys.shape
        w = min(self.window, T - self.n_sink, hidden_states.shape[1])
        try:
            queries = self._window_queries(module, hidden_states, w)
        except (AttributeError, NotImplementedError):
            return self._fallback.score_prefill(keys, values, layer_idx)
        p = _launch_window_attention(keys, queries, self.n_sink, T - w, D ** -0.5)
        core = _launch_score(keys[:, self.n_sink:], values[:, self.n_sink:], None, p, H, 0, self.epsilon)
        top = core.max().reshape(1, 1).expand(H, self.n_sink)
        return self._maybe_normalize(torch.cat([top, core], dim=1))
