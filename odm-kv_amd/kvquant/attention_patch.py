"""Attention-function patch: fused packed-cache decode, and head-wise masking for the dense path.

Stands where the reference's kvquant/attention_patch.py:13-62 stands.  Two behaviours:

* decode (one query token, or a block of new tokens such as the question after a prefill) on a module
  whose layer has a packed store attached (``module._odmkv_state``): the attention output comes from
  the fused LUT kernel over the packed cache (``TurboQuantAdaptiveKVCacheState.decode_attention`` /
  ``decode_attention_block``); the dense ``key``/``value`` tensors handed in by the model are not read,
  except for the new tokens, which the store does not hold yet when the attention function runs (the
  press appends them in its forward hook, afterwards).  Evicted tokens are absent from the store, so
  no fake keys are needed.
* everything else goes to the wrapped attention function as in the reference, with evicted keys
  replaced by a fake key whose weight underflows to zero (``search_hyperplane``).
"""
from __future__ import annotations

import functools
import os

import torch
from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

_PATCH_ATTR = "_kvtoken_quant_attention_patched"
# how many decode calls took the fused kernel / the wrapped attention function (diagnostics)
call_counts = {"fused": 0, "dense": 0}


def search_hyperplane(x: torch.Tensor, max_iter: int = 1000) -> torch.Tensor:
    """A key y with <q, y> << 0 for every query q in x [n, m, d]: returns -1e5 * y / |y|^2 where y
    has a positive inner product with all rows (perceptron-style updates from the mean)."""
    dtype = x.dtype
    x = x.float()
    y = x.mean(dim=1)
    for _ in range(max_iter):
        wrong = torch.bmm(x, y.unsqueeze(-1)) <= 0
        if not wrong.any():
            return (-1e5 * y / y.norm(dim=-1, keepdim=True) ** 2).to(dtype)
        y = y + (x * wrong).sum(dim=1) / wrong.sum(dim=1).clamp(min=1)
    raise ValueError("Could not find fake keys such that exp(<q, k>) ~= 0")


def fused_decode_enabled() -> bool:
    return os.environ.get("ODMKV_FUSED_DECODE", "1") != "0"


_causal_checked: dict = {}


def _store_part_is_open(attention_mask: torch.Tensor, store_len: int) -> bool:
    """True when the boolean / additive mask of a multi-token step lets every query see every stored token (what a
    causal mask without padding does).  The same mask object goes to every layer of a forward: checked once."""
    hit = _causal_checked.get("last")
    if hit is not None and hit[0] is attention_mask and hit[1] == store_len:      # (the entry keeps the tensor alive)
        return hit[2]
    part = attention_mask[..., :store_len]
    ok = bool(part.all()) if attention_mask.dtype == torch.bool else bool((part == 0).all())
    _causal_checked["last"] = (attention_mask, store_len, ok)
    return ok


def _fused_decode(module, query, key, value, attention_mask, dropout, kwargs):
    """Attention output [B, L, Hq, D] from the packed store, or None when this call is not a decode step (one token, or
    a block of tokens that all see the whole store) over a store that is in step with the dense cache."""
    state = getattr(module, "_odmkv_state", None)
    if state is None or not fused_decode_enabled():
        return None
    B, Hq, L, D = query.shape
    if dropout or (L == 1 and attention_mask is not None):
        return None
    if kwargs.get("sliding_window") is not None or kwargs.get("softcap") is not None or kwargs.get("s_aux") is not None:
        return None
    # a cache layer without a dense copy hands over the new tokens only, tagged with the store's length
    store_len = getattr(key, "_odmkv_store_len", None)
    k_len = key.shape[2] if store_len is None else store_len + key.shape[2]
    if state.batch_size != B:
        return None
    scaling = kwargs.get("scaling")
    if scaling is None:
        scaling = D ** -0.5
    if L > 1:
        return _fused_block(state, query, key, value, attention_mask, scaling, k_len)
    if state.seq_len not in (k_len - 1, k_len):
        return None
    if state.seq_len == k_len - 1 and getattr(state, "exact_decode_append", False):
        # the press keeps new tokens exact until its buffer flushes: store the token now (the press's hook sees
        # the store already in step and does not append it again) and attend, in one library call
        return state.decode_step(query, key[:, :, -1:, :], value[:, :, -1:, :], scaling=scaling,
                                 out_dtype=query.dtype).view(B, 1, Hq, D)
    if state.seq_len == k_len:
        return state.decode_attention(query, scaling=scaling, out_dtype=query.dtype).view(B, 1, Hq, D)
    else:
        # merge the newest (still dense) token with the store's partial result by log-sum-exp
        out, lse = state.decode_attention(query, scaling=scaling, return_lse=True)
        G = Hq // key.shape[1]
        k_new = key[:, :, -1, :].float().repeat_interleave(G, dim=1)
        v_new = value[:, :, -1, :].float().repeat_interleave(G, dim=1)
        q16 = query[:, :, 0, :].float()
        l_new = (q16 * k_new).sum(-1) * scaling
        m = torch.maximum(lse, l_new)
        w_old, w_new = torch.exp(lse - m), torch.exp(l_new - m)
        out = (out * w_old.unsqueeze(-1) + v_new * w_new.unsqueeze(-1)) / (w_old + w_new).unsqueeze(-1)
    return out.to(query.dtype).view(B, 1, Hq, D)


def _fused_block(state, query, key, value, attention_mask, scaling, k_len):
    """A block of L new tokens after the prefill (the reference runner feeds every question this way,
    benchmark/core/pipeline.py:170-185; the reference's wrapper treats any q_len != k_len alike,
    attention_patch.py:38-48): every new token sees the whole store, through the fused kernel, and the new tokens at or
    before its own position, through a small dense product over the L tokens the model handed over; the two parts
    are merged by their log-sum-exps.  The store must not hold the new tokens yet (the press appends them in its
    hook, afterwards), and the mask, if there is one, must leave the stored tokens open."""
    B, Hq, L, D = query.shape
    if state.seq_len != k_len - L:
        return None
    if attention_mask is not None:
        if attention_mask.dim() != 4 or attention_mask.shape[-2] != L or attention_mask.shape[-1] != k_len:
            return None
        if not _store_part_is_open(attention_mask, k_len - L):
            return None
    out_s, lse_s = state.decode_attention_block(query, scaling=scaling)          # [B, Hq, L, D], [B, Hq, L]
    G = Hq // key.shape[1]
    k_new = key[:, :, -L:, :].float().repeat_interleave(G, dim=1)                # [B, Hq, L, D]
    v_new = value[:, :, -L:, :].float().repeat_interleave(G, dim=1)
    logits = torch.matmul(query.float(), k_new.transpose(-1, -2)) * scaling      # [B, Hq, L, L]
    if attention_mask is None:
        keep = torch.ones(L, L, dtype=torch.bool, device=query.device).tril()
        logits = logits.masked_fill(~keep, float("-inf"))
    elif attention_mask.dtype == torch.bool:
        logits = logits.masked_fill(~attention_mask[..., -L:], float("-inf"))
    else:
        logits = logits + attention_mask[..., -L:].float()
    lse_n = torch.logsumexp(logits, dim=-1)                                      # every token sees itself: finite
    out_n = torch.matmul(torch.exp(logits - lse_n.unsqueeze(-1)), v_new)
    m = torch.maximum(lse_s, lse_n)
    w_s, w_n = torch.exp(lse_s - m).unsqueeze(-1), torch.exp(lse_n - m).unsqueeze(-1)
    out = (out_s * w_s + out_n * w_n) / (w_s + w_n)
    return out.to(query.dtype).transpose(1, 2).contiguous()                      # [B, L, Hq, D]


def _attention_patch(func):
    if getattr(func, _PATCH_ATTR, False):
        return func

    @functools.wraps(func)
    def wrapper(module, query, key, value, attention_mask, dropout=0.0, **kwargs):
        if query.shape[2] == key.shape[2] and not hasattr(key, "_odmkv_store_len"):      # a prefill (no cached tokens)
            module.masked_key_indices = None
            module._odmkv_state = None
        else:
            if query.shape[2] == 1:
                # the newest token's query, after RoPE: the press's flush scores its buffer with it and need not
                # project and rotate the hidden state a second time
                object.__setattr__(module, "_odmkv_last_query", query)         # (past nn.Module's slower __setattr__)
            fused = _fused_decode(module, query, key, value, attention_mask, dropout, kwargs)
            if fused is not None:
                call_counts["fused"] += 1
                return fused, None
            if (key.dim() == 4 and key.shape[2] > 1 and key.stride(2) == 0) or hasattr(key, "_odmkv_store_len"):
                raise RuntimeError(
                    "this layer's dense cache was released (release_dense_cache=True) and the call cannot take the "
                    "fused decode path (padding mask, dropout, sliding window, soft cap or a batch the store was "
                    "not built for): keep the dense cache for such calls")
            call_counts["dense"] += 1
            if getattr(module, "masked_key_indices", None) is not None:
                bsz, num_heads, seq_len, head_dim = query.shape
                n_kv = key.shape[1]
                q = query.view(bsz, n_kv, num_heads // n_kv, seq_len, head_dim)
                q = q.reshape(bsz * n_kv, (num_heads // n_kv) * seq_len, head_dim)
                fake_keys = search_hyperplane(q).view(bsz, n_kv, head_dim)
                b_idx, h_idx, s_idx = module.masked_key_indices
                key[b_idx, h_idx, s_idx] = fake_keys[b_idx, h_idx]
        if "cu_seq_lens_k" in kwargs:
            kwargs["cu_seq_lens_k"][-1] = key.shape[-2]
        return func(module, query, key, value, attention_mask, dropout, **kwargs)

    setattr(wrapper, _PATCH_ATTR, True)
    return wrapper


def patch_attention_functions() -> None:
    """Wrap every registered attention function once (a wrapped one is recognised by its mark and left alone)."""
    for name in list(ALL_ATTENTION_FUNCTIONS.keys()):
        ALL_ATTENTION_FUNCTIONS[name] = _attention_patch(ALL_ATTENTION_FUNCTIONS[name])
