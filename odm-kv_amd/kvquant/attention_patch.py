"""Attention-function patch: fused packed-cache decode, and head-wise masking for the dense path.

Stands where the reference's kvquant/attention_patch.py:13-62 stands.  Two behaviours:

* decode (one query token) on a module whose layer has a packed store attached
  (``module._odmkv_state``): the attention output comes from the fused LUT kernel over the packed
  cache (``TurboQuantAdaptiveKVCacheState.decode_attention``); the dense ``key``/``value`` tensors
  handed in by the model are not read, except for the newest token, which the store does not hold
  yet when the attention function runs (the press appends it in its forward hook, afterwards).
  Evicted tokens are absent from the store, so no fake keys are needed.
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


def _fused_decode(module, query, key, value, attention_mask, dropout, kwargs):
    """Attention output [B, 1, Hq, D] from the packed store, or None when this call is not a plain
    single-token decode over a store that is in step with the dense cache."""
    state = getattr(module, "_odmkv_state", None)
    if state is None or not fused_decode_enabled():
        return None
    if query.shape[2] != 1 or attention_mask is not None or dropout:
        return None
    if kwargs.get("sliding_window") is not None or kwargs.get("softcap") is not None or kwargs.get("s_aux") is not None:
        return None
    k_len = key.shape[2]
    if state.seq_len not in (k_len - 1, k_len) or state.batch_size != query.shape[0]:
        return None
    scaling = kwargs.get("scaling")
    if scaling is None:
        scaling = query.shape[-1] ** -0.5
    B, Hq, _, D = query.shape
    if state.seq_len == k_len - 1 and getattr(state, "exact_decode_append", False):
        # the press keeps new tokens exact until its buffer flushes: store the token now, the
        # press's hook sees the store already in step and does not append it again
        state.append_all_exact(key[:, :, -1:, :], value[:, :, -1:, :])
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


def _attention_patch(func):
    if getattr(func, _PATCH_ATTR, False):
        return func

    @functools.wraps(func)
    def wrapper(module, query, key, value, attention_mask, dropout=0.0, **kwargs):
        if query.shape[2] == key.shape[2]:
            module.masked_key_indices = None
            module._odmkv_state = None
        else:
            if query.shape[2] == 1:
                # the newest token's query, after RoPE: the press's flush scores its buffer with it and need not
                # project and rotate the hidden state a second time
                module._odmkv_last_query = query
            fused = _fused_decode(module, query, key, value, attention_mask, dropout, kwargs)
            if fused is not None:
                call_counts["fused"] += 1
                return fused, None
            if key.dim() == 4 and key.shape[2] > 1 and key.stride(2) == 0:
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
    for name, func in list(ALL_ATTENTION_FUNCTIONS.items()):
        if getattr(func, _PATCH_ATTR, False):
            continue
        ALL_ATTENTION_FUNCTIONS[name] = _attention_patch(func)
