"""TurboQuantPerTokenBackendPress: the ODM-KV press that keeps the packed mixed-precision cache.

Host-side mirror of the reference class (kvquant/adaptive_backend_press.py:22-682): same
constructor, hook protocol, prefill finalisation (:292-325), decode buffering (:383-458), flush
(:464-595), flush attention (:601-665) and cached-ratio allocation (:198-290).  Differences that
follow from running on the packed store:

* decode attention is computed by the fused LUT kernel over the store (see attention_patch.py),
  not by the HF attention function over a re-materialised cache; the HF cache tensors are still
  kept in step (quantised positions overwritten in place) so the dense path remains usable;
* layer-wise allocation of all layers runs as one batched allocator launch;
* flush scoring handles all kv-heads of a sequence in one launch instead of a loop per head, and
  the cached-ratio allocation ranks all heads with one sort;
* ``release_dense_cache=True`` (a constructor argument the reference does not have) swaps each
  packed layer of the model's cache for one that keeps no dense copy (hf_cache.py).
"""
from __future__ import annotations

import contextlib
import math
from typing import Optional

import torch
from torch import nn

from kvquant import _lib
from kvquant.allocator import optimal_scores_to_bits, ratio_scores_to_bits, scores_to_bits
from kvquant.attention_patch import fused_decode_enabled
from kvquant.attention_utils import _aligned_rotary_outputs, _apply_rotary_pos_emb_q, _get_query_states
from kvquant.hf_cache import PackedCacheLayer
from kvquant.press import TurboQuantPerTokenPress, full_attention_modules
from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState, release_staging, reserve_state_memory


def _levels_by_rank(levels, ratios, n: int):
    """Level of the token of every rank 0..n-1 (ascending score) under `ratio_scores_to_bits`'
    tier sizes: round(share * n) tokens per tier from the lowest level up, the last tier takes the rest."""
    import numpy as np
    share = torch.tensor(ratios, dtype=torch.float64)
    share = (share / share.sum()).tolist()
    tiers = sorted(zip(levels, share), key=lambda t: t[0])
    out = np.empty(n, np.int32)
    cursor = 0
    for i, (b, frac) in enumerate(tiers):
        count = n - cursor if i == len(tiers) - 1 else min(int(round(frac * n)), n - cursor)
        out[cursor:cursor + count] = b
        cursor += count
    return out


class TurboQuantPerTokenBackendPress(TurboQuantPerTokenPress):
    def __init__(self, *, value_group_size: int = 32, key_quantizer: str = "prod", value_quantizer: str = "minmax",
                 scorer=None, bit_levels: tuple[int, ...] = (0, 2, 4, 8, 16), ratios: Optional[tuple[float, ...]] = None,
                 target_avg_bits: Optional[float] = None, eviction_cost: float = 5.0, above_target_alpha: float = 1.0,
                 n_outlier_channels: int = 0, outlier_min_bits: int = 4, seed: int = 42, decode_quant: bool = True,
                 sink_tokens: int = 0, layerwise: bool = False, buffer_size: int = 128, initial_layers_fp16: int = 0,
                 allow_decode_eviction: bool = False, release_dense_cache: bool = False):
        min_bits = 2 if key_quantizer in ("prod", "turboquant_prod", "turboquantprod") else 1
        invalid = [b for b in bit_levels if b not in (0, 16) and b < min_bits]
        if invalid:
            raise ValueError(f"TurboQuantPerTokenBackendPress does not support key bit-levels below "
                             f"{min_bits} with key_quantizer={key_quantizer!r}: {invalid}")
        super().__init__(scorer=scorer, bit_levels=bit_levels, ratios=ratios, target_avg_bits=target_avg_bits,
                         eviction_cost=eviction_cost, above_target_alpha=above_target_alpha,
                         n_outlier_channels=n_outlier_channels, outlier_min_bits=outlier_min_bits, seed=seed,
                         decode_quant=decode_quant, sink_tokens=sink_tokens, layerwise=layerwise,
                         quantizer="turboquant", value_quantizer=value_quantizer,
                         value_group_size=value_group_size, allow_decode_eviction=allow_decode_eviction)
        self.key_quantizer = key_quantizer
        self.buffer_size = buffer_size
        self.initial_layers_fp16 = initial_layers_fp16
        # not in the reference: once a layer's prefill is packed, swap its cache layer for one that
        # keeps no dense copy (kvquant/hf_cache.py); decode then needs the fused attention path
        if release_dense_cache and not decode_quant:
            raise ValueError("release_dense_cache needs decode_quant=True: new tokens must reach the packed store")
        self.release_dense_cache = bool(release_dense_cache)
        self._states: dict[int, TurboQuantAdaptiveKVCacheState] = {}
        self._buffer_counts: dict[int, int] = {}
        self._buffer_start_seqs: dict[int, int] = {}
        # (layer, head) -> ((level, fraction), ...) observed in the prefill allocation
        self._observed_ratios: dict[tuple[int, int], tuple[tuple[int, float], ...]] = {}

    def _build_tables(self, model) -> None:
        return          # the state builds its rotations and tables when it is created

    def _get_or_create_state(self, layer_idx: int, keys: torch.Tensor) -> TurboQuantAdaptiveKVCacheState:
        state = self._states.get(layer_idx)
        if state is not None:
            return state
        levels = self.bit_levels
        if self.buffer_size > 0 and 16 not in levels:
            levels = tuple(sorted(set(levels) | {16}))
        state = TurboQuantAdaptiveKVCacheState(
            head_dim=keys.shape[-1], bit_levels=levels, key_quantizer=self.key_quantizer,
            value_quantizer=self.value_quantizer, value_group_size=self.value_group_size,
            device=keys.device, dtype=keys.dtype, seed=self.seed + layer_idx * 7,
            outlier_min_bits=self.outlier_min_bits, quant_headroom=self.buffer_size > 0 and self.decode_quant)
        state.exact_decode_append = self.buffer_size > 0 and self.decode_quant
        self._states[layer_idx] = state
        return state

    @staticmethod
    def _packed_layer(cache, layer_idx: int) -> Optional[PackedCacheLayer]:
        layers = getattr(cache, "layers", None)
        if layers is not None and layer_idx < len(layers) and isinstance(layers[layer_idx], PackedCacheLayer):
            return layers[layer_idx]
        return None

    def _release_dense(self, cache, layer_idx: int, state) -> None:
        """Swap the layer's dense tensors for aliased views of its last token."""
        if not self.release_dense_cache or layer_idx < self.initial_layers_fp16:
            return
        if not hasattr(cache, "layers") or self._packed_layer(cache, layer_idx) is not None:
            return
        if not fused_decode_enabled():
            raise RuntimeError("release_dense_cache needs the fused decode path (ODMKV_FUSED_DECODE=0 is set)")
        keys, values = self._get_cache_tensors(cache, layer_idx)
        cache.layers[layer_idx] = PackedCacheLayer(state, keys, values)

    def _attach(self, cache, layer_idx: int, module: nn.Module, state) -> None:
        # plain attributes, set past nn.Module's own __setattr__ (its checks for parameters, buffers and submodules cost
        # more than the rest of the hook on a decode step)
        object.__setattr__(module, "masked_key_indices", state.masked_key_indices())
        object.__setattr__(module, "_odmkv_state", state)
        if hasattr(cache, "layers"):
            cache.layers[layer_idx]._tq_backend_state = state

    @staticmethod
    def _attached(cache, layer_idx: int, module: nn.Module, state) -> bool:
        """Whether _attach(state) has run for this module and cache layer (an exact append changes nothing it sets)."""
        if module.__dict__.get("_odmkv_state") is not state:
            return False
        layers = getattr(cache, "layers", None)
        return layers is None or getattr(layers[layer_idx], "_tq_backend_state", None) is state

    def _sync_cache_from_state(self, cache, layer_idx: int, module: nn.Module, state, *, prefill_fast: bool = False,
                               start: int = 0) -> None:
        """`start`: only positions >= start have changed in the store (a flush re-stores the buffered tokens)."""
        if self._packed_layer(cache, layer_idx) is not None:
            self._attach(cache, layer_idx, module, state)            # no dense copy to bring up to date
            return
        if prefill_fast:
            keys, values = self._get_cache_tensors(cache, layer_idx)
            state.materialize_quantized_into(keys, values, start=start)
        else:
            keys, values = state.materialize()
            self._set_cache_tensors(cache, layer_idx, keys, values)
        self._attach(cache, layer_idx, module, state)

    # ------------------------------------------------------------------ cached ratios
    def _record_observed_ratios(self, layer_idx: int, bits: torch.Tensor) -> None:
        """Level fractions per kv-head over the bulk of the prefill (sinks and the protected tail
        left out), taken before the window override."""
        if bits.dim() != 3 or bits.shape[-1] == 0:
            return
        B, H, T = bits.shape
        start = min(int(self.sink_tokens), T) if self.sink_tokens > 0 else 0
        end = T - min(int(self.buffer_size), T) if self.buffer_size > 0 else T
        if end <= start:
            start, end = 0, T
        bulk = bits[..., start:end].reshape(B * H, end - start)
        levels = sorted(set(int(b) for b in self.bit_levels) | {16})
        lv = torch.tensor(levels, device=bits.device, dtype=bits.dtype)
        counts = (bulk.unsqueeze(-1) == lv).sum(dim=1).cpu()                 # [B*H, K], one transfer
        for row in range(B * H):
            c = counts[row]
            total = int(c.sum())
            if total == 0:
                continue
            fracs = (c.float() / total).tolist()
            self._observed_ratios[(layer_idx, row % H)] = tuple(
                (b, f) for b, f, n in zip(levels, fracs, c.tolist()) if n > 0)

    def _allocate_bits_via_cached_ratios(self, scores, positions, num_heads, layer_idx, allowed_levels,
                                         batch_size: Optional[int] = None):
        """Rank tiers per kv-head with the level shares seen at prefill.  With `batch_size` the
        caller states that the tokens come ordered (batch, head, position) with the same count in
        every (batch, head): all heads are then ranked by one sort instead of a loop of sorts."""
        if not all((layer_idx, h) in self._observed_ratios for h in range(num_heads)):
            return None
        tiers = []
        for h in range(num_heads):
            kept = [(b, r) for b, r in self._observed_ratios[(layer_idx, h)] if b in allowed_levels and r > 0]
            if not kept:
                return None
            total = sum(r for _, r in kept)
            tiers.append(tuple(zip(*[(b, r / total) for b, r in kept])))
        n_tok = scores.shape[0]
        if batch_size is not None and n_tok > 0 and n_tok % (batch_size * num_heads) == 0:
            B, H, n = int(batch_size), int(num_heads), n_tok // (batch_size * num_heads)
            rows = scores.reshape(B, H, n).permute(1, 0, 2).reshape(H, B * n)       # one row per head
            order = torch.argsort(rows, dim=1, stable=True)
            by_rank = torch.empty(H, B * n, dtype=torch.int32)
            for h, (levels, ratios) in enumerate(tiers):
                by_rank[h] = torch.from_numpy(_levels_by_rank(levels, ratios, B * n))
            out = torch.empty(H, B * n, dtype=torch.int32, device=scores.device)
            out.scatter_(1, order, by_rank.to(scores.device, non_blocking=True))
            return out.reshape(H, B, n).permute(1, 0, 2).reshape(-1)
        bits = torch.empty_like(scores, dtype=torch.int32)
        head_indices = positions[:, 1]
        for h in range(num_heads):
            levels, ratios = tiers[h]
            mask = head_indices == h
            if not mask.any():
                continue
            bits[mask] = ratio_scores_to_bits(scores[mask], tuple(levels), tuple(ratios)).to(torch.int32)
        return bits

    # ------------------------------------------------------------------ prefill
    def _finalize_each_layer(self) -> bool:
        # with the dense copy released there is a reason not to wait for the last layer: each layer's
        # fp16 keys and values are freed while the prefill of the layers above it is still running
        return self.layerwise and self.release_dense_cache

    def _finalize_prefill(self, cache) -> None:
        if self.n_outlier_channels > 0:
            raise NotImplementedError("outlier-channel separation is not built (n_outlier_channels must be 0)")
        for layer_idx, bits in self._allocate_bits_for_prefill().items():
            keys, values = self._get_cache_tensors(cache, layer_idx)
            self._record_observed_ratios(layer_idx, bits)
            if layer_idx < self.initial_layers_fp16:
                bits = torch.full_like(bits, 16)
            elif self.buffer_size > 0:
                bits = bits.clone()
                bits[..., -min(self.buffer_size, bits.shape[-1]):] = 16
            state = self._get_or_create_state(layer_idx, keys)
            state.prefill(keys, values, bits.to(dtype=torch.int32, device=keys.device))
            module = self._layer_modules.get(layer_idx)
            if module is not None:
                if self.release_dense_cache and layer_idx >= self.initial_layers_fp16:
                    self._release_dense(cache, layer_idx, state)
                self._sync_cache_from_state(cache, layer_idx, module, state, prefill_fast=True)
            if self.buffer_size > 0:
                self._buffer_start_seqs[layer_idx] = int(keys.shape[2])
                self._buffer_counts[layer_idx] = 0
            if self._last_hooked_layer_idx is None or layer_idx == self._last_hooked_layer_idx:
                release_staging(keys.device)             # the prompt is stored: the worst-case staging store can go
        self._reset_prefill_state()

    # ------------------------------------------------------------------ hook
    def _forward_hook(self, module: nn.Module, args, kwargs, output):
        cache, hidden_states = self._hook_inputs(module, args, kwargs)
        if cache is None or hidden_states is None:
            return output
        layer_idx = int(module.layer_idx)
        self._layer_modules[layer_idx] = module
        keys, values = self._get_cache_tensors(cache, layer_idx)
        if self._head_dim is None:
            self._head_dim = keys.shape[-1]
        q_len, cache_len = hidden_states.shape[1], keys.shape[2]
        if cache_len == q_len:
            self._prefill_hook(module, cache, hidden_states, layer_idx, keys, values)
            return output
        if not self.decode_quant or layer_idx < self.initial_layers_fp16:
            return output

        state = self._get_or_create_state(layer_idx, keys)
        if self.buffer_size > 0:
            buf_start = self._buffer_start_seqs.get(layer_idx)
            if buf_start is not None and buf_start > state.seq_len:        # the cache was trimmed
                self._buffer_start_seqs[layer_idx] = state.seq_len
                self._buffer_counts[layer_idx] = 0

        already_stored = state.seq_len == cache_len       # the fused attention path stored the token
        if already_stored and q_len == 1 and self.buffer_size > 0:
            # the usual decode step: nothing to store, the buffer grows by one token
            count = self._buffer_counts.get(layer_idx, 0) + 1
            self._buffer_counts[layer_idx] = count
            if count >= self.buffer_size:
                self._flush_decode_buffer(state, layer_idx, cache, module, hidden_states)
            elif not self._attached(cache, layer_idx, module, state):
                self._attach(cache, layer_idx, module, state)
            return output
        packed_layer = self._packed_layer(cache, layer_idx)
        if packed_layer is not None:
            new_k, new_v = packed_layer.recent            # the layer's tensors alias one token
        else:
            new_k = keys[:, :, -q_len:, :]
            new_v = values[:, :, -q_len:, :]
        if self.buffer_size > 0:
            if not already_stored:
                state.append_all_exact(new_k, new_v)
            if q_len > 1:
                # a multi-token call after the prefill is prompt text (e.g. the question): it stays
                # exact and out of reach of the flush
                self._buffer_start_seqs[layer_idx] = state.seq_len
                self._attach(cache, layer_idx, module, state)
                return output
            self._buffer_counts[layer_idx] = self._buffer_counts.get(layer_idx, 0) + q_len
            if self._buffer_counts[layer_idx] >= self.buffer_size:
                self._flush_decode_buffer(state, layer_idx, cache, module, hidden_states)
                return output
            self._attach(cache, layer_idx, module, state)
            return output

        batch_bits = []
        for b in range(keys.shape[0]):
            h_batch = hidden_states[b:b + 1]
            if q_len == 1:
                scores = self._score_decode(new_k[b, :, 0, :], new_v[b, :, 0, :], layer_idx, module=module,
                                            hidden_states=h_batch).unsqueeze(-1)
            else:
                scores = self._score_prefill(new_k[b], new_v[b], layer_idx, module=module, hidden_states=h_batch)
            batch_bits.append(scores_to_bits(scores, self._decode_bit_levels))
        bits = torch.stack(batch_bits, dim=0).to(dtype=torch.int32, device=keys.device)
        state.append(new_k, new_v, bits)
        self._sync_cache_from_state(cache, layer_idx, module, state, prefill_fast=True)
        return output

    # ------------------------------------------------------------------ flush
    def _flush_decode_buffer(self, state, layer_idx: int, cache, module: nn.Module,
                             hidden_states: Optional[torch.Tensor] = None) -> None:
        """Score the buffered (exact) decode tokens with the current query and re-store them at the
        levels the budget gives them."""
        buffer_start = self._buffer_start_seqs.get(layer_idx)
        if buffer_start is None:
            self._sync_cache_from_state(cache, layer_idx, module, state, prefill_fast=True)
            return
        if self._flush_on_device(state, layer_idx, cache, module, hidden_states, int(buffer_start)):
            return
        positions, buf_keys, buf_values = state.get_buffer_tokens(buffer_start)
        if positions.shape[0] == 0:
            self._buffer_start_seqs[layer_idx] = state.seq_len
            self._buffer_counts[layer_idx] = 0
            self._sync_cache_from_state(cache, layer_idx, module, state, prefill_fast=True)
            return

        attn = self._flush_attention(module, hidden_states, buf_keys, positions, state)
        if attn is not None and self.scorer is not None:
            # tokens are ordered (batch, head, position) with the same count in every (batch, head)
            B, H = state.batch_size, state.num_heads
            n_buf = positions.shape[0] // (B * H)
            scores = torch.empty_like(attn, dtype=torch.float32)
            kb = buf_keys.reshape(B, H, n_buf, -1)
            vb = buf_values.reshape(B, H, n_buf, -1)
            ab = attn.reshape(B, H, n_buf)
            for b in range(B):
                scores.view(B, H, n_buf)[b] = self.scorer.score_with_attn(kb[b], vb[b], ab[b], module=module).float()
        elif attn is not None:
            scores = attn.pow(2) * buf_values.float().pow(2).sum(-1)
        else:
            scores = buf_keys.float().pow(2).sum(-1) + buf_values.float().pow(2).sum(-1)

        lo, hi = torch.aminmax(scores)
        spread = hi - lo                                     # stays on the device: no wait for the scores here
        scores = torch.where(spread > 1e-8, (scores - lo) / spread.clamp_min(1e-30), torch.full_like(scores, 0.5))

        levels = self._decode_bit_levels
        allowed = set(levels)
        bits = None
        if self.ratios is not None:
            pairs = [(b, r) for b, r in zip(self.bit_levels, self.ratios) if b in allowed]
            if pairs:
                flush_levels, flush_ratios = zip(*pairs)
                bits = ratio_scores_to_bits(scores, tuple(flush_levels), tuple(flush_ratios))
        elif self.target_avg_bits is not None:
            bits = self._allocate_bits_via_cached_ratios(scores, positions, state.num_heads, layer_idx, allowed,
                                                         batch_size=state.batch_size)
            if bits is None:
                eps = self._ensure_epsilon(scores.device)
                bits = optimal_scores_to_bits(
                    scores, levels, self.target_avg_bits, {b: eps.get(b, 0.0) for b in levels},
                    eviction_cost=self.eviction_cost, n_outlier=self.n_outlier_channels,
                    head_dim=self._head_dim or 128, outlier_min_bits=self.outlier_min_bits,
                    above_target_alpha=self.above_target_alpha)
        if bits is None:
            bits = scores_to_bits(scores, levels)

        state.flush_buffer(buffer_start, bits)
        self._buffer_start_seqs[layer_idx] = state.seq_len
        self._buffer_counts[layer_idx] = 0
        self._sync_cache_from_state(cache, layer_idx, module, state, prefill_fast=True, start=int(buffer_start))

    @torch.no_grad()
    def _flush_on_device(self, state, layer_idx: int, cache, module: nn.Module, hidden_states, buffer_start: int) -> bool:
        """The flush in a handful of launches and without reading anything back, where its inputs allow it: the
        budget is a target (levels by the per-head shares cached at prefill), the scorer is the risk scorer (or
        none), every head buffers the same positions and the buffer is small enough for the kernels
        (odmkv_exact_tail, odmkv_flush_score, odmkv_flush_rank).  False: nothing was done, the caller goes the
        general way (as it does when `device_flush` is set to False on the press).  With `record_flush` set on the
        press the attention weights, scores and levels of the last flush are kept in `last_flush` (for tests)."""
        from .scorer import RiskScorer
        if not getattr(self, "device_flush", True):
            return False
        if self.ratios is not None or self.target_avg_bits is None or hidden_states is None:
            return False
        if self.scorer is not None and type(self.scorer).score_with_attn is not RiskScorer.score_with_attn:
            return False
        B, H = state.batch_size, state.num_heads
        n_buf = state.seq_len - buffer_start
        if n_buf <= 0 or n_buf > 2048 or B * n_buf > 4096:
            return False
        table = self._by_rank_table(layer_idx, H, B * n_buf, state.device)
        if table is None:
            return False
        q_kv = self._flush_query(module, hidden_states, state)
        if q_kv is None:
            return False
        rows = state.exact_tail(n_buf)
        if rows is None:
            return False
        k, v = rows
        by_rank, counts = table
        dev = state.device
        q32 = q_kv.reshape(B * H, -1).float().contiguous()
        record = bool(getattr(self, "record_flush", False))
        attn = torch.empty(B * H, n_buf, dtype=torch.float32, device=dev) if record else None
        scores = torch.empty(B * H, n_buf, dtype=torch.float32, device=dev)
        minmax = torch.empty(B * H, 2, dtype=torch.float32, device=dev)
        bits = torch.empty(B, H, n_buf, dtype=torch.int32, device=dev)
        st = _lib.stream_ptr(dev)
        eps = float(self.scorer.epsilon) if self.scorer is not None else 0.0
        _lib.check(_lib.lib.odmkv_flush_score(
            k.data_ptr(), v.data_ptr(), _lib.dtype_code(k), B * H, n_buf, q32.data_ptr(), 1.0 / math.sqrt(k.shape[-1]),
            eps, 0 if self.scorer is not None else 1, _lib.ptr(attn), scores.data_ptr(), minmax.data_ptr(), st))
        _lib.check(_lib.lib.odmkv_flush_rank(scores.data_ptr(), minmax.data_ptr(), B, H, n_buf, by_rank.data_ptr(),
                                             bits.data_ptr(), st))
        if record:
            self.last_flush = {"layer": layer_idx, "start": buffer_start, "q_kv": q_kv, "keys": k, "values": v,
                               "attn": attn.reshape(B, H, n_buf), "scores": scores.reshape(B, H, n_buf), "bits": bits}
        # with one sequence the level counts of every head are those of its table: no read-back in the append
        state.flush_buffer(buffer_start, bits, rows=rows, known_counts=counts if B == 1 else None)
        self._buffer_start_seqs[layer_idx] = state.seq_len
        self._buffer_counts[layer_idx] = 0
        self._sync_cache_from_state(cache, layer_idx, module, state, prefill_fast=True, start=buffer_start)
        return True

    def _by_rank_table(self, layer_idx: int, num_heads: int, n_tok: int, device):
        """(device int32 [H, n_tok]: level of every rank per kv-head, host int64 [H, 6]: tokens per level 0, 2, 3, 4, 8,
        16) from the shares cached at prefill, as `_allocate_bits_via_cached_ratios` forms them; None when a head
        has no usable shares.  Kept per layer; the entry is keyed by the shares it was expanded from, so a press
        that sees another prompt (whose prefill overwrites the shares) never flushes with the old prompt's table."""
        import numpy as np
        allowed = set(self._decode_bit_levels)
        shares = []
        for h in range(num_heads):
            got = self._observed_ratios.get((layer_idx, h))
            kept = tuple((b, r) for b, r in (got or ()) if b in allowed and r > 0)
            if not kept:
                return None
            shares.append(kept)
        cache = self.__dict__.setdefault("_by_rank_cache", {})
        slot, key = (layer_idx, str(device)), (num_heads, n_tok, tuple(shares))
        hit = cache.get(slot)
        if hit is not None and hit[0] == key:
            return hit[1]
        rows = []
        for kept in shares:
            total = sum(r for _, r in kept)
            levels, ratios = zip(*[(b, r / total) for b, r in kept])
            rows.append(_levels_by_rank(levels, ratios, n_tok))
        by_rank = np.stack(rows)
        counts = np.stack([(by_rank == b).sum(axis=1) for b in _lib.LEVEL_ORDER], axis=1).astype(np.int64)
        cache[slot] = (key, (torch.from_numpy(by_rank).to(device), counts))      # one entry per layer: the old table goes
        return cache[slot][1]

    @torch.no_grad()
    def _flush_query(self, module: nn.Module, hidden_states, state) -> Optional[torch.Tensor]:
        """[B, H, d]: the current query at the last position (RoPE applied), averaged over each GQA group; None if
        it cannot be formed."""
        if hidden_states is None or not hasattr(module, "layer_idx"):
            return None
        H = state.num_heads
        # the attention call of this very step left the token's query (post-RoPE) on the module: what the
        # reference recomputes from the hidden state (q_proj, RoPE at the last position) is that tensor
        q = getattr(module, "_odmkv_last_query", None)
        module._odmkv_last_query = None
        if (q is not None and q.dim() == 4 and q.shape[0] == hidden_states.shape[0] == state.batch_size and q.shape[2] == 1
                and q.shape[1] % H == 0 and q.shape[3] == state.head_dim and hidden_states.shape[1] == 1):
            B, Hq, _, d = q.shape
            return q[:, :, 0, :].reshape(B, H, Hq // H, d).mean(dim=2)
        try:
            q = _get_query_states(module, hidden_states)                    # [B, Hq, q, d]
        except (AttributeError, NotImplementedError, ValueError):
            return None
        rotary_emb = getattr(module, "rotary_emb", None)
        if rotary_emb is not None:
            pos_ids = torch.arange(state.seq_len - 1, state.seq_len, device=q.device).unsqueeze(0)
            cos, sin = _aligned_rotary_outputs(rotary_emb, q, pos_ids)
            q = _apply_rotary_pos_emb_q(q, cos, sin)
        B, Hq, _, d = q.shape
        return q[:, :, -1, :].reshape(B, H, Hq // H, d).mean(dim=2)

    @torch.no_grad()
    def _flush_attention(self, module: nn.Module, hidden_states, buf_keys: torch.Tensor,
                         positions: torch.Tensor, state) -> Optional[torch.Tensor]:
        """Attention weights [N_buf] of the current query (GQA mean, RoPE at the last position) over
        the buffered keys, softmax within each (batch, head); None if the query cannot be formed."""
        q_kv = self._flush_query(module, hidden_states, state)
        if q_kv is None:
            return None
        B, H, d = q_kv.shape
        n_buf = positions.shape[0] // (B * H)
        if n_buf * B * H != positions.shape[0]:
            return None
        keys = buf_keys.reshape(B, H, n_buf, d)
        logits = (q_kv.unsqueeze(2) * keys).sum(-1) / math.sqrt(d)           # [B, H, n_buf]
        return torch.softmax(logits, dim=-1).reshape(-1)

    @contextlib.contextmanager
    def __call__(self, model):
        self._states, self._buffer_counts, self._buffer_start_seqs = {}, {}, {}
        try:
            with super().__call__(model):
                devices = [p.device for _, attn in full_attention_modules(model) for p in list(attn.parameters())[:1]]
                for device in set(devices):
                    if device.type == "cuda":
                        reserve_state_memory(device, devices.count(device))
                yield
        finally:
            self._states, self._buffer_counts, self._buffer_start_seqs = {}, {}, {}
