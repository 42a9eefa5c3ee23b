"""TurboQuantPerTokenPress: per-(layer, head, token) mixed-precision compression of an HF cache.

Host-side mirror of the reference class of the same name (kvquant/press.py:104-692): same
constructor, same hook protocol (``with press(model):``), same scoring / allocation glue
(``_build_sink_mask`` :218-224, ``_compute_bits`` :235-299, ``_allocate_bits_for_prefill``
:328-384).  Scores, allocation and quantisation run in the HIP kernels; this press writes the
quantise->dequantise result back into the HF cache in place and records evicted positions as
head-wise masks (the cache length never changes).  ``TurboQuantPerTokenBackendPress`` derives from
it and keeps the packed representation instead.
"""
from __future__ import annotations

import contextlib
import inspect
from typing import Optional

import torch
from torch import nn

from kvquant.allocator import (DEFAULT_BIT_LEVELS, calibrate_epsilon, optimal_scores_to_bits,
                               optimal_scores_to_bits_batched, ratio_scores_to_bits, scores_to_bits)
from kvquant.attention_patch import patch_attention_functions
from kvquant.scorer import BaseScorer
from kvquant.tq_backend import TurboQuantMSE, normalize_value_quantizer


def _qd_keys(kq: TurboQuantMSE, x: torch.Tensor) -> torch.Tensor:
    return kq.dequantize(kq.quantize(x))


def _qd_values_mse(vq: TurboQuantMSE, x: torch.Tensor) -> torch.Tensor:
    norms = x.norm(dim=-1, keepdim=True).clamp(min=1e-8)
    return vq.dequantize(vq.quantize(x / norms)) * norms


def _qd_scalar(x: torch.Tensor, b: int) -> torch.Tensor:
    """Per-vector asymmetric round-to-nearest quantisation, x: [N, d]."""
    n_levels = 2 ** b
    lo = x.amin(dim=-1, keepdim=True)
    scale = ((x.amax(dim=-1, keepdim=True) - lo) / (n_levels - 1)).clamp(min=1e-8)
    return ((x - lo) / scale).round().clamp(0, n_levels - 1) * scale + lo


def _qd_values_group(x: torch.Tensor, b: int, group_size: int = 32) -> torch.Tensor:
    """Per-group asymmetric min-max quantisation of values, x: [N, d]."""
    N, d = x.shape
    if d % group_size != 0 or d < group_size:
        return _qd_scalar(x, b)
    g = x.reshape(N, d // group_size, group_size)
    lo = g.min(dim=-1, keepdim=True).values
    scale = ((g.max(dim=-1, keepdim=True).values - lo) / (2 ** b - 1)).clamp(min=1e-10)
    return (((g - lo) / scale).round().clamp(0, 2 ** b - 1) * scale + lo).reshape(N, d)


def _backbone(model):
    """The module that owns the decoder layers (a causal LM wraps it once, a multimodal model twice)."""
    for name in ("model", "language_model"):
        model = getattr(model, name, model)
    return model


def full_attention_modules(model):
    """(layer index, attention module) of every decoder layer with full (not sliding-window) attention."""
    layers = getattr(_backbone(model), "layers", None)
    if layers is None:
        raise ValueError(f"Cannot find transformer layers in {type(model)}")
    found = []
    for index, layer in enumerate(layers):
        attn = getattr(layer, "self_attn", None)
        if attn is not None and not getattr(attn, "is_sliding", False):
            found.append((index, attn))
    return found


@contextlib.contextmanager
def hooked_attention(model, hook, adopt=None):
    """Every full-attention module of `model` calls `hook(module, args, kwargs, output)` after its forward for the
    duration of the block; yields the hooked layer indices.  A module without a ``layer_idx`` gets its position in
    the stack; `adopt(module)`, if given, runs once per module before its hook is registered.  Shared by all presses
    (the reference registers its hooks in each press's ``__call__``: kvquant/press.py:638-692)."""
    handles, indices = [], []
    try:
        for index, attn in full_attention_modules(model):
            if not hasattr(attn, "layer_idx"):
                attn.layer_idx = index
            if adopt is not None:
                adopt(attn)
            handles.append(attn.register_forward_hook(hook, with_kwargs=True))
            indices.append(index)
        yield indices
    finally:
        for handle in handles:
            handle.remove()


class _QuantizerPool:
    """The press's TurboQuantMSE instances, one per (role, head_dim, width, device, dtype), built on first use.
    Keys rotate with the press's seed, values with seed + 1000 (kvquant/press.py:202-212)."""
    _SEED_OFFSET = {"key": 0, "value": 1000}

    def __init__(self, seed: int):
        self._seed = seed
        self._made: dict = {}

    def get(self, role: str, head_dim: int, width: int, device, dtype) -> TurboQuantMSE:
        slot = (role, head_dim, width, device, dtype)
        q = self._made.get(slot)
        if q is None:
            q = self._made[slot] = TurboQuantMSE(head_dim, width, device=device, dtype=dtype,
                                                 seed=self._seed + self._SEED_OFFSET[role])
        return q

    def build(self, roles, head_dim: int, widths, devices, dtype) -> None:
        for role in roles:
            for width in widths:
                for device in devices:
                    self.get(role, head_dim, width, device, dtype)


class TurboQuantPerTokenPress:
    def __init__(self, scorer: Optional[BaseScorer] = None, bit_levels: tuple[int, ...] = DEFAULT_BIT_LEVELS,
                 ratios: Optional[tuple[float, ...]] = None, target_avg_bits: Optional[float] = None,
                 eviction_cost: float = 5.0, above_target_alpha: float = 1.0, n_outlier_channels: int = 0,
                 outlier_min_bits: int = 4, seed: int = 42, decode_quant: bool = False, sink_tokens: int = 0,
                 layerwise: bool = False, quantizer: str = "turboquant", value_quantizer: str = "minmax",
                 value_group_size: int = 32, allow_decode_eviction: bool = False):
        if scorer is None:
            raise ValueError("TurboQuantPerTokenPress requires an explicit scorer.")
        self.scorer, self.seed = scorer, seed
        # the budget: fixed shares per level, or an average width met by the Lagrangian allocation
        self.bit_levels, self.ratios, self.target_avg_bits = bit_levels, ratios, target_avg_bits
        self.eviction_cost, self.above_target_alpha = eviction_cost, above_target_alpha
        # the quantisers
        self.quantizer, self.value_quantizer = quantizer, normalize_value_quantizer(value_quantizer)
        self.value_group_size, self.n_outlier_channels, self.outlier_min_bits = value_group_size, n_outlier_channels, outlier_min_bits
        # what happens to which tokens
        self.sink_tokens, self.layerwise, self.decode_quant = sink_tokens, layerwise, decode_quant
        self.allow_decode_eviction = bool(allow_decode_eviction)
        kept = tuple(bit_levels) if self.allow_decode_eviction else tuple(b for b in bit_levels if b != 0)
        self._decode_bit_levels = kept or (16,)              # levels a decode-time token may get
        self._epsilon: Optional[dict[int, float]] = None     # distortion per width, calibrated on first use
        self._head_dim: Optional[int] = None
        self._quantizers = _QuantizerPool(seed)
        self._model = None
        self._prefill_hooks_fired = 0
        self._score_prefill_supports_kwargs = self._supports_kwargs(self.scorer.score_prefill)
        self._score_decode_supports_kwargs = self._supports_kwargs(self.scorer.score_decode)
        self._hooked_layer_indices: list[int] = []
        self._last_hooked_layer_idx: Optional[int] = None
        self._layer_modules: dict[int, nn.Module] = {}
        self._reset_prefill_state()

    # ------------------------------------------------------------------ scores -> bits
    def _build_sink_mask(self, H: int, T: int, device) -> Optional[torch.Tensor]:
        """[H, T] bool, True = sink token (kept at 16 bits, outside the budget)."""
        n_sink = min(self.sink_tokens, T)
        if n_sink <= 0:
            return None
        return (torch.arange(T, device=device) < n_sink).expand(H, T).contiguous()

    @staticmethod
    def _supports_kwargs(method) -> bool:
        """Whether a scorer's method takes the module and the hidden states (by name, or through **kwargs)."""
        for p in inspect.signature(method).parameters.values():
            if p.kind is inspect.Parameter.VAR_KEYWORD or p.name in ("module", "hidden_states"):
                return True
        return False

    def _ensure_epsilon(self, device) -> dict[int, float]:
        if self._epsilon is None:
            self._epsilon = calibrate_epsilon(
                self._head_dim or 128, self.bit_levels, seed=self.seed, device=device,
                value_group_size=self.value_group_size, n_outlier=self.n_outlier_channels,
                outlier_min_bits=self.outlier_min_bits, value_quantizer=self.value_quantizer)
        return self._epsilon

    def _compute_bits(self, scores: torch.Tensor, sink_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """ratios -> fixed-ratio allocation; target_avg_bits -> Lagrangian allocation; neither ->
        uniform partition (sinks forced to 16)."""
        if self.ratios is not None:
            return ratio_scores_to_bits(scores, self.bit_levels, self.ratios, sink_mask)
        if self.target_avg_bits is not None:
            return optimal_scores_to_bits(
                scores, self.bit_levels, self.target_avg_bits, self._ensure_epsilon(scores.device), sink_mask,
                eviction_cost=self.eviction_cost, n_outlier=self.n_outlier_channels,
                head_dim=self._head_dim or 128, outlier_min_bits=self.outlier_min_bits,
                above_target_alpha=self.above_target_alpha)
        bits = scores_to_bits(scores, self.bit_levels)
        if sink_mask is not None:
            bits = bits.clone()
            bits[sink_mask] = 16
        return bits

    def _reset_prefill_state(self) -> None:
        self._prefill_scores: dict[int, torch.Tensor] = {}
        self._prefill_sink_masks: dict[int, Optional[torch.Tensor]] = {}

    @staticmethod
    def _get_cache_tensors(cache, layer_idx: int):
        layers = getattr(cache, "layers", None)
        if layers is None:                                   # caches of older transformers: two lists of tensors
            return cache.key_cache[layer_idx], cache.value_cache[layer_idx]
        return layers[layer_idx].keys, layers[layer_idx].values

    @staticmethod
    def _set_cache_tensors(cache, layer_idx: int, keys: torch.Tensor, values: torch.Tensor) -> None:
        layers = getattr(cache, "layers", None)
        if layers is not None:
            layers[layer_idx].keys, layers[layer_idx].values = keys, values
        else:                                                # caches of older transformers: two lists of tensors
            cache.key_cache[layer_idx], cache.value_cache[layer_idx] = keys, values

    @staticmethod
    def _bits_to_masked_indices(bits: torch.Tensor):
        masked = (bits == 0).nonzero(as_tuple=True)
        return None if masked[0].numel() == 0 else masked

    def _batched_lagrangian_ok(self) -> bool:
        return (self.ratios is None and self.target_avg_bits is not None and self.n_outlier_channels == 0
                and self.sink_tokens >= 0)

    def _allocate_bits_for_prefill(self) -> dict[int, torch.Tensor]:
        """Bits per layer, [B, H, T] int32.  layerwise: every (layer, sequence) gets its own budget;
        otherwise one budget per sequence over all layers' tokens."""
        ordered = sorted(self._prefill_scores)
        if not ordered:
            return {}
        bits_by_layer = {l: torch.empty_like(s, dtype=torch.int32) for l, s in self._prefill_scores.items()}
        batch_size = self._prefill_scores[ordered[0]].shape[0]

        if self.layerwise and self._batched_lagrangian_ok():
            # all (layer, sequence) rows that share a shape and a device in one batched launch;
            # every row is an independent problem, so the result is that of the per-row calls
            groups: dict = {}
            for l in ordered:
                s = self._prefill_scores[l]
                groups.setdefault((tuple(s.shape), s.device), []).append(l)
            for (shape, device), layers in groups.items():
                B, H, T = shape
                rows = torch.stack([self._prefill_scores[l] for l in layers], dim=0).reshape(len(layers) * B, H * T)
                bits = optimal_scores_to_bits_batched(
                    rows.detach(), self.bit_levels, [self.target_avg_bits] * rows.shape[0],
                    self._ensure_epsilon(device), period=T, n_sink=min(max(self.sink_tokens, 0), T),
                    eviction_cost=self.eviction_cost, above_target_alpha=self.above_target_alpha)
                bits = bits.reshape(len(layers), B, H, T)
                for i, l in enumerate(layers):
                    bits_by_layer[l] = bits[i]
            return bits_by_layer

        for b in range(batch_size):
            if self.layerwise:
                for l in ordered:
                    sink = self._prefill_sink_masks[l]
                    bits_by_layer[l][b] = self._compute_bits(self._prefill_scores[l][b].detach(),
                                                             None if sink is None else sink.detach())
                continue
            target = self._prefill_scores[ordered[0]][b].device
            flat_scores, flat_sink, any_sink = [], [], False
            for l in ordered:
                s = self._prefill_scores[l][b]
                sink = self._prefill_sink_masks[l]
                flat_scores.append(s.detach().reshape(-1).to(target))
                if sink is None:
                    flat_sink.append(torch.zeros(s.numel(), dtype=torch.bool, device=target))
                else:
                    any_sink = True
                    flat_sink.append(sink.detach().reshape(-1).to(target))
            flat_bits = self._compute_bits(torch.cat(flat_scores), torch.cat(flat_sink) if any_sink else None)
            cursor = 0
            for l in ordered:
                s = self._prefill_scores[l][b]
                bits_by_layer[l][b] = flat_bits[cursor:cursor + s.numel()].reshape(s.shape).to(s.device)
                cursor += s.numel()
        return bits_by_layer

    def _score_prefill(self, keys, values, layer_idx, *, module, hidden_states, col_sum=None):
        if self._score_prefill_supports_kwargs:
            kwargs = {"module": module, "hidden_states": hidden_states}
            if col_sum is not None:
                kwargs["col_sum"] = col_sum
            return self.scorer.score_prefill(keys, values, layer_idx, **kwargs)
        return self.scorer.score_prefill(keys, values, layer_idx)

    def _score_decode(self, key, value, layer_idx, *, module, hidden_states):
        if self._score_decode_supports_kwargs:
            return self.scorer.score_decode(key, value, layer_idx, module=module, hidden_states=hidden_states)
        return self.scorer.score_decode(key, value, layer_idx)

    # ------------------------------------------------------------------ in-place quantisation
    def _apply_bits(self, keys: torch.Tensor, values: torch.Tensor, bits: torch.Tensor) -> None:
        """keys, values [H, T, d] are overwritten with their quantise->dequantise images at every
        position whose level is neither 0 nor 16."""
        H, T, d = keys.shape
        device, dtype = keys.device, keys.dtype
        for b in sorted(set(self.bit_levels)):
            if b in (0, 16):
                continue
            mask = bits == b
            if not mask.any():
                continue
            h_idx, t_idx = mask.nonzero(as_tuple=True)
            if self.quantizer == "scalar":
                keys[h_idx, t_idx] = _qd_scalar(keys[h_idx, t_idx].float(), b).to(dtype)
                values[h_idx, t_idx] = _qd_scalar(values[h_idx, t_idx].float(), b).to(dtype)
                continue
            keys[h_idx, t_idx] = _qd_keys(self._quantizers.get("key", d, b, device, dtype), keys[h_idx, t_idx]).to(dtype)
            if self.value_quantizer == "mse":
                values[h_idx, t_idx] = _qd_values_mse(self._quantizers.get("value", d, b, device, dtype), values[h_idx, t_idx]).to(dtype)
            else:
                values[h_idx, t_idx] = _qd_values_group(values[h_idx, t_idx].float(), b, self.value_group_size).to(dtype)

    def _finalize_prefill(self, cache) -> None:
        for layer_idx, bits in self._allocate_bits_for_prefill().items():
            keys, values = self._get_cache_tensors(cache, layer_idx)
            keys, values = keys.clone(), values.clone()
            for b in range(keys.shape[0]):
                self._apply_bits(keys[b], values[b], bits[b])
            self._set_cache_tensors(cache, layer_idx, keys, values)
            module = self._layer_modules.get(layer_idx)
            if module is not None:
                module.masked_key_indices = self._bits_to_masked_indices(bits)
        self._reset_prefill_state()

    # ------------------------------------------------------------------ hooks
    def _hook_inputs(self, module, args, kwargs):
        cache = kwargs.get("past_key_values")
        hidden_states = kwargs.get("hidden_states")
        if hidden_states is None and args:
            hidden_states = args[0]
        return cache, hidden_states

    def _prefill_hook(self, module, cache, hidden_states, layer_idx, keys, values) -> None:
        layer_scores = []
        for b in range(keys.shape[0]):
            layer_scores.append(self._score_prefill(keys[b], values[b], layer_idx, module=module,
                                                    hidden_states=hidden_states[b:b + 1]))
            self._prefill_hooks_fired += 1
        self._prefill_scores[layer_idx] = torch.stack(layer_scores, dim=0)
        self._prefill_sink_masks[layer_idx] = self._build_sink_mask(keys.shape[1], keys.shape[2], keys.device)
        if (self._last_hooked_layer_idx is None or layer_idx == self._last_hooked_layer_idx
                or self._finalize_each_layer()):
            self._finalize_prefill(cache)

    def _finalize_each_layer(self) -> bool:
        """Whether a layer's prefill is allocated and stored as soon as its own hook has fired
        (possible when layers have independent budgets) instead of after the last layer's."""
        return False

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
        elif self.decode_quant:
            for b in range(keys.shape[0]):
                k_new, v_new = keys[b, :, -q_len:, :], values[b, :, -q_len:, :]
                h_batch = hidden_states[b:b + 1]
                if q_len == 1:
                    scores = self._score_decode(k_new[:, 0, :], v_new[:, 0, :], layer_idx, module=module,
                                                hidden_states=h_batch).unsqueeze(-1)
                else:
                    scores = self._score_prefill(k_new, v_new, layer_idx, module=module, hidden_states=h_batch)
                self._apply_bits(k_new, v_new, scores_to_bits(scores, self._decode_bit_levels))
        return output

    def _build_tables(self, model) -> None:
        """Rotations and codebooks for every quantised width, on every device that holds an attention module, before
        the first hook fires (built lazily they would sit in the first prefill's time; kvquant/press.py:594-620)."""
        if self.quantizer == "scalar":
            return
        cfg = model.config
        head_dim = getattr(cfg, "head_dim", None) or cfg.hidden_size // cfg.num_attention_heads
        first = next(model.parameters())
        devices = {p.device for _, attn in full_attention_modules(model) for p in list(attn.parameters())[:1]} or {first.device}
        widths = sorted(set(self.bit_levels) - {0, 16})
        roles = ("key", "value") if self.value_quantizer == "mse" else ("key",)
        self._quantizers.build(roles, head_dim, widths, devices, first.dtype)

    def _adopt_module(self, attn: nn.Module) -> None:
        attn.masked_key_indices = None
        rotary = getattr(_backbone(self._model), "rotary_emb", None)
        if rotary is not None:
            try:
                attn.rotary_emb = rotary               # scorers that rebuild queries read it from the module
            except Exception:                          # a module that refuses the attribute keeps working without it
                pass

    def _forget_run(self) -> None:
        self._hooked_layer_indices = []
        self._last_hooked_layer_idx = None
        self._layer_modules = {}
        self._reset_prefill_state()

    @contextlib.contextmanager
    def __call__(self, model):
        """For the duration of the block the press sees every full-attention module's forward."""
        full_attention_modules(model)                      # raises for a model without decoder layers
        self._build_tables(model)
        patch_attention_functions()
        self._forget_run()
        self._model = model
        try:
            with hooked_attention(model, self._forward_hook, adopt=self._adopt_module) as indices:
                self._hooked_layer_indices = indices
                self._last_hooked_layer_idx = indices[-1] if indices else None
                yield
        finally:
            # the eviction masks stay on the modules: decode outside the block must keep honouring them; the attention
            # patch clears them at the next fresh prefill
            self._model = None
            self._forget_run()
