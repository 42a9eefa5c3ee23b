"""TurboQuantBackendPress: uniform-width backend press (every token at key_bits / value_bits).

Not part of the ODM-KV mixed-precision path; kept so that the names the reference's
kvquant/__init__.py:10-17 exports exist.  A thin version of kvquant/backend_press.py:15-148 for the
MSE quantiser: historical tokens are quantised->dequantised in place in the HF cache with the row
kernels, the most recent ``buffer_size`` tokens stay exact.  Other quantiser families raise.
"""
from __future__ import annotations

import contextlib
from dataclasses import dataclass, field
from typing import Any, Optional

import torch
from torch import nn

from kvquant.press import hooked_attention
from kvquant.tq_backend import TurboQuantMSE, normalize_key_quantizer, normalize_value_quantizer


@dataclass
class TurboQuantBackendPress:
    key_bits: int = 3
    value_bits: int = 2
    key_quantizer: str = "mse"
    value_quantizer: str = "minmax"
    value_group_size: int = 32
    buffer_size: int = 128
    initial_layers_count: int = 0
    initial_layers_key_bits: Optional[int] = None
    seed: int = 42
    decode_quant: bool = True
    _done: dict = field(default_factory=dict, init=False, repr=False)      # layer -> tokens already quantised
    _qs: dict = field(default_factory=dict, init=False, repr=False)

    def __post_init__(self):
        if normalize_key_quantizer(self.key_quantizer) != "mse" or normalize_value_quantizer(self.value_quantizer) != "mse":
            raise NotImplementedError("TurboQuantBackendPress is built for key_quantizer='mse', value_quantizer='mse' only")

    def _layer_key_bits(self, layer_idx: int) -> int:
        if self.initial_layers_count > 0 and self.initial_layers_key_bits is not None and layer_idx < self.initial_layers_count:
            return self.initial_layers_key_bits
        return self.key_bits

    def _q(self, bits: int, seed: int, ref: torch.Tensor) -> TurboQuantMSE:
        key = (bits, seed, ref.device, ref.dtype)
        if key not in self._qs:
            self._qs[key] = TurboQuantMSE(ref.shape[-1], bits, device=ref.device, dtype=ref.dtype, seed=seed)
        return self._qs[key]

    def _quantise_span(self, layer_idx: int, keys: torch.Tensor, values: torch.Tensor, lo: int, hi: int) -> None:
        if hi <= lo:
            return
        seed = self.seed + layer_idx * 7
        kq = self._q(self._layer_key_bits(layer_idx), seed, keys)
        vq = self._q(self.value_bits, seed + 2000, values)
        k = keys[:, :, lo:hi, :]
        v = values[:, :, lo:hi, :]
        keys[:, :, lo:hi, :] = kq.dequantize(kq.quantize(k.reshape(-1, k.shape[-1]))).reshape(k.shape).to(keys.dtype)
        values[:, :, lo:hi, :] = vq.dequantize(vq.quantize(v.reshape(-1, v.shape[-1]))).reshape(v.shape).to(values.dtype)

    def forward_hook(self, module: nn.Module, _input: tuple, kwargs: dict, output: Any) -> Any:
        # the layer's input arrives by keyword in current transformers, positionally in older ones
        hidden_states = kwargs["hidden_states"] if kwargs.get("hidden_states") is not None else (_input[0] if _input else None)
        cache, layer_idx = kwargs.get("past_key_values"), getattr(module, "layer_idx", None)
        if any(x is None for x in (hidden_states, cache, layer_idx)):
            return output
        layer_idx = int(layer_idx)
        layer = cache.layers[layer_idx]
        keys, values = layer.keys, layer.values
        q_len, cache_len = hidden_states.shape[1], keys.shape[2]
        if cache_len == q_len:
            self._done[layer_idx] = 0
        elif not self.decode_quant:
            return output
        done = min(self._done.get(layer_idx, 0), cache_len)
        upto = max(cache_len - self.buffer_size, 0)
        self._quantise_span(layer_idx, keys, values, done, upto)
        self._done[layer_idx] = max(done, upto)
        return output

    @contextlib.contextmanager
    def __call__(self, model):
        self._done = {}
        try:
            with hooked_attention(model, self.forward_hook):
                yield
        finally:
            self._done = {}
