"""A `transformers` cache layer whose tokens live only in the packed store.

The reference keeps a dense fp16 copy of every layer's keys and values in the model's
`DynamicCache` next to its quantised banks (kvquant/adaptive_backend_press.py:131-149 writes the
dequantised rows back into it) and `DynamicLayer.update` re-concatenates that copy at every decode
step.  With the fused decode kernel nothing reads the copy any more, so a press built with
``release_dense_cache=True`` swaps each layer of the cache for a `PackedCacheLayer` once the
prefill has been packed:

* ``keys`` / ``values`` keep the shape ``[B, H, T, D]`` the model and the mask code look at, but
  are stride-0 views of the newest token: no memory, no concatenation;
* a single-token ``update`` re-aliases the views; the attention function takes the token from
  them and everything older from the store;
* an ``update`` with several tokens (prompt text after the prefill) returns the new tokens alone, tagged
  with the store's length: the attention patch runs the block through the fused kernel as well;
* ``crop`` truncates the store; a harness that rewinds the cache the reference's way
  (benchmark/core/pipeline.py:211-228: ``layer._tq_backend_state.truncate`` and a slice of
  ``layer.keys``) works on it unchanged.

The dense attention path cannot run on the aliased views; the attention patch refuses them.
"""
from __future__ import annotations

import torch
from transformers.cache_utils import DynamicLayer


class PackedCacheLayer(DynamicLayer):
    def __init__(self, state, keys: torch.Tensor, values: torch.Tensor):
        """`state` holds every token of `keys`/`values` ([B, H, T, D], the layer's dense cache so
        far); only their last token is kept."""
        super().__init__()
        if state.seq_len != keys.shape[-2]:
            raise ValueError(f"the packed store holds {state.seq_len} tokens, the cache layer {keys.shape[-2]}")
        self.dtype, self.device = keys.dtype, keys.device
        self.is_initialized = True
        self.state = state
        self._tq_backend_state = state
        self.recent = (keys[:, :, -1:, :].clone(), values[:, :, -1:, :].clone())
        self._alias(keys.shape[-2])

    def _alias(self, length: int) -> None:
        k, v = self.recent
        self.keys = k[:, :, -1:, :].expand(-1, -1, length, -1)
        self.values = v[:, :, -1:, :].expand(-1, -1, length, -1)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, *args, **kwargs):
        q_len = key_states.shape[-2]
        before = self.keys.shape[-2]
        if q_len == 1:
            self.recent = (key_states, value_states)
            self._alias(before + 1)
            return self.keys, self.values
        if self.state.seq_len != before:
            raise RuntimeError(f"the packed store holds {self.state.seq_len} tokens, the cache layer {before}: "
                               "a multi-token step needs the two in step")
        # the new tokens alone, tagged with the number of tokens the store holds: the attention patch takes the
        # stored part from the fused kernel and the block's own attention from these (nothing is dequantised)
        key_states._odmkv_store_len = before
        value_states._odmkv_store_len = before
        self.recent = (key_states, value_states)
        self._alias(before + q_len)
        return key_states, value_states

    def crop(self, tokens_to_remove: int) -> None:
        current = self.keys.shape[-2]
        if tokens_to_remove > 0:                      # legacy meaning: the length to keep
            if tokens_to_remove >= current:
                return
            tokens_to_remove = current - tokens_to_remove
        if tokens_to_remove == 0:
            return
        length = max(current - abs(tokens_to_remove), 0)
        self.state.truncate(length)
        self._alias(length)

    # the dense-tensor operations of the base class have no meaning on aliased views
    def reset(self) -> None:
        raise NotImplementedError("PackedCacheLayer cannot be reset in place: start a new cache")

    def reorder_cache(self, beam_idx) -> None:
        raise NotImplementedError("PackedCacheLayer does not support beam reordering")

    def batch_repeat_interleave(self, repeats: int) -> None:
        raise NotImplementedError("PackedCacheLayer does not support batch expansion")

    def batch_select_indices(self, indices) -> None:
        raise NotImplementedError("PackedCacheLayer does not support batch selection")

    def offload(self) -> None:
        return

    def prefetch(self) -> None:
        return


def is_aliased(t: torch.Tensor) -> bool:
    """True for the stride-0 token views a `PackedCacheLayer` hands out."""
    return t.dim() == 4 and t.shape[2] > 1 and t.stride(2) == 0
