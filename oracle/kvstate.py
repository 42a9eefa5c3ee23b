"""Oracle: the mixed-precision KV store (banks of tokens keyed by bit level).

Follows /root/reference/kvquant/tq_adaptive_backend.py
  ExactBank                         :31-70
  QuantizedBank.append / materialize :149-174, 205-242  (key/value quantiser "mse", no OCS)
  TurboQuantAdaptiveKVCacheState    :245-541
    append :350-374, append_all_exact :380-425, truncate :427-437,
    materialize :439-452, materialize_quantized_into :454-464,
    get_buffer_tokens :466-479, flush_buffer :481-532, masked_key_indices :534-541
Every quantised level of a state shares one key rotation (seed) and one value rotation
(seed + 2000) (tq_adaptive_backend.py:120-130).
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .quantizer import Quantized, dequantize, quantize, random_rotation


class _Bank:
    def __init__(self):
        self.pos = np.zeros((0, 3), np.int64)      # rows (batch, head, token)

    @property
    def size(self) -> int:
        return int(self.pos.shape[0])


class _ExactBank(_Bank):
    def __init__(self):
        super().__init__()
        self.k: Optional[torch.Tensor] = None
        self.v: Optional[torch.Tensor] = None

    def append(self, pos, k, v):
        if pos.shape[0] == 0:
            return
        self.pos = np.concatenate([self.pos, pos])
        self.k = k.clone() if self.k is None else torch.cat([self.k, k])
        self.v = v.clone() if self.v is None else torch.cat([self.v, v])

    def keep(self, mask: np.ndarray):
        self.pos = self.pos[mask]
        if self.size == 0:
            self.k = self.v = None
        else:
            m = torch.from_numpy(mask)
            self.k, self.v = self.k[m], self.v[m]


class _QuantBank(_Bank):
    def __init__(self, bits: int):
        super().__init__()
        self.bits = bits
        self.kc = self.vc = None      # uint8 codes [N, d]
        self.kn = self.vn = None      # fp32 norms [N]

    def append(self, pos, kq: Quantized, vq: Quantized):
        if pos.shape[0] == 0:
            return
        first = self.size == 0
        self.pos = np.concatenate([self.pos, pos])
        self.kc = kq.codes if first else np.concatenate([self.kc, kq.codes])
        self.vc = vq.codes if first else np.concatenate([self.vc, vq.codes])
        self.kn = kq.norms if first else np.concatenate([self.kn, kq.norms])
        self.vn = vq.norms if first else np.concatenate([self.vn, vq.norms])

    def keep(self, mask: np.ndarray):
        self.pos = self.pos[mask]
        self.kc, self.vc, self.kn, self.vn = self.kc[mask], self.vc[mask], self.kn[mask], self.vn[mask]


class KVState:
    """CPU model of ``TurboQuantAdaptiveKVCacheState`` with key_quantizer = value_quantizer = "mse"."""

    def __init__(self, head_dim: int, bit_levels, dtype=torch.float16, seed: int = 42,
                 order: str = "blas"):
        self.head_dim = head_dim
        self.bit_levels = tuple(sorted(set(int(b) for b in bit_levels)))
        self.dtype = dtype
        self.order = order
        self.pi_k = random_rotation(head_dim, seed)
        self.pi_v = random_rotation(head_dim, seed + 2000)
        self._reset()

    def _reset(self):
        self.batch_size = self.num_heads = self.seq_len = 0
        self.exact = _ExactBank()
        self.banks = {b: _QuantBank(b) for b in self.bit_levels if b not in (0, 16)}
        self.masked = np.zeros((0, 3), np.int64)

    # -- routing ---------------------------------------------------------------------------
    def _route(self, level: int, pos: np.ndarray, k: torch.Tensor, v: torch.Tensor):
        if level == 0:
            self.masked = np.concatenate([self.masked, pos])
        elif level == 16:
            self.exact.append(pos, k, v)
        else:
            self.banks[level].append(pos, quantize(k, self.pi_k, level, order=self.order),
                                     quantize(v, self.pi_v, level, order=self.order))

    def prefill(self, keys, values, bits):
        self._reset()
        self.append(keys, values, bits)

    def append(self, keys: torch.Tensor, values: torch.Tensor, bits: torch.Tensor):
        if keys.shape != values.shape or keys.dim() != 4 or tuple(bits.shape) != tuple(keys.shape[:3]):
            raise ValueError("expected keys/values [B,H,T,D] and bits [B,H,T]")
        if self.batch_size == 0:
            self.batch_size, self.num_heads = int(keys.shape[0]), int(keys.shape[1])
        b_np = bits.detach().cpu().numpy().astype(np.int32)
        for level in self.bit_levels:
            local = np.argwhere(b_np == level)             # row-major (b, h, t), like nonzero
            if local.shape[0] == 0:
                continue
            li = torch.from_numpy(local)
            k = keys[li[:, 0], li[:, 1], li[:, 2]]
            v = values[li[:, 0], li[:, 1], li[:, 2]]
            pos = local.astype(np.int64).copy()
            pos[:, 2] += self.seq_len
            self._route(level, pos, k, v)
        self.seq_len += int(keys.shape[2])

    def append_all_exact(self, keys: torch.Tensor, values: torch.Tensor):
        B, H, T, D = keys.shape
        if self.batch_size == 0:
            self.batch_size, self.num_heads = B, H
        if T == 0:
            return
        bb, hh, tt = np.meshgrid(np.arange(B), np.arange(H), np.arange(T) + self.seq_len, indexing="ij")
        pos = np.stack([bb.ravel(), hh.ravel(), tt.ravel()], axis=-1).astype(np.int64)
        self.exact.append(pos, keys.reshape(-1, D), values.reshape(-1, D))
        self.seq_len += T

    def truncate(self, seq_len: int):
        seq_len = int(seq_len)
        if seq_len >= self.seq_len:
            return
        self.seq_len = seq_len
        if self.exact.size:
            self.exact.keep(self.exact.pos[:, 2] < seq_len)
        self.masked = self.masked[self.masked[:, 2] < seq_len]
        for bank in self.banks.values():
            if bank.size:
                bank.keep(bank.pos[:, 2] < seq_len)

    # -- read back -------------------------------------------------------------------------
    def _scatter_quantized(self, keys, values):
        for bank in self.banks.values():
            if bank.size == 0:
                continue
            p = torch.from_numpy(bank.pos)
            dk = dequantize(Quantized(bank.kc, bank.kn, bank.bits), self.pi_k).to(keys.dtype)
            dv = dequantize(Quantized(bank.vc, bank.vn, bank.bits), self.pi_v).to(values.dtype)
            keys[p[:, 0], p[:, 1], p[:, 2]] = dk
            values[p[:, 0], p[:, 1], p[:, 2]] = dv

    def materialize(self):
        keys = torch.zeros(self.batch_size, self.num_heads, self.seq_len, self.head_dim, dtype=self.dtype)
        values = torch.zeros_like(keys)
        if self.exact.size:
            p = torch.from_numpy(self.exact.pos)
            keys[p[:, 0], p[:, 1], p[:, 2]] = self.exact.k.to(keys.dtype)
            values[p[:, 0], p[:, 1], p[:, 2]] = self.exact.v.to(values.dtype)
        self._scatter_quantized(keys, values)
        return keys, values

    def materialize_quantized_into(self, keys, values):
        self._scatter_quantized(keys, values)

    def visible_mask(self) -> torch.Tensor:
        """bool [B, H, T]: False at evicted (0-bit) positions."""
        m = torch.ones(self.batch_size, self.num_heads, self.seq_len, dtype=torch.bool)
        if self.masked.shape[0]:
            p = torch.from_numpy(self.masked)
            m[p[:, 0], p[:, 1], p[:, 2]] = False
        return m

    def masked_key_indices(self):
        if self.masked.shape[0] == 0:
            return None
        p = torch.from_numpy(self.masked)
        return p[:, 0], p[:, 1], p[:, 2]

    def level_map(self) -> np.ndarray:
        """int32 [B, H, T] bit level stored at every position (test helper)."""
        out = np.full((self.batch_size, self.num_heads, self.seq_len), -1, np.int32)
        for lvl, pos in [(0, self.masked), (16, self.exact.pos)] + [(b, k.pos) for b, k in self.banks.items()]:
            if pos.shape[0]:
                out[pos[:, 0], pos[:, 1], pos[:, 2]] = lvl
        return out

    # -- decode buffer ---------------------------------------------------------------------
    def get_buffer_tokens(self, start: int):
        if self.exact.size:
            m = self.exact.pos[:, 2] >= start
            if m.any():
                mt = torch.from_numpy(m)
                return self.exact.pos[m], self.exact.k[mt], self.exact.v[mt]
        empty = torch.empty(0, self.head_dim, dtype=self.dtype)
        return np.zeros((0, 3), np.int64), empty, empty.clone()

    def flush_buffer(self, start: int, new_bits: torch.Tensor):
        if self.exact.size == 0:
            return
        m = self.exact.pos[:, 2] >= start
        if not m.any():
            return
        mt = torch.from_numpy(m)
        pos, k, v = self.exact.pos[m], self.exact.k[mt], self.exact.v[mt]
        self.exact.keep(~m)
        nb = new_bits.detach().cpu().numpy().astype(np.int32)
        routed = np.zeros(nb.shape[0], bool)
        for level in self.bit_levels:
            lm = nb == level
            if not lm.any():
                continue
            routed |= lm
            lt = torch.from_numpy(lm)
            self._route(level, pos[lm], k[lt], v[lt])
        if not routed.all():
            o = ~routed
            self.exact.append(pos[o], k[torch.from_numpy(o)], v[torch.from_numpy(o)])

    def packed_bytes(self, norm_bytes: int = 4) -> int:
        """Payload a fused decode kernel has to read: true b-bit codes for K and V, their norms,
        and fp16 rows of the exact tokens."""
        d = self.head_dim
        total = self.exact.size * 2 * d * 2
        for b, bank in self.banks.items():
            total += bank.size * (2 * b * d // 8 + 2 * norm_bytes)
        return total
