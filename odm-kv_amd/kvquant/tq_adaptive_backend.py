"""Mixed-precision KV store on the GPU: bit-packed tiles instead of per-level banks.

``TurboQuantAdaptiveKVCacheState`` keeps the constructor and the method set of the reference's
class of the same name (kvquant/tq_adaptive_backend.py:245-541): ``prefill``, ``append``,
``append_all_exact``, ``truncate``, ``materialize``, ``materialize_quantized_into``,
``get_buffer_tokens``, ``flush_buffer``, ``masked_key_indices`` - and adds what a packed store
makes possible: ``decode_attention`` (fused LUT attention straight from the packed bytes) and
``packed_bytes``.

Layout (see include/odmkv.h): per bit level, tokens of one (sequence, kv-head) form a segment of
64-token tiles in ascending position; codes lie in the order the decode kernel's matrix operands take
them (keys: 4 tokens x 32 dims per 16*w bytes, values: 16 tokens x 8 dims), norms fp32.
Evicted (0-bit) tokens are not stored at all.  The host keeps a mirror of every segment's length,
so that after the one synchronisation an ``append`` needs (to size the buffers from the level
counts) no later call has to read anything back.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Optional

import numpy as np
import torch

from . import _lib
from ._lib import lib, Packed, TILE, HEAD_DIM, WIDTHS
from .tq_backend import (cached_rotation, codebook_table, decode_tables, normalize_key_quantizer,
                         normalize_value_quantizer)

_LEVEL_INDEX = {2: 0, 3: 1, 4: 2, 8: 3, 16: 4}


def _exact_index_tables():
    """[64, 128] element index of (slot, dim) inside an exact tile, for keys and for values
    (the layouts of include/odmkv.h)."""
    slot = np.arange(TILE)[:, None]
    dim = np.arange(HEAD_DIM)[None, :]
    kb, kn = 2 * (slot >> 5) + (slot & 1), 4 * ((slot >> 3) & 3) + ((slot >> 1) & 3)      # key block and column of the slot
    k_idx = (((4 * kb + ((dim >> 3) & 3)) * TILE) + 16 * (dim >> 5) + kn) * 8 + (dim & 7)
    v_idx = (((8 * (slot >> 5) + (dim >> 4)) * TILE) + 16 * ((slot >> 3) & 3) + (dim & 15)) * 8 + (slot & 7)
    return k_idx.astype(np.int64), v_idx.astype(np.int64)


_EXACT_K_IDX, _EXACT_V_IDX = _exact_index_tables()
_CU_COUNT: dict = {}


def _compute_units(device) -> int:
    key = str(device)
    if key not in _CU_COUNT:
        _CU_COUNT[key] = torch.cuda.get_device_properties(device).multi_processor_count
    return _CU_COUNT[key]
_TILE_BYTES = [TILE * 16 * w + 2 * TILE * 4 for w in WIDTHS] + [2 * TILE * HEAD_DIM * 2]
# what one compute unit was measured to need per 64-token tile of each level (nanoseconds; 2, 3, 4, 8 bits, exact rows)
# and per work item (microseconds: start, table, query rotation, combining the wavefronts)
_TILE_COST = [300, 420, 450, 890, 1310]
_ITEM_FIXED_US = 4.0           # what the cuts without chains are compared with (its choices were measured shape by shape)
# Chains (a workgroup that walks several quantised levels of a pair, _build_items) by a rule, not by the cost model, which
# is off by a third either way on lists of several rounds: they are taken when the quantised runs number at least 1.5 per
# compute unit and 2.5 per pair, cut so that the workgroups number 1.5 per compute unit or, with more pairs than that,
# one per pair beside the exact items.  Measured whole calls: 64 sequences x 2048 tokens x 8 kv-heads, four levels each:
# 90 -> 67 us; 16 x 8192 tokens with four levels: 44 -> 36 us; 16 x 8192 tokens with two levels (c3): no gain at any cut,
# not taken by the rule.  The link and rotation costs below only rank the workgroups for the dispatch order.
_CHAIN_LINK_US = 1.8
_PAIR_CHAIN_RUNS_PER_PLACE = 1.5      # two workgroups per compute unit: chains where the runs number this many per place
_CHAIN_ROTATE_US = 1.0
_CHAIN_RUNS_PER_CU = 1.5
_CHAIN_RUNS_PER_PAIR = 2.5


_U64x33 = C.c_uint64 * 33
_U64x5 = C.c_uint64 * 5
# index of a buffer in the layout of odmkv_store_layout: name -> (first index, step per level)
_SLOT = {"seg_tile": (0, 1), "seg_count": (5, 1), "knorm": (10, 2), "vnorm": (11, 2), "kexact": (18, 0), "vexact": (19, 0),
         "pos": (20, 1), "kcodes": (25, 2), "vcodes": (26, 2)}


class _Layout:
    """Where the buffers of a store lie inside one allocation (odmkv_store_layout) for given segment tables."""

    def __init__(self, seg_tile: np.ndarray, nseg: int):
        self.tables = np.ascontiguousarray(seg_tile, dtype=np.int32)     # [5, nseg + 1]
        self.tables_ptr = self.tables.ctypes.data
        self.nseg = nseg
        self.offsets, self.sizes, marks = _U64x33(), _U64x33(), _U64x5()
        _lib.check(lib.odmkv_store_layout(self.tables_ptr, nseg, self.offsets, self.sizes, marks))
        self.tables_end, self.counts_end, self.zero_end, self.pos_end, self.total = (int(m) for m in marks)

    @classmethod
    def blank(cls, nseg: int) -> "_Layout":
        """Arrays for odmkv_store_finish_staged to fill; `adopt` reads the marks afterwards."""
        self = cls.__new__(cls)
        self.tables = np.zeros((5, nseg + 1), np.int32)
        self.tables_ptr = self.tables.ctypes.data
        self.nseg = nseg
        self.offsets, self.sizes, self.marks = _U64x33(), _U64x33(), _U64x5()
        return self

    def adopt(self) -> "_Layout":
        self.tables_end, self.counts_end, self.zero_end, self.pos_end, self.total = (int(m) for m in self.marks)
        return self

    def init(self, arena: torch.Tensor, stream: int, counts_only: bool = False) -> None:
        """Tables written, counters / norms / exact rows cleared, positions -1 (counts_only: just the tables and
        the segment counts): one launch, the tables in its arguments."""
        zero_end = self.counts_end if counts_only else self.zero_end
        fill_end = self.counts_end if counts_only else self.pos_end
        _lib.check(lib.odmkv_store_init(arena.data_ptr(), self.tables_ptr, 5, self.nseg + 1, C.addressof(self.offsets),
                                        self.tables_end, zero_end, fill_end, stream))

    def struct(self, arena: torch.Tensor, B: int, H: int, exact_dtype: torch.dtype) -> Packed:
        p = Packed()
        _lib.check(lib.odmkv_store_bind(arena.data_ptr(), self.offsets, self.tables_ptr, self.nseg, B, H,
                                        _lib.BF16 if exact_dtype == torch.bfloat16 else _lib.F16, C.byref(p)))
        return p


class _Buffers:
    """The store's buffers inside one allocation; tensor views are made when somebody asks."""

    def __init__(self, arena: torch.Tensor, layout: _Layout, exact_dtype: torch.dtype):
        self.arena = arena
        self.layout = layout
        self._exact_dtype = exact_dtype

    def view(self, name: str, li=None) -> torch.Tensor:
        first, step = _SLOT[name]
        i = first + step * (li or 0)
        off, nbytes = int(self.layout.offsets[i]), int(self.layout.sizes[i])
        dtype = (torch.int32 if name in ("seg_tile", "seg_count", "pos") else torch.float32 if name in ("knorm", "vnorm")
                 else self._exact_dtype if name in ("kexact", "vexact") else torch.uint8)
        return self.arena[off:off + nbytes].view(dtype)

    def __getitem__(self, name: str):
        if name in ("kexact", "vexact"):
            return self.view(name)
        n = 5 if name in ("pos", "seg_tile", "seg_count") else 4
        return [self.view(name, li) for li in range(n)]


_ARENA_HINT: dict = {}     # (device, segments, tokens) -> bytes of the last store first filled with that shape
_STAGING_LIMIT = 4 << 30   # bytes a staging store may take (1.4 % of the device's memory; a 131072-token layer of 8 KV
#                            heads takes 1.2 GB); larger first fills wait for the counts instead
_STAGING: dict = {}        # (device, stream) -> _Staging: one per stream, rebuilt when the shape changes
_MAILBOX: dict = {}        # (device, stream) -> (page-locked int32 tensor, ..., event): where the level counts arrive


def _dev_key(dev) -> str:
    d = torch.device(dev)
    return f"{d.type}:{torch.cuda.current_device() if d.index is None else d.index}"


def reserve_state_memory(device, n_states: int) -> None:
    """Grow the allocator's small-block pool, in one go, by what `n_states` stores will keep in it (rotations, operand
    and centroid tables, work lists: about a third of a megabyte each).  Otherwise the pool grows by one 2 MB device
    allocation every few layers of a first prefill, 0.2 ms of host time each, at whatever small request comes next:
    between the kernels of a layer's compression.  The blocks go back to the pool at once; a process that has served a
    prompt before has them anyway."""
    hold = [torch.empty(384 << 10, dtype=torch.uint8, device=device) for _ in range(int(n_states))]
    del hold


def release_staging(device=None) -> None:
    """Hand the staging stores (of one device, or of all) back to the allocator: a press does so when the last layer
    of a prefill is stored, so that the decode steps which follow do not hold a worst-case store they never use.
    (Work already queued on the staging store's stream keeps its memory until it has run: the allocator returns a
    block to the stream it was requested on.)"""
    for key in [k for k in _STAGING if device is None or k[0] == _dev_key(device)]:
        del _STAGING[key]


class _Staging:
    """A store whose every segment has room for all T tokens of a call at every level: it can be filled before the
    level counts are known.  The first fill of a store quantises into it while the host still waits for the counts
    and lays out the store proper; odmkv_store_gather then moves the tiles that hold tokens."""

    def __init__(self, dev, B: int, H: int, T: int, exact_dtype: torch.dtype):
        nseg = B * H
        self.key = (B, H, T, exact_dtype)
        per_seg = (T + TILE - 1) // TILE
        self.seg_tile = np.tile(np.arange(nseg + 1, dtype=np.int64) * per_seg, (5, 1))
        self.layout = _Layout(self.seg_tile, nseg)
        self.bufs = _Buffers(torch.empty(self.layout.total, dtype=torch.uint8, device=dev), self.layout, exact_dtype)
        self.packed = self.layout.struct(self.bufs.arena, B, H, exact_dtype)

    @staticmethod
    def bytes_needed(nseg: int, T: int) -> int:
        tiles = nseg * ((T + TILE - 1) // TILE)
        return tiles * (sum(2 * TILE * 16 * w + 2 * TILE * 4 for w in WIDTHS) + 2 * TILE * HEAD_DIM * 2 + 5 * TILE * 4)

    def reset(self, stream: int) -> None:
        """Tables in place, segment counts zero; everything else is written before it is read."""
        self.layout.init(self.bufs.arena, stream, counts_only=True)


def _staging_for(dev, stream: int, B: int, H: int, T: int, exact_dtype: torch.dtype) -> "_Staging":
    got = _STAGING.get((_dev_key(dev), stream))
    if got is None or got.key != (B, H, T, exact_dtype):
        _STAGING.pop((_dev_key(dev), stream), None)          # the old one is released before the new one is requested
        got = _STAGING[(_dev_key(dev), stream)] = _Staging(dev, B, H, T, exact_dtype)
    return got


def _mailbox(dev, stream: int, numel: int):
    """(page-locked int32 tensor, device int32 tensor, event, the event's handle): where the level counts of the fills
    queued on `stream` arrive (one box per stream: fills on two streams of a device do not share it)."""
    got = _MAILBOX.get((_dev_key(dev), stream))
    if got is None or got[0].numel() < numel:
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(dev))          # (the handle exists once the event has been recorded)
        ev.synchronize()
        n = max(numel, 4096)
        got = _MAILBOX[(_dev_key(dev), stream)] = (torch.zeros(n, dtype=torch.int32, pin_memory=True),
                                    torch.empty(n, dtype=torch.int32, device=dev), ev, int(ev.cuda_event))
    return got


HEAD_DIM_OPS = 128 * 128      # elements of one part of the operand table
_ROT_OPS_CACHE: dict = {}


def _rotation_operands(pi_k: torch.Tensor) -> torch.Tensor:
    """The key rotation as the matrix operands of the decode kernel's query rotation (odmkv_rotation_operands):
    int16 [32768] on pi_k's device, built once per rotation tensor (rotations are cached per (dim, seed, device), so
    every layer's state that shares a seed shares the table)."""
    key = (pi_k.data_ptr(), str(pi_k.device))
    hit = _ROT_OPS_CACHE.get(key)
    if hit is None or hit[0] is not pi_k:
        ops = torch.empty(2 * HEAD_DIM_OPS, dtype=torch.int16, device=pi_k.device)
        _lib.check(lib.odmkv_rotation_operands(pi_k.data_ptr(), ops.data_ptr(), _lib.stream_ptr(pi_k.device)))
        hit = _ROT_OPS_CACHE[key] = (pi_k, ops)
    return hit[1]


def _empty_positions(device) -> torch.Tensor:
    return torch.empty((0, 3), dtype=torch.long, device=device)


class TurboQuantAdaptiveKVCacheState:
    def __init__(self, head_dim: int, bit_levels, value_group_size: int = 32, device=None,
                 dtype: torch.dtype = torch.float16, key_quantizer: str = "prod",
                 value_quantizer: str = "minmax", seed: int = 42, outlier_indices=None,
                 regular_indices=None, outlier_min_bits: int = 4, exact_slack: int = 256,
                 quant_headroom: bool = False):
        levels = tuple(sorted(set(int(b) for b in bit_levels)))
        self.key_quantizer = normalize_key_quantizer(key_quantizer)
        self.value_quantizer = normalize_value_quantizer(value_quantizer)
        min_bits = 2 if self.key_quantizer == "prod" else 1
        invalid = [b for b in levels if b not in (0, 16) and b < min_bits]
        if invalid:
            raise ValueError(
                f"Adaptive TurboQuant backend requires key bits >= {min_bits} "
                f"for key_quantizer={self.key_quantizer!r}; unsupported levels: {invalid}")
        if self.key_quantizer != "mse" or self.value_quantizer != "mse":
            raise NotImplementedError(
                "the packed GPU store implements key_quantizer='mse' and value_quantizer='mse' "
                "(the paper configuration); QJL keys and min-max values are not built")
        if outlier_indices is not None or regular_indices is not None:
            raise NotImplementedError("outlier-channel separation is not built (n_outlier_channels must be 0)")
        unsupported = [b for b in levels if b not in (0, 2, 3, 4, 8, 16)]
        if unsupported:
            raise ValueError(f"bit levels must come from (0, 2, 3, 4, 8, 16); got {unsupported}")
        if head_dim != HEAD_DIM:
            raise ValueError(f"the HIP kernels are written for head_dim {HEAD_DIM}, got {head_dim}")
        self.head_dim = head_dim
        self.bit_levels = levels
        group = min(value_group_size, head_dim)
        if head_dim % group != 0:
            group = math.gcd(head_dim, group)
        self.value_group_size = max(1, group)
        self.device = torch.device(device) if device is not None else torch.device("cuda")
        self.dtype = dtype
        self.seed = seed
        self.outlier_min_bits = outlier_min_bits
        self.exact_slack = int(exact_slack)
        # room in the quantised segments from the first fill on, for a store that decode-time flushes will add to
        self.quant_headroom = bool(quant_headroom)
        if self.device.type != "cuda":
            raise RuntimeError("the packed KV store lives on the GPU; there is no CPU path")
        self.pi_k = cached_rotation(head_dim, self.device, seed)
        self.pi_v = cached_rotation(head_dim, self.device, seed + 2000)
        # the key rotation as the decode kernel's matrix operands (fp16 high + low parts in operand order)
        self._pi_k_ops = _rotation_operands(self.pi_k)
        self.codebooks = codebook_table(head_dim, self.device)
        self._decode_cb, inv = decode_tables(head_dim, self.device)
        self._decode_inv = (C.c_float * 4)(*inv)
        self._decode_cb_host = (C.c_float * 284)(*self._decode_cb.cpu().tolist())
        self._exact_torch_dtype = torch.bfloat16 if dtype == torch.bfloat16 else torch.float16
        self._reset()

    # ------------------------------------------------------------------ storage
    def _reset(self) -> None:
        self.batch_size = 0
        self.num_heads = 0
        self.seq_len = 0
        self._nseg = 0
        self._counts = None           # np.int64 [5, nseg]   tokens stored per level and segment
        self._exact_room = None       # tokens every exact segment can still take (None: not known)
        self._seg_tile = None         # np.int64 [5, nseg+1] first tile of each segment
        self._bufs = None
        self._level_store = None      # uint8 [B, H, capacity]: bit level of every position (grown by doubling)
        self._masked = None           # cached (indices of evicted positions,) or None when stale
        self._items = None
        self._item_order = None
        self._worklist = None         # ctypes twin of odmkv_worklist_t over the tensors above
        self._step = None             # decode_step's odmkv_step_t with what it was built for and what it points to
        self._items_choice = None     # (winning items-per-compute-unit multiple, packed bytes it was chosen at)
        self._packed = None

    @property
    def _level_map(self):
        """uint8 [B, H, seq_len]: bit level of every position (a view of the growing store)."""
        return None if self._level_store is None else self._level_store[:, :, :self.seq_len]

    def _extend_levels(self, lm: torch.Tensor, owned: bool = False) -> None:
        """Write the levels of T new positions behind the current ones (before seq_len is advanced).  owned: lm is
        a tensor nobody else holds; the first fill of a store keeps it as the level store instead of copying it."""
        B, H, T = lm.shape
        need = self.seq_len + T
        if owned and self._level_store is None and self.seq_len == 0 and T >= 256 and lm.is_contiguous():
            self._level_store = lm
            return
        if self._level_store is None or self._level_store.shape[2] < need:
            cap = max(need, 2 * (0 if self._level_store is None else self._level_store.shape[2]), 256)
            # positions behind seq_len read 16, so that a single exact token needs no write
            grown = torch.full((B, H, cap), 16, dtype=torch.uint8, device=self.device)
            if self._level_store is not None and self.seq_len:
                grown[:, :, :self.seq_len] = self._level_store[:, :, :self.seq_len]
            self._level_store = grown
        self._level_store[:, :, self.seq_len:need] = lm

    def _alloc(self, seg_tile: np.ndarray) -> "_Buffers":
        """All buffers of the store as views into one allocation: the segment tables, the counters, norms and
        exact rows (zeroed; exact rows take part in the products as they are: a zero weight does not silence a
        NaN), the positions (-1), then the codes (left as they come: every code the kernels read is written
        first or is a padding lane masked by count)."""
        dev = self.device
        layout = _Layout(seg_tile, self._nseg)
        off = layout.total
        arena = getattr(self, "_arena", None)
        if arena is not None and self._level_store is not None and (self._level_store.untyped_storage().data_ptr()
                                                                    == arena.untyped_storage().data_ptr()):
            self._level_store = self._level_store.clone()    # the level map of a staged first fill lies behind the old store
        if arena is None or arena.numel() < off or arena.device != dev:
            arena = torch.empty(off + off // 8, dtype=torch.uint8, device=dev)
            self._arena_spare = None
        elif self._bufs is not None:
            # the live store is in this arena: build the new one elsewhere, keep the old as the spare
            spare = getattr(self, "_arena_spare", None)
            if spare is None or spare.numel() < off:
                spare = torch.empty(off + off // 8, dtype=torch.uint8, device=dev)
            arena, self._arena_spare = spare, arena
        self._arena = arena
        layout.init(arena, _lib.stream_ptr(dev))
        return _Buffers(arena, layout, self._exact_torch_dtype)

    def _make_struct(self) -> None:
        self._packed = self._bufs.layout.struct(self._bufs.arena, self.batch_size, self.num_heads, self._exact_torch_dtype)

    def _capacity_tiles(self, counts: np.ndarray) -> np.ndarray:
        """Tiles per (level, segment) for `counts` tokens; exact segments get room to grow."""
        cap = (counts + TILE - 1) // TILE
        cap[4] = (counts[4] + self.exact_slack + TILE - 1) // TILE
        return cap

    def _ensure_capacity(self, new_counts: np.ndarray) -> None:
        """Make every segment large enough for `new_counts`, moving stored tiles if it must grow."""
        if self._bufs is not None:
            have = np.diff(self._seg_tile, axis=1)
            if np.all((new_counts + TILE - 1) // TILE <= have):
                return
        cap = self._capacity_tiles(new_counts)
        if self._bufs is not None or self.quant_headroom:
            # a store that grows once will grow again (every decode-time flush adds tokens to the
            # quantised levels): leave a sixteenth of head-room so that the tiles move rarely
            cap[:4] += np.maximum(cap[:4] // 16, 2)
        if self._bufs is not None:
            cap = np.maximum(cap, np.diff(self._seg_tile, axis=1))
        seg_tile = np.zeros((5, self._nseg + 1), np.int64)
        seg_tile[:, 1:] = np.cumsum(cap, axis=1)
        new = self._alloc(seg_tile)
        if self._bufs is not None:
            old, old_tile = self._bufs, self._seg_tile
            for li in range(5):
                used = (self._counts[li] + TILE - 1) // TILE
                if used.sum() == 0:
                    continue
                src = np.concatenate([np.arange(old_tile[li, s], old_tile[li, s] + used[s]) for s in range(self._nseg)])
                dst = np.concatenate([np.arange(seg_tile[li, s], seg_tile[li, s] + used[s]) for s in range(self._nseg)])
                src_t = torch.from_numpy(src).to(self.device)
                dst_t = torch.from_numpy(dst).to(self.device)
                names = ["pos"] + (["kcodes", "vcodes", "knorm", "vnorm"] if li < 4 else [])
                for name in names:
                    o, n = old[name][li], new[name][li]
                    per = o.numel() // max(int(old_tile[li, -1]), 1)
                    n.view(-1, per)[dst_t] = o.view(-1, per)[src_t]
                if li == 4:
                    for name in ("kexact", "vexact"):
                        new[name].view(-1, TILE * HEAD_DIM)[dst_t] = old[name].view(-1, TILE * HEAD_DIM)[src_t]
                new["seg_count"][li].copy_(old["seg_count"][li])
        self._bufs = new
        self._seg_tile = seg_tile
        self._exact_room = None
        self._make_struct()

    # ------------------------------------------------------------------ validation
    def _validate_shapes(self, keys: torch.Tensor, values: torch.Tensor, bits: Optional[torch.Tensor]) -> None:
        if keys.shape != values.shape:
            raise ValueError(f"Mismatched key/value shapes: {keys.shape} vs {values.shape}")
        if keys.dim() != 4:
            raise ValueError(f"Expected keys/values with shape [B, H, T, D], got {keys.shape}")
        if bits is not None and tuple(bits.shape) != tuple(keys.shape[:3]):
            raise ValueError(f"Expected bits shape {tuple(keys.shape[:3])}, got {tuple(bits.shape)}")
        if keys.shape[-1] != self.head_dim:
            raise ValueError(f"Expected head_dim {self.head_dim}, got {keys.shape[-1]}")
        _lib.require_gpu(keys, "keys")
        _lib.require_gpu(values, "values")
        if self.batch_size == 0:
            self.batch_size = int(keys.shape[0])
            self.num_heads = int(keys.shape[1])
            self._nseg = self.batch_size * self.num_heads
            self._counts = np.zeros((5, self._nseg), np.int64)
        elif self.batch_size != int(keys.shape[0]) or self.num_heads != int(keys.shape[1]):
            raise ValueError(
                f"Adaptive backend state shape changed from (B={self.batch_size}, H={self.num_heads}) "
                f"to (B={keys.shape[0]}, H={keys.shape[1]})")

    @staticmethod
    def _rows_ok(t: torch.Tensor) -> bool:
        align = 4 if t.dtype == torch.float32 else 8
        return (t.stride(-1) == 1 and all(s % align == 0 for s in t.stride()[:-1])
                and t.stride(2) >= t.shape[-1] and t.data_ptr() % 16 == 0)

    # ------------------------------------------------------------------ writes
    def prefill(self, keys: torch.Tensor, values: torch.Tensor, bits: torch.Tensor) -> None:
        self._reset()
        self.append(keys, values, bits)

    def append(self, keys: torch.Tensor, values: torch.Tensor, bits: torch.Tensor,
               _pos_offset: Optional[int] = None, _known_counts: Optional[np.ndarray] = None) -> None:
        """_known_counts (int [B*H, 6], levels 0, 2, 3, 4, 8, 16): what odmkv_level_counts would return for `bits`,
        when the caller knows it without looking (levels assigned by rank with fixed shares): no read-back."""
        self._validate_shapes(keys, values, bits)
        B, H, T, D = keys.shape
        if T == 0:
            return
        dev = self.device
        bits = bits.to(device=dev, dtype=torch.int32).contiguous()
        if not self._rows_ok(keys):
            keys = keys.contiguous()
        if not self._rows_ok(values) or values.stride() != keys.stride():
            values = values.contiguous()
            keys = keys.contiguous()
        st = _lib.stream_ptr(dev)
        fresh = self._bufs is None and getattr(self, "_arena", None) is None       # the store's first tokens
        hint_key = (str(dev), self._nseg, T)
        pos_offset = self.seq_len if _pos_offset is None else int(_pos_offset)
        ws_bytes = lib.odmkv_pack_workspace_bytes(B, H, T)
        # The first fill of a store does not wait for the level counts: the tokens are quantised into a staging store
        # laid out for the worst case while the counts travel and the host lays the store out; the tiles are moved after.
        staged = (self._bufs is None and _known_counts is None and _pos_offset is None and T >= 4 * TILE
                  and _Staging.bytes_needed(self._nseg, T) <= _STAGING_LIMIT)
        # A staged first fill keeps its level map (one byte per token) behind the store, in the same allocation: a tensor
        # of its own would now and then make the allocator open a new segment (a device allocation, 0.2 ms of host time)
        # between this call's kernels.
        lm_bytes = (B * H * T + 255) & ~255 if staged else 0
        stg = None
        if _known_counts is not None:
            counts = np.asarray(_known_counts, np.int64).reshape(self._nseg, 6)
        elif staged:
            n_chunks = lib.odmkv_pack_count_chunks(T)                 # the counts arrive chunk by chunk
            box, box_dev, arrived, arrived_handle = _mailbox(dev, st, self._nseg * n_chunks * 6)
            arrived.synchronize()                                     # (the last reader of the box is long done)
            stg = _staging_for(dev, st, B, H, T, self._exact_torch_dtype)
            ws = _lib.workspace(dev, ws_bytes, "pack")
            lay = stg.layout
            _lib.check(lib.odmkv_quant_pack_staged(
                keys.data_ptr(), values.data_ptr(), _lib.dtype_code(keys), B, H, T,
                keys.stride(0), keys.stride(1), keys.stride(2), bits.data_ptr(), pos_offset,
                self.pi_k.data_ptr(), self.pi_v.data_ptr(), self.codebooks.data_ptr(),
                C.byref(stg.packed), stg.bufs.arena.data_ptr(), lay.tables_ptr, C.addressof(lay.offsets),
                lay.tables_end, lay.counts_end, box_dev.data_ptr(), box.data_ptr(), arrived_handle,
                ws.data_ptr(), ws_bytes, st))
            if fresh and hint_key in _ARENA_HINT:
                self._arena = torch.empty(_ARENA_HINT[hint_key], dtype=torch.uint8, device=dev)
            arrived.synchronize()                                     # the one wait: for the counts alone
            # what remains up to the launch of the gather is one call (the GPU has the quantiser's run to wait for it)
            new_lay, new_packed, counts32 = _Layout.blank(self._nseg), Packed(), np.zeros((self._nseg, 6), np.int32)
            need = C.c_uint64(0)
            for attempt in (0, 1):
                arena = getattr(self, "_arena", None)
                rc = lib.odmkv_store_finish_staged(
                    box.data_ptr(), n_chunks, B, H, T, int(self.exact_slack), int(self.quant_headroom),
                    _lib.BF16 if self._exact_torch_dtype == torch.bfloat16 else _lib.F16,
                    None if arena is None else arena.data_ptr(), 0 if arena is None else max(arena.numel() - lm_bytes, 0),
                    C.byref(stg.packed), counts32.ctypes.data, new_lay.tables_ptr, new_lay.offsets, new_lay.sizes,
                    new_lay.marks, C.byref(new_packed), C.byref(need), st)
                if rc != -2 or attempt == 1:
                    break
                self._arena = torch.empty(int(need.value) + int(need.value) // 8 + lm_bytes, dtype=torch.uint8, device=dev)
                self._arena_spare = None
            _lib.check(rc)
            counts = counts32.astype(np.int64)
        else:
            counts_dev = torch.empty(self._nseg, 6, dtype=torch.int32, device=dev)
            _lib.check(lib.odmkv_level_counts(bits.data_ptr(), B, H, T, counts_dev.data_ptr(), st))
            if fresh and hint_key in _ARENA_HINT:
                # while the counts are on their way: room for a store the size of the last one of this shape (a
                # layer's store is about as large as its neighbour's).  A new device allocation costs as much as
                # packing the layer; here it runs beside the kernels still in the queue.  Too small a guess is
                # replaced in _alloc.
                self._arena = torch.empty(_ARENA_HINT[hint_key], dtype=torch.uint8, device=dev)
            counts = counts_dev.cpu().numpy().astype(np.int64)        # the one synchronisation
        if int(counts.sum()) != self._nseg * T:
            raise ValueError("bits must take values in (0, 2, 3, 4, 8, 16)")
        present = {lvl for lvl, c in zip(_lib.LEVEL_ORDER, counts.sum(axis=0)) if c > 0}
        if not present <= set(self.bit_levels):
            raise ValueError(f"bits use levels {sorted(present - set(self.bit_levels))} outside bit_levels={self.bit_levels}")
        new_counts = self._counts + counts[:, 1:].T
        if stg is not None:
            # laid out, prepared and filled by odmkv_store_finish_staged above
            self._bufs = _Buffers(self._arena, new_lay.adopt(), self._exact_torch_dtype)
            self._seg_tile = new_lay.tables.astype(np.int64)
            self._packed = new_packed
        else:
            self._ensure_capacity(new_counts)
        if fresh:
            _ARENA_HINT[hint_key] = self._arena.numel()
        if stg is None:
            ws = _lib.workspace(dev, ws_bytes, "pack")
            _lib.check(lib.odmkv_quant_pack(
                keys.data_ptr(), values.data_ptr(), _lib.dtype_code(keys), B, H, T,
                keys.stride(0), keys.stride(1), keys.stride(2), bits.data_ptr(), pos_offset,
                self.pi_k.data_ptr(), self.pi_v.data_ptr(), self.codebooks.data_ptr(),
                C.byref(self._packed), ws.data_ptr(), ws_bytes, st))
        self._counts = new_counts
        self._exact_room = None
        if stg is not None:
            lm = self._arena[self._arena.numel() - lm_bytes:][:B * H * T].view(B, H, T)
            lm.copy_(bits)
        else:
            lm = bits.to(torch.uint8)
        if _pos_offset is None:
            self._extend_levels(lm, owned=True)
            self.seq_len += T
        else:
            self._level_store[:, :, pos_offset:pos_offset + T] = lm
        if not (_known_counts is not None and _pos_offset is not None and int(counts[:, 0].sum()) == 0):
            self._masked = None           # (a re-store without evictions leaves the evicted set as it was)
        self._items = None

    def append_all_exact(self, keys: torch.Tensor, values: torch.Tensor) -> None:
        """Every new token goes to the exact (16-bit) segments."""
        self._validate_shapes(keys, values, None)
        B, H, T, D = keys.shape
        if T == 0:
            return
        if T > 1 or self._bufs is None or keys.dtype != self._exact_torch_dtype:
            bits = torch.full((B, H, T), 16, dtype=torch.int32, device=self.device)
            self.append(keys, values, bits)
            return
        had = self._seg_tile
        room = self._exact_room
        new_counts = None
        if room is None or room <= 0:
            new_counts = self._counts.copy()
            new_counts[4] += 1
            self._ensure_capacity(new_counts)
            # tokens every exact segment can still take before a tile has to be added (the usual decode step
            # then skips the capacity arithmetic)
            room = int((np.diff(self._seg_tile[4]) * TILE - new_counts[4]).min()) + 1
        # the token is read where it lies (the newest row of the model's cache): no staging copies
        k, v = keys[:, :, 0, :], values[:, :, 0, :]
        if k.stride(2) != 1 or v.stride() != k.stride():
            k, v = k.contiguous(), v.contiguous()
        _lib.check(lib.odmkv_append_exact(C.byref(self._packed), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1),
                                          self.seq_len, _lib.stream_ptr(self.device)))
        if new_counts is None:
            self._counts[4] += 1
        else:
            self._counts = new_counts
        self._exact_room = room - 1
        if self._level_store.shape[2] < self.seq_len + 1:
            self._extend_levels(torch.full((B, H, 1), 16, dtype=torch.uint8, device=self.device))
        # otherwise nothing to write: the level store reads 16 behind seq_len (an exact token leaves
        # the evicted set as it is)
        self.seq_len += 1
        if had is not self._seg_tile:
            self._items = None

    def truncate(self, seq_len: int) -> None:
        seq_len = int(seq_len)
        if seq_len >= self.seq_len:
            return
        self._level_store[:, :, seq_len:self.seq_len].fill_(16)       # the store reads 16 behind seq_len
        self.seq_len = seq_len
        self._masked = None
        # positions ascend inside a segment, so the survivors are a prefix of it
        for li in range(5):
            if self._counts[li].sum() == 0:
                continue
            pos = self._bufs["pos"][li].cpu().numpy()
            for s in range(self._nseg):
                c = int(self._counts[li, s])
                if c:
                    first = int(self._seg_tile[li, s]) * TILE
                    self._counts[li, s] = int(np.searchsorted(pos[first:first + c], seq_len, side="left"))
                    self._exact_room = None
            self._bufs["seg_count"][li].copy_(torch.from_numpy(self._counts[li].astype(np.int32)))
        self._items = None

    # ------------------------------------------------------------------ reads
    def _dequant_into(self, keys: torch.Tensor, values: torch.Tensor, include_exact: bool, start: int = 0) -> None:
        if self._bufs is None:
            return
        if not (self._rows_ok(keys) and self._rows_ok(values) and keys.stride() == values.stride()):
            raise ValueError("materialisation targets must be row-contiguous [B, H, T, D] tensors with equal strides")
        _lib.check(lib.odmkv_dequant_from(
            C.byref(self._packed), keys.data_ptr(), values.data_ptr(), _lib.dtype_code(keys),
            int(start), int(keys.shape[2]), keys.stride(0), keys.stride(1), keys.stride(2),
            self.pi_k.data_ptr(), self.pi_v.data_ptr(), self.codebooks.data_ptr(),
            1 if include_exact else 0, _lib.stream_ptr(self.device)))

    def materialize(self, dtype: torch.dtype | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """Dense (keys, values) of the whole store in the state's dtype, as the reference returns them; `dtype`
        (an addition) asks for another one: float32 keeps the dequantised values unrounded."""
        keys = torch.zeros(self.batch_size, self.num_heads, self.seq_len, self.head_dim,
                           device=self.device, dtype=self.dtype if dtype is None else dtype)
        values = torch.zeros_like(keys)
        self._dequant_into(keys, values, True)
        return keys, values

    def materialize_quantized_into(self, keys: torch.Tensor, values: torch.Tensor, start: int = 0) -> None:
        """Overwrite the quantised positions of existing dense tensors; exact and evicted
        positions are left as they are.  `start` (an addition): only positions >= start."""
        self._dequant_into(keys, values, False, start)

    def masked_key_indices(self):
        """Indices (b, h, t) of the evicted positions, or None when there are none.  The answer is
        kept until positions are stored with levels again (exact appends cannot evict)."""
        if self._level_store is None:
            return None
        if self._masked is None:
            idx = (self._level_map == 0).nonzero(as_tuple=True)
            self._masked = (idx if idx[0].numel() else None,)
        return self._masked[0]

    def visible_mask(self) -> torch.Tensor:
        return self._level_map != 0

    def level_counts(self) -> dict[int, int]:
        out = {b: int(self._counts[_LEVEL_INDEX[b]].sum()) for b in (2, 3, 4, 8, 16)}
        out[0] = self.batch_size * self.num_heads * self.seq_len - sum(out.values())
        return out

    def packed_bytes(self) -> int:
        """Bytes the fused decode kernel has to read: codes + norms of the quantised tokens and the
        fp16 rows of the exact ones (positions and segment tables are not read by it)."""
        total = int(self._counts[4].sum()) * 2 * HEAD_DIM * 2
        for li, w in enumerate(WIDTHS):
            total += int(self._counts[li].sum()) * (2 * w * HEAD_DIM // 8 + 8)
        return total

    # ------------------------------------------------------------------ decode buffer
    def _exact_rows(self, start: int):
        """(positions [N,3] long, keys [N,D], values [N,D]) of exact tokens at positions >= start,
        ordered by (batch, head, position)."""
        if self._bufs is None or self._counts[4].sum() == 0:
            return None
        pos = self._bufs["pos"][4]
        slots, bh = [], []
        pos_host = pos.cpu().numpy()
        for s in range(self._nseg):
            c = int(self._counts[4, s])
            first = int(self._seg_tile[4, s]) * TILE
            k = int(np.searchsorted(pos_host[first:first + c], start, side="left"))
            slots.append(np.arange(first + k, first + c))
            bh.append(np.full(c - k, s))
        slots = np.concatenate(slots)
        if slots.size == 0:
            return None
        bh = np.concatenate(bh)
        # element (slot, dim) of tile t sits at t * 8192 + index table[slot % 64, dim]
        base = torch.from_numpy((slots // TILE) * (TILE * HEAD_DIM)).to(self.device)[:, None]
        kidx = base + torch.from_numpy(_EXACT_K_IDX[slots % TILE]).to(self.device)
        vidx = base + torch.from_numpy(_EXACT_V_IDX[slots % TILE]).to(self.device)
        krows = self._bufs["kexact"].view(-1)[kidx]
        vrows = self._bufs["vexact"].view(-1)[vidx]
        p3 = np.stack([bh // self.num_heads, bh % self.num_heads, pos_host[slots]], axis=-1).astype(np.int64)
        return torch.from_numpy(p3).to(self.device), krows, vrows

    def get_buffer_tokens(self, buffer_start_seq: int):
        got = self._exact_rows(int(buffer_start_seq))
        if got is None:
            empty = torch.empty(0, self.head_dim, device=self.device, dtype=self.dtype)
            return _empty_positions(self.device), empty, empty.clone()
        return got

    def exact_tail(self, n_tail: int):
        """(keys, values) [B, H, n_tail, D] of the store's exact dtype: the newest n_tail tokens of every exact
        segment, oldest first, in one launch and without reading anything back (the host's own mirror of the
        segment lengths says whether every segment holds that many); None otherwise."""
        n_tail = int(n_tail)
        if self._bufs is None or n_tail <= 0 or int(self._counts[4].min()) < n_tail:
            return None
        k = torch.empty(self.batch_size, self.num_heads, n_tail, self.head_dim, dtype=self._exact_torch_dtype, device=self.device)
        v = torch.empty_like(k)
        _lib.check(lib.odmkv_exact_tail(C.byref(self._packed), n_tail, k.data_ptr(), v.data_ptr(), _lib.stream_ptr(self.device)))
        return k, v

    def flush_buffer(self, buffer_start_seq: int, new_bits: torch.Tensor, rows=None, known_counts=None) -> None:
        """Re-quantise the exact tokens at positions >= buffer_start_seq to `new_bits` (one entry
        per token, in the order `get_buffer_tokens` returns them).  `rows` = (keys, values) [B, H, n, D] as
        `exact_tail` returned them for the same tokens and `known_counts` (see `append`) spare the gather and the
        read-back."""
        start = int(buffer_start_seq)
        n_buf = self.seq_len - start
        B, H = self.batch_size, self.num_heads
        if rows is not None:
            k, v = rows
            if tuple(k.shape) != (B, H, n_buf, self.head_dim):
                raise ValueError("flush_buffer: rows do not cover the positions >= buffer_start_seq")
        else:
            got = self._exact_rows(start)
            if got is None:
                return
            pos3, krows, vrows = got
            if pos3.shape[0] != self._nseg * n_buf:
                raise ValueError("flush_buffer expects every position >= buffer_start_seq to be exact in every head")
            k = krows.reshape(B, H, n_buf, self.head_dim).contiguous()
            v = vrows.reshape(B, H, n_buf, self.head_dim).contiguous()
        bits = new_bits.to(device=self.device, dtype=torch.int32).reshape(B, H, n_buf)
        # drop the buffered tokens from the exact segments, then append them at their new levels
        self._counts[4] -= n_buf
        self._exact_room = None
        self._bufs["seg_count"][4].copy_(torch.from_numpy(self._counts[4].astype(np.int32)))
        self.append(k, v, bits, _pos_offset=start, _known_counts=known_counts)

    # ------------------------------------------------------------------ fused attention
    def _build_items(self, target_items: Optional[int] = None, min_item_bytes: Optional[int] = None) -> None:
        """The decode work list: every (segment, level) run of tiles cut into items of about equal
        cost, one workgroup (one compute unit) per item.

        The cost of a tile is what the kernel was measured to need for it per level (the 2-bit loop is
        bound by instruction issue, the wider ones and the exact rows by memory), plus a fixed part per item.
        With a target the cut is the coarsest one that does not exceed it.  Without one, a few cuts
        are compared by the time a longest-first assignment of their items to the compute units
        would take, and the best is kept; when it has more items than compute units, the order in which
        the workgroups take the items (longest first) is handed to the kernel as well.  Items of sixteen
        tiles and more on average are run by sixteen (or twelve) wavefronts, shorter ones by eight.  A list
        with more items than compute units is cut for two eight-wavefront workgroups per compute unit
        (`two_per_cu`), as chains of a pair's levels where the runs alone are many more than those places."""
        import os
        n_cu = _compute_units(self.device)
        env_target = int(os.environ.get("ODMKV_DECODE_ITEMS", 0))
        min_item_bytes = int(os.environ.get("ODMKV_DECODE_MIN_ITEM_BYTES", 16384)) if min_item_bytes is None else min_item_bytes
        used = (self._counts + TILE - 1) // TILE
        used[4] = np.diff(self._seg_tile[4])              # exact segments grow between rebuilds
        total_bytes = sum(int(used[li].sum()) * _TILE_BYTES[li] for li in range(5))
        total = sum(int(used[li].sum()) * _TILE_COST[li] for li in range(5))      # cost units: nanoseconds of one compute unit
        min_item_bytes = min_item_bytes * _TILE_COST[0] // _TILE_BYTES[0]          # the same floor, as a cost
        # the runs of tiles, segment by segment (the merge finds a segment's items next to each other), as arrays
        run_li, run_s = np.nonzero(used.T > 0)[1], np.nonzero(used.T > 0)[0]
        run_nt = used[run_li, run_s].astype(np.int64)
        run_t0 = self._seg_tile[run_li, run_s].astype(np.int64)
        run_cnt = self._counts[run_li, run_s].astype(np.int64)
        tile_cost = np.asarray(_TILE_COST, np.float64)

        def steps_of(per_item: int) -> np.ndarray:                     # tiles per item, by level
            return np.maximum(1, np.rint(per_item / tile_cost).astype(np.int64))

        def n_pieces(per_item: int) -> int:
            step = steps_of(per_item)[run_li]
            return int((-(-run_nt // step)).sum())

        def fit(target: int) -> int:
            # the coarsest cut with at most `target` items (a run's last piece may be short)
            per_item = max(total // max(target, 1), min_item_bytes)
            while n_pieces(per_item) > target and per_item < total:
                per_item += max(per_item // 64, 1)
            return per_item

        def cut(per_item: int) -> np.ndarray:
            # rows (segment, level, first tile, tiles, tokens in those tiles, segment's first tile, -, -)
            step = steps_of(per_item)[run_li]
            pieces = -(-run_nt // step)
            run = np.repeat(np.arange(run_nt.size), pieces)
            a0 = (np.arange(run.size) - np.repeat(np.cumsum(pieces) - pieces, pieces)) * step[run]
            n = np.minimum(step[run], run_nt[run] - a0)
            out = np.zeros((run.size, 8), np.int64)
            out[:, 0], out[:, 1], out[:, 2], out[:, 3] = run_s[run], run_li[run], run_t0[run] + a0, n
            out[:, 4], out[:, 5] = np.minimum(run_cnt[run] - a0 * TILE, n * TILE), run_t0[run]
            return out

        # -- chains: the quantised levels of a segment as ONE run of work, cut into pieces of equal cost; a piece that
        # crosses a level boundary becomes consecutive items of one workgroup (one query rotation, one result)
        qr = run_li < 4
        q_s, q_li, q_nt, q_t0, q_cnt = run_s[qr], run_li[qr], run_nt[qr], run_t0[qr], run_cnt[qr]
        q_cost = q_nt * tile_cost[q_li]
        q_end = np.cumsum(q_cost)
        q_start = q_end - q_cost
        seg_cost = np.bincount(q_s, q_cost, minlength=self._nseg) if q_s.size else np.zeros(self._nseg)
        seg_start = np.cumsum(seg_cost) - seg_cost
        q_first = np.ones(q_s.size, bool)
        q_first[1:] = q_s[1:] != q_s[:-1]                               # a segment's first quantised run

        def chain_pieces(per_item: int) -> np.ndarray:                  # workgroups per segment
            return np.ceil(seg_cost / max(per_item, 1)).astype(np.int64)

        def cut_exact(per_item: int) -> np.ndarray:
            keep = run_li == 4
            step = steps_of(per_item)[4]
            nt, t0 = run_nt[keep], run_t0[keep]
            pieces = -(-nt // step)
            run = np.repeat(np.arange(nt.size), pieces)
            a0 = (np.arange(run.size) - np.repeat(np.cumsum(pieces) - pieces, pieces)) * step
            n = np.minimum(step, nt[run] - a0)
            out = np.zeros((run.size, 8), np.int64)
            out[:, 0], out[:, 1], out[:, 2], out[:, 3] = run_s[keep][run], 4, t0[run] + a0, n
            out[:, 4], out[:, 5] = np.minimum(run_cnt[keep][run] - a0 * TILE, n * TILE), t0[run]
            return out

        def cut_chained(per_item: int) -> np.ndarray:
            # rows as in cut(), word 6 = items that follow in the same workgroup, word 7 = 1 for those items
            k = chain_pieces(per_item)
            nb = np.maximum(k - 1, 0)
            b_s = np.repeat(np.arange(self._nseg), nb)                  # one row per inner piece boundary
            b_j = np.arange(b_s.size) - np.repeat(np.cumsum(nb) - nb, nb) + 1
            x = seg_start[b_s] + b_j * seg_cost[b_s] / k[b_s]           # where the boundary lies on the line of all runs' cost
            run = np.minimum(np.searchsorted(q_end, x, side="right"), q_s.size - 1)
            off = np.clip(np.rint((x - q_start[run]) / tile_cost[q_li[run]]).astype(np.int64), 0, q_nt[run])
            at_end = off == q_nt[run]                                   # a boundary on a run's end belongs to the next run's start
            run, off = np.where(at_end, np.minimum(run + 1, q_s.size - 1), run), np.where(at_end, 0, off)
            # the items' starts: every run's first tile, and the boundaries inside runs
            st_run = np.concatenate([np.arange(q_s.size), run])
            st_off = np.concatenate([np.zeros(q_s.size, np.int64), off])
            st_head = np.concatenate([q_first, np.ones(run.size, bool)])  # starts a workgroup's chain
            order_ = np.lexsort((~st_head, st_off, st_run))             # duplicates: the one that starts a chain first
            st_run, st_off, st_head = st_run[order_], st_off[order_], st_head[order_]
            uniq = np.ones(st_run.size, bool)
            uniq[1:] = (st_run[1:] != st_run[:-1]) | (st_off[1:] != st_off[:-1])
            st_run, st_off, st_head = st_run[uniq], st_off[uniq], st_head[uniq]
            nxt = np.append(st_off[1:], 0)
            last_of_run = np.append(st_run[1:] != st_run[:-1], True)
            n = np.where(last_of_run, q_nt[st_run], nxt) - st_off
            out = np.zeros((st_run.size, 8), np.int64)
            out[:, 0], out[:, 1], out[:, 2], out[:, 3] = q_s[st_run], q_li[st_run], q_t0[st_run] + st_off, n
            out[:, 4], out[:, 5] = np.minimum(q_cnt[st_run] - st_off * TILE, n * TILE), q_t0[st_run]
            head_idx = np.flatnonzero(st_head)
            follow = np.diff(np.append(head_idx, st_run.size)) - 1
            out[head_idx, 6] = follow
            out[:, 7] = ~st_head
            both = np.concatenate([out, cut_exact(per_item)])
            return both[np.lexsort((both[:, 2], both[:, 1] & 7, both[:, 0]))]

        def fit_chained(target: int) -> int:
            per_item = max(total // max(target, 1), min_item_bytes)
            n_exact = lambda p: int((-(-run_nt[run_li == 4] // steps_of(p)[4])).sum())
            while int(chain_pieces(per_item).sum()) + n_exact(per_item) > target and per_item < total:
                per_item += max(per_item // 64, 1)
            return per_item

        def cost(items: np.ndarray, fixed: float = _ITEM_FIXED_US) -> np.ndarray:
            # microseconds of one workgroup, roughly: per workgroup (an item with word 7 set adds to the one before it)
            own = items[:, 3] * tile_cost[items[:, 1] & 7] * 1e-3
            head = items[:, 7] == 0
            group = np.cumsum(head) - 1
            return (fixed + np.bincount(group, own, minlength=int(head.sum()))
                    + _CHAIN_LINK_US * items[head, 6] + np.where(items[head, 6] > 0, _CHAIN_ROTATE_US, 0.0))

        def makespan(items: np.ndarray, fixed: float = _ITEM_FIXED_US) -> float:
            import heapq
            free = [0.0] * n_cu
            for c in sorted(cost(items, fixed).tolist(), reverse=True):
                heapq.heappush(free, heapq.heappop(free) + c)
            return max(free)

        chain_env = os.environ.get("ODMKV_DECODE_CHAINS")                # "0": never, "1": always (measurements)
        pair_env = os.environ.get("ODMKV_DECODE_PAIRS")                  # the same for two workgroups per compute unit
        may_chain = q_s.size > 0 and bool((~q_first).any()) and chain_env != "0"
        explicit = target_items if target_items is not None else (env_target or None)
        paired = pair_env == "1"
        if explicit is not None:
            items = cut_chained(fit_chained(int(explicit))) if (may_chain and chain_env == "1") else cut(fit(int(explicit)))
        else:
            # the comparison is repeated only when the store has grown by more than 5 % since the
            # last one (a decode-time flush adds a fraction of a percent): until then its winner is re-cut
            chosen = self._items_choice
            if chosen is not None and abs(total_bytes - chosen[1]) <= 0.05 * chosen[1]:
                items = (cut_chained(fit_chained(int(n_cu * chosen[0]))) if chosen[2] and may_chain
                         else cut(fit(int(n_cu * chosen[0]))))
                paired = chosen[3]
            else:
                best = None
                if chain_env != "1" or not may_chain:
                    for mult in (1.0, 1.5, 2.0, 3.0, 4.0):
                        cand = cut(fit(int(n_cu * mult)))
                        t = makespan(cand)
                        if best is None or t < best[0] - 1e-9:
                            best = (t, cand, mult, False)
                n_pairs = int(q_first.sum())
                n_exact = int((run_li == 4).sum())
                if pair_env != "0" and (paired or (best is not None and len(best[1]) > n_cu)):
                    # More items than compute units: the workgroups would run in rounds, each paying its start (work item,
                    # rotation, table, first bytes: about 4 us) and its end (combine) with the compute unit to itself.
                    # Two eight-wavefront workgroups per compute unit overlap one's start and end with the other's
                    # stream (measured: a 16 x 8192-token batch 28.1 -> 25.9 us, 64 x 2048 tokens 52 -> 40 us; lists of
                    # one item per compute unit lose 5-10 %, and keep the wide workgroups).  Cut for one round of the
                    # 2 x n_cu places; where the runs alone are many more than that, chain a pair's levels instead.
                    paired = True
                    if may_chain and (chain_env == "1" or q_s.size + n_exact > _PAIR_CHAIN_RUNS_PER_PLACE * 2 * n_cu):
                        mult = max(2.0, (n_pairs + n_exact) / n_cu)
                        best = (0.0, cut_chained(fit_chained(int(n_cu * mult))), mult, True)
                    else:
                        best = (0.0, cut(fit(2 * n_cu)), 2.0, False)
                elif may_chain and (chain_env == "1" or (q_s.size >= _CHAIN_RUNS_PER_CU * n_cu
                                                         and q_s.size >= _CHAIN_RUNS_PER_PAIR * n_pairs)):
                    mult = max(1.5, (n_pairs + n_exact) / n_cu)
                    best = (0.0, cut_chained(fit_chained(int(n_cu * mult))), mult, True)
                items = best[1]
                self._items_choice = (best[2], total_bytes, best[3], paired)
        arr = items.astype(np.int32).reshape(-1, 8)
        per_seg = np.bincount(arr[:, 0], minlength=self._nseg) if len(items) else np.zeros(self._nseg, np.int64)
        ranges = np.concatenate([[0], np.cumsum(per_seg)])          # items are generated in segment order
        order = None
        heads = np.flatnonzero(arr[:, 7] == 0) if len(items) else np.zeros(0, np.int64)
        chained = len(items) > 0 and heads.size != len(items)
        paired = paired and len(items) > 0
        if len(items) > n_cu or chained or paired:
            # the workgroups' first items, longest workgroup first
            order = heads[np.argsort(-cost(items), kind="stable")].astype(np.int32)
            if paired and order.size > n_cu:
                # two per compute unit: the first n_cu workgroups land one per compute unit, the next n_cu beside them in
                # the same order of compute units; taken shortest first, the shortest joins the longest (a 16 x 8192-token
                # batch 26.0 -> 25.5 us; long and short alternating: 32 us)
                order = np.concatenate([order[:n_cu], order[n_cu:2 * n_cu][::-1], order[2 * n_cu:]]).astype(np.int32)
        # one upload for the item table, the ranges and the order (the parts start at multiples of 4 integers)
        n_arr, n_rng = arr.size, (ranges.size + 3) & ~3
        blob = np.zeros(n_arr + n_rng + (0 if order is None else order.size), np.int32)
        blob[:n_arr] = arr.reshape(-1)
        blob[n_arr:n_arr + ranges.size] = ranges
        if order is not None:
            blob[n_arr + n_rng:] = order
        dev_blob = torch.from_numpy(blob).to(self.device)
        self._item_order = None if order is None else dev_blob[n_arr + n_rng:]
        self._items = (dev_blob[:n_arr].view(-1, 8), dev_blob[n_arr:n_arr + ranges.size], len(items))
        w = _lib.Worklist()
        w.items, w.item_range = self._items[0].data_ptr(), self._items[1].data_ptr()
        w.dispatch_order = _lib.ptr(self._item_order)
        w.n_items = len(items)
        w.n_workgroups = int(heads.size) if chained else 0
        # wavefronts per item: eight for short items (less set-up, a lighter combine); for long ones sixteen where
        # the narrow levels carry the bytes (their loop wants four wavefronts per SIMD) and twelve where 4- and 8-bit
        # tokens do (memory-bound: a third unit in flight per wavefront pays more than the fourth wavefront)
        if chained:                                                     # quantised tiles per workgroup
            qi = (arr[:, 1] & 7) < 4
            quant = np.bincount((np.cumsum(arr[:, 7] == 0) - 1)[qi], arr[qi, 3])
            quant = quant[quant > 0]
        else:
            quant = arr[arr[:, 1] < 4, 3] if len(items) else arr[:0, 3]
        q_bytes = [int(used[li].sum()) * _TILE_BYTES[li] for li in range(4)]
        wide = (q_bytes[2] + q_bytes[3]) >= 0.4 * max(sum(q_bytes), 1)
        # (items of 6 to 15 tiles that are mostly 3 bits and wider: twelve as well, 2-3 % ahead of eight, measured on
        # a 28-head, 3-bit store of 32k tokens: their loops wait on memory, and a third unit in flight pays)
        medium = bool(quant.size) and 6 <= quant.mean() < 16 and (sum(q_bytes) - q_bytes[0]) >= 0.5 * max(sum(q_bytes), 1)
        auto = (12 if medium else 8) if not (quant.size and quant.mean() >= 16) else (12 if wide else 16)
        w.wavefronts = 8 if paired else (int(os.environ.get("ODMKV_DECODE_WAVES", 0)) or auto)
        w.two_per_cu = int(paired)
        self._worklist = w

    def decode_attention_block(self, query: torch.Tensor, scaling: Optional[float] = None):
        """The same for a block of L query tokens per sequence that all see the whole store (the question after a
        prefill, a draft to verify): query [B, Hq, L, D] -> (out fp32 [B, Hq, L, D], lse fp32 [B, Hq, L]).

        The kernel's GQA sharing carries the block: the L tokens of a kv-head's G query heads are handed over as G * L
        heads of that kv-head, up to 8 per call, so the packed bytes are streamed once per 8 // G tokens instead of
        once per token (attention among the L tokens themselves is the caller's: see attention_patch)."""
        _lib.require_gpu(query, "query")
        if query.dim() != 4:
            raise ValueError(f"query must be [B, Hq, L, D], got {tuple(query.shape)}")
        B, Hq, L, D = query.shape
        H = self.num_heads
        if Hq % H:
            raise ValueError(f"{Hq} query heads do not divide over {H} kv heads")
        G = Hq // H
        if G > 8:
            raise ValueError(f"GQA group {G} exceeds 8")
        per = max(1, 8 // G)
        out = torch.empty(B, Hq, L, D, dtype=torch.float32, device=self.device)
        lse = torch.empty(B, Hq, L, dtype=torch.float32, device=self.device)
        q5 = query.reshape(B, H, G, L, D)
        for l0 in range(0, L, per):
            lc = min(per, L - l0)
            qv = q5[:, :, :, l0:l0 + lc].permute(0, 1, 3, 2, 4).reshape(B, H * lc * G, D).contiguous()
            o, s = self.decode_attention(qv, scaling=scaling, return_lse=True)
            out.view(B, H, G, L, D)[:, :, :, l0:l0 + lc] = o.view(B, H, lc, G, D).permute(0, 1, 3, 2, 4)
            lse.view(B, H, G, L)[:, :, :, l0:l0 + lc] = s.view(B, H, lc, G).permute(0, 1, 3, 2)
        return out, lse

    def decode_attention(self, query: torch.Tensor, scaling: Optional[float] = None,
                         return_lse: bool = False, out_dtype: torch.dtype = torch.float32):
        """softmax(scaling * q K^T) V over the stored tokens, for one query token per sequence.

        query: [B, Hq, D] or [B, Hq, 1, D] on the GPU, fp16 / bf16 / fp32 (read as it is); returns
        [B, Hq, D] of `out_dtype` (accumulated in fp32, rounded once) and, on request, lse fp32 [B, Hq]."""
        _lib.require_gpu(query, "query")
        if self._bufs is None:
            raise ValueError("the store is empty")
        q = query.reshape(query.shape[0], query.shape[1], self.head_dim)
        if q.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            q = q.float()
        q = q.contiguous()
        B, Hq, D = q.shape
        if B != self.batch_size or Hq % self.num_heads != 0:
            raise ValueError(f"query heads {tuple(q.shape)} do not match the store (B={self.batch_size}, Hkv={self.num_heads})")
        if self._items is None:
            self._build_items()
        items, ranges, n_items = self._items
        scale = 1.0 / math.sqrt(D) if scaling is None else float(scaling)
        out = torch.empty(B, Hq, D, dtype=out_dtype, device=self.device)
        lse = torch.empty(B, Hq, dtype=torch.float32, device=self.device) if return_lse else None
        ws_bytes = lib.odmkv_decode_workspace_bytes(B, Hq, n_items)
        ws = _lib.workspace(self.device, ws_bytes, "decode")
        _lib.check(lib.odmkv_decode_attn(
            q.data_ptr(), _lib.dtype_code(q), B, Hq, scale, C.byref(self._packed), C.byref(self._worklist),
            self._pi_k_ops.data_ptr(), self.pi_v.data_ptr(), self._decode_cb.data_ptr(),
            self._decode_cb_host, self._decode_inv, out.data_ptr(), _lib.dtype_code(out), _lib.ptr(lse), ws.data_ptr(), ws_bytes,
            _lib.stream_ptr(self.device)))
        return (out, lse) if return_lse else out

    def decode_step(self, query: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, scaling: Optional[float] = None,
                    out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """``append_all_exact(keys, values)`` (one new token, [B, Hkv, 1, D]) followed by ``decode_attention(query)``:
        what one layer does in one decode step under a press that buffers new tokens exact.  When the exact segments
        have room for the token (every step but the one in 64 that opens a tile) both run in one library call whose
        constant arguments are kept in a block per store and work list."""
        room = self._exact_room
        if (room is None or room <= 0 or self._bufs is None or keys.shape[2] != 1 or keys.dtype != self._exact_torch_dtype
                or self._level_store.shape[2] < self.seq_len + 1 or not query.is_contiguous()
                or query.dtype not in (torch.float16, torch.bfloat16, torch.float32)):
            self.append_all_exact(keys, values)
            return self.decode_attention(query, scaling=scaling, out_dtype=out_dtype)
        _lib.require_gpu(query, "query")
        self._validate_shapes(keys, values, None)
        B, Hq = query.shape[0], query.shape[1]
        if self._items is None:
            self._build_items()
        scale = 1.0 / math.sqrt(self.head_dim) if scaling is None else float(scaling)
        stream = _lib.stream_ptr(self.device)
        key = (Hq, query.dtype, out_dtype, scale, stream)
        blk = self._step
        if blk is None or blk[4] is not self._packed or blk[5] is not self._worklist or blk[0] != key:
            if B != self.batch_size or Hq % self.num_heads != 0 or query.numel() != B * Hq * self.head_dim:
                raise ValueError(f"query {tuple(query.shape)} does not match the store (B={self.batch_size}, Hkv={self.num_heads})")
            ws_bytes = lib.odmkv_decode_workspace_bytes(B, Hq, self._items[2])
            ws = _lib.workspace(self.device, ws_bytes, "decode")
            st = _lib.Step(C.pointer(self._packed), C.pointer(self._worklist), self._pi_k_ops.data_ptr(), self.pi_v.data_ptr(),
                           self._decode_cb.data_ptr(), self._decode_cb_host, self._decode_inv, ws.data_ptr(), ws_bytes, B, Hq,
                           _lib.dtype_code(query), _lib._DT[out_dtype], scale)
            blk = self._step = (key, st, C.byref(st), ws, self._packed, self._worklist)
        k, v = keys[:, :, 0, :], values[:, :, 0, :]
        if k.stride(2) != 1 or v.stride() != k.stride():
            k, v = k.contiguous(), v.contiguous()
        out = torch.empty(B, Hq, self.head_dim, dtype=out_dtype, device=self.device)
        _lib.check(lib.odmkv_decode_step(blk[2], query.data_ptr(), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1),
                                         self.seq_len, out.data_ptr(), None, stream))
        self._counts[4] += 1
        self._exact_room = room - 1
        self.seq_len += 1
        return out
