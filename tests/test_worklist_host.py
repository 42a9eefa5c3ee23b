"""CPU: how the decode work list is cut (TurboQuantAdaptiveKVCacheState._build_items), on segment tables made up here.

The cutter is host arithmetic over the store's tile counts; only its last step uploads the tables.  A state object is
put together without a GPU (device "cpu", 256 compute units assumed) and the lists are checked for what the kernels
rely on: every stored tile is covered exactly once, by items that stay inside one (sequence, kv-head, level) run;
chained items follow their workgroup's first item, in the same pair, with ascending levels; the dispatch order names
every workgroup's first item once; lists with more items than compute units ask for two workgroups per compute unit.
"""
import numpy as np
import pytest
import torch

TILE = 64


def _state(counts: np.ndarray, exact_capacity_tiles: int = 0):
    """A state with `counts` [5 levels, nseg] tokens per (level, segment) and nothing on a GPU."""
    from kvquant import tq_adaptive_backend as tq
    tq._CU_COUNT["cpu"] = 256
    st = tq.TurboQuantAdaptiveKVCacheState.__new__(tq.TurboQuantAdaptiveKVCacheState)
    st.device = torch.device("cpu")
    st._nseg = counts.shape[1]
    st._counts = counts.astype(np.int64)
    cap = (counts + TILE - 1) // TILE
    cap[4] = np.maximum(cap[4], exact_capacity_tiles)
    st._seg_tile = np.zeros((5, st._nseg + 1), np.int64)
    st._seg_tile[:, 1:] = np.cumsum(cap, axis=1)
    st._items = st._item_order = st._worklist = st._items_choice = None
    return st


def _check(st, n_cu=256):
    items = st._items[0].numpy().astype(np.int64)
    ranges = st._items[1].numpy()
    w = st._worklist
    assert w.n_items == len(items) == st._items[2]
    used = (st._counts + TILE - 1) // TILE
    used[4] = np.diff(st._seg_tile[4])
    # every stored tile once, inside its run
    for li in range(5):
        seen = np.zeros(int(st._seg_tile[li, -1]), np.int32)
        for bh, lv, t0, nt, ntok, seg0, follow, cont in items[(items[:, 1] & 7) == li]:
            assert seg0 == st._seg_tile[li, bh] and t0 >= seg0 and t0 + nt <= seg0 + used[li, bh] and nt > 0
            assert li == 4 or 0 < ntok <= nt * TILE          # (exact items: the kernel reads the segment's count itself)
            seen[t0:t0 + nt] += 1
        for s in range(st._nseg):
            a = int(st._seg_tile[li, s])
            assert (seen[a:a + used[li, s]] == 1).all() and (seen[a + used[li, s]:int(st._seg_tile[li, s + 1])] == 0).all()
    # a segment's items lie next to each other, and the ranges say where
    assert ranges[0] == 0 and ranges[-1] == len(items) and (np.diff(items[:, 0]) >= 0).all()
    for s in range(st._nseg):
        assert (items[ranges[s]:ranges[s + 1], 0] == s).all()
    heads = np.flatnonzero(items[:, 7] == 0)
    chained = heads.size != len(items)
    assert w.n_workgroups == (heads.size if chained else 0)
    for i in heads:
        chain = items[i:i + items[i, 6] + 1]
        assert (chain[1:, 7] == 1).all() and (chain[:, 0] == chain[0, 0]).all()
        if len(chain) > 1:
            assert ((chain[:, 1] & 7) < 4).all() and (np.diff(chain[:, 1] & 7) > 0).all() and len(chain) <= 4
    assert int((items[heads, 6] + 1).sum()) == len(items)
    if st._item_order is None:
        assert len(items) <= n_cu and not chained and w.two_per_cu == 0 and w.dispatch_order in (None, 0)
    else:
        assert sorted(st._item_order.numpy().tolist()) == heads.tolist()
    if w.two_per_cu:
        assert w.wavefronts == 8 and st._item_order is not None
    return items, heads


def test_one_long_sequence_gets_an_item_per_compute_unit():
    # 8 kv-heads x 32768 tokens, nearly all 2-bit (the 32k-token layer of the headline workload)
    counts = np.zeros((5, 8), np.int64)
    counts[0], counts[1], counts[4] = 32500, 136, 132
    st = _state(counts, exact_capacity_tiles=7)
    st._build_items()
    items, heads = _check(st)
    w = st._worklist
    assert 200 <= len(items) <= 256 and w.two_per_cu == 0 and w.n_workgroups == 0 and w.wavefronts == 16


def test_a_batch_with_two_levels_a_pair_runs_two_workgroups_per_compute_unit():
    # 16 sequences x 8 kv-heads, 75 tiles of 2 bits and 40 of 3 bits each, three exact tiles
    counts = np.zeros((5, 128), np.int64)
    counts[0], counts[1], counts[4] = 75 * TILE - 9, 40 * TILE - 30, 132
    st = _state(counts)
    st._build_items()
    items, heads = _check(st)
    w = st._worklist
    assert w.two_per_cu == 1 and w.n_workgroups == 0 and 256 < len(items) <= 640
    # the dispatch order: the 256 longest first, then the rest shortest first (the shortest joins the longest)
    order = st._item_order.numpy()
    cost = items[order, 3] * np.asarray([300, 420, 450, 890, 1310])[items[order, 1] & 7]
    assert (np.diff(cost[:256]) <= 0).all() and (np.diff(cost[256:512]) >= 0).all() and cost[255] >= cost[256:].max()


def test_a_batch_of_short_sequences_chains_the_levels_of_a_pair(monkeypatch):
    # 64 sequences x 8 kv-heads x 2048 tokens over four quantised levels and the exact rows
    rng = np.random.default_rng(3)
    counts = np.zeros((5, 512), np.int64)
    for s in range(512):
        counts[:, s] = rng.multinomial(1900, [0.55, 0.2, 0.15, 0.07, 0.03]) + np.array([0, 0, 0, 0, 132])
    counts[2, 5] = 0                                          # a pair without 4-bit tokens
    st = _state(counts)
    st._build_items()
    items, heads = _check(st)
    w = st._worklist
    assert w.two_per_cu == 1 and 0 < w.n_workgroups < len(items) and (items[:, 6] > 0).any()
    # the same store with pairs switched off: chains on wide workgroups; with both off: an item per run, at least
    monkeypatch.setenv("ODMKV_DECODE_PAIRS", "0")
    st._items_choice = None
    st._build_items()
    _check(st)
    assert st._worklist.two_per_cu == 0 and 0 < st._worklist.n_workgroups < st._worklist.n_items
    monkeypatch.setenv("ODMKV_DECODE_CHAINS", "0")
    st._items_choice = None
    st._build_items()
    items, _ = _check(st)
    assert st._worklist.n_workgroups == 0 and len(items) >= int((counts > 0).sum())


@pytest.mark.parametrize("target", [1, 7, 64, 300, 5000])
def test_explicit_targets_and_ragged_stores(target, monkeypatch):
    rng = np.random.default_rng(target)
    counts = rng.integers(0, 4000, size=(5, 6)).astype(np.int64)
    counts[:, 2] = 0                                          # a pair with no tokens at all
    counts[1:, 4] = 0                                         # a pair with one level only
    counts[4] = np.minimum(counts[4], 300)
    for chains in ("0", "1"):
        monkeypatch.setenv("ODMKV_DECODE_CHAINS", chains)
        st = _state(counts)
        st._build_items(target, 1)
        items, heads = _check(st)
        assert (items[:, 0] != 2).all()
