"""Pins for ``oracle.flush`` (decode-time compression of the token buffer,
reference: kvquant/adaptive_backend_press.py:198-290, 464-665) and the product's host logic for the
same step against it, on the CPU."""
import math

import numpy as np
import pytest
import torch

from oracle import flush as ofl
from oracle.scorer import risk_score_with_attn


def _buffer(seed, B=2, H=3, n=7, d=16, shuffle=True):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, H, n, d, generator=g)
    v = torch.randn(B, H, n, d, generator=g)
    bb, hh, tt = np.meshgrid(np.arange(B), np.arange(H), np.arange(n) + 100, indexing="ij")
    pos = np.stack([bb.ravel(), hh.ravel(), tt.ravel()], -1).astype(np.int64)
    flat_k, flat_v = k.reshape(-1, d), v.reshape(-1, d)
    if shuffle:                                            # the routine must not rely on the order
        perm = torch.randperm(pos.shape[0], generator=g).numpy()
        pos, flat_k, flat_v = pos[perm], flat_k[perm], flat_v[perm]
    return k, v, pos, flat_k, flat_v


def test_flush_attention_against_fp64_softmax_per_head():
    B, H, G, n, d = 2, 3, 4, 7, 16
    k, v, pos, fk, fv = _buffer(1, B, H, n, d)
    q = torch.randn(B, H * G, d, generator=torch.Generator().manual_seed(2))
    got = ofl.flush_attention(q, fk, pos, H)
    for b in range(B):
        for h in range(H):
            # group mean written as a loop over the heads of the group, softmax written out in fp64
            qm = sum(q[b, h * G + g].double() for g in range(G)) / G
            logit = np.array([float(qm @ k[b, h, t].double()) / math.sqrt(d) for t in range(n)])
            w = np.exp(logit - logit.max())
            w /= w.sum()
            for t in range(n):
                i = int(np.flatnonzero((pos[:, 0] == b) & (pos[:, 1] == h) & (pos[:, 2] == 100 + t))[0])
                assert abs(float(got[i]) - w[t]) < 1e-6
    # one weight distribution per (batch, head)
    sums = np.zeros((B, H))
    np.add.at(sums, (pos[:, 0], pos[:, 1]), got.numpy())
    np.testing.assert_allclose(sums, 1.0, atol=1e-5)
    # the mean over the group is taken before the dot product: G = 1 with the mean query gives the same
    qm = q.reshape(B, H, G, d).mean(2)
    torch.testing.assert_close(ofl.flush_attention(qm, fk, pos, H), got, rtol=1e-5, atol=1e-7)


def test_flush_scores_are_score_with_attn_per_head_then_minmax(golden):
    B, H, n, d = 2, 2, 9, 16
    k, v, pos, fk, fv = _buffer(3, B, H, n, d)
    q = torch.randn(B, H * 2, d, generator=torch.Generator().manual_seed(4))
    attn = ofl.flush_attention(q, fk, pos, H)
    got = ofl.flush_scores(fk, fv, attn, pos, H, epsilon=1e-2)
    raw = torch.empty(B, H, n)
    for b in range(B):
        for h in range(H):
            a = torch.stack([attn[int(np.flatnonzero((pos[:, 0] == b) & (pos[:, 1] == h) & (pos[:, 2] == 100 + t))[0])]
                             for t in range(n)])
            raw[b, h] = risk_score_with_attn(k[b, h:h + 1], v[b, h:h + 1], a[None], 1e-2)[0]
    want = (raw - raw.min()) / (raw.max() - raw.min())
    for i in range(pos.shape[0]):
        assert abs(float(got[i]) - float(want[pos[i, 0], pos[i, 1], pos[i, 2] - 100])) < 1e-6
    assert float(got.min()) == 0.0 and float(got.max()) == 1.0
    # the scorer itself is the golden-pinned one
    s = risk_score_with_attn(torch.from_numpy(golden["swa_k"]), torch.from_numpy(golden["swa_v"]),
                             torch.from_numpy(golden["swa_a"]))
    np.testing.assert_allclose(s.numpy(), golden["swa_out"], rtol=1e-6)
    # degenerate spread, and the two fallbacks
    assert (ofl.minmax(torch.full((5,), 3.0)) == 0.5).all()
    no_scorer = ofl.flush_scores(fk, fv, attn, pos, H, use_scorer=False)
    torch.testing.assert_close(no_scorer, ofl.minmax(attn.pow(2) * fv.pow(2).sum(-1)))
    norm_only = ofl.flush_scores(fk, fv, None, pos, H)
    torch.testing.assert_close(norm_only, ofl.minmax(fk.pow(2).sum(-1) + fv.pow(2).sum(-1)))


def test_record_observed_ratios_counts_the_bulk_only():
    bits = torch.tensor([[[16, 16, 2, 2, 2, 4, 0, 0, 8, 16, 16],
                          [16, 16, 3, 3, 3, 3, 3, 3, 3, 16, 16]]], dtype=torch.int32)
    got = ofl.record_observed_ratios(bits, sink_tokens=2, buffer_size=2)
    assert got[0] == ((0, 2 / 7), (2, 3 / 7), (4, 1 / 7), (8, 1 / 7)) or all(
        abs(a[1] - b[1]) < 1e-7 and a[0] == b[0] for a, b in zip(got[0], ((0, 2 / 7), (2, 3 / 7), (4, 1 / 7), (8, 1 / 7))))
    assert got[1][0][0] == 3 and abs(got[1][0][1] - 1.0) < 1e-7 and len(got[1]) == 1
    # sink + window cover everything: fall back to the whole row
    got = ofl.record_observed_ratios(bits[..., :3], sink_tokens=2, buffer_size=2)
    assert [b for b, _ in got[0]] == [2, 16]
    # the last batch row of a head wins
    two = torch.stack([bits[0], torch.full_like(bits[0], 4)])
    got = ofl.record_observed_ratios(two, sink_tokens=2, buffer_size=2)
    assert got[0] == ((4, 1.0),) and got[1] == ((4, 1.0),)


def test_cached_ratio_bits_one_head_is_the_golden_routine(golden):
    scores = torch.from_numpy(golden["ratio_scores"])               # [rows, n]
    levels, ratios = (2, 3, 4, 8, 16), (0.5, 0.2, 0.15, 0.1, 0.05)
    observed = {0: tuple(zip(levels, ratios))}
    for r in range(scores.shape[0]):
        n = scores.shape[1]
        pos = np.stack([np.zeros(n), np.zeros(n), np.arange(n)], -1).astype(np.int64)
        got = ofl.cached_ratio_bits(scores[r], pos, 1, observed, levels)
        assert (got.numpy() == golden["ratio_bits"][r]).all()


def test_cached_ratio_bits_drops_evicted_share_and_ranks_each_head_over_all_batch_rows():
    B, H, n = 2, 2, 10
    g = torch.Generator().manual_seed(5)
    scores = torch.rand(B * H * n, generator=g)
    bb, hh, tt = np.meshgrid(np.arange(B), np.arange(H), np.arange(n), indexing="ij")
    pos = np.stack([bb.ravel(), hh.ravel(), tt.ravel()], -1).astype(np.int64)
    observed = {0: ((0, 0.5), (2, 0.25), (4, 0.25)), 1: ((2, 0.2), (8, 0.8))}
    got = ofl.cached_ratio_bits(scores, pos, H, observed, (2, 3, 4, 8, 16)).numpy()
    # head 0: 0-bit share dropped, 2 and 4 bits renormalised to one half each over its 20 tokens
    h0 = pos[:, 1] == 0
    s0 = scores.numpy()[h0]
    order = np.argsort(s0, kind="stable")
    want0 = np.empty(20, np.int32)
    want0[order[:10]] = 2
    want0[order[10:]] = 4
    assert (got[h0] == want0).all()
    h1 = pos[:, 1] == 1
    assert sorted(got[h1].tolist()) == [2] * 4 + [8] * 16
    assert got[h1][np.argsort(scores.numpy()[h1], kind="stable")[:4]].tolist() == [2] * 4
    # with eviction allowed the 0-bit share stays
    got = ofl.cached_ratio_bits(scores, pos, H, observed, (0, 2, 3, 4, 8, 16)).numpy()
    assert sorted(got[h0].tolist()) == [0] * 10 + [2] * 5 + [4] * 5
    # a head without a record, or whose levels are all disallowed: no answer (the caller falls back)
    assert ofl.cached_ratio_bits(scores, pos, H, {0: observed[0]}, (2, 4)) is None
    assert ofl.cached_ratio_bits(scores, pos, H, {0: ((0, 1.0),), 1: observed[1]}, (2, 4, 8)) is None


def test_product_host_logic_matches_the_oracle_on_the_cpu():
    """The press's batched cached-ratio allocation and its share recording (device-agnostic torch
    code) against the oracle's loops."""
    from kvquant import RiskScorer
    from kvquant.adaptive_backend_press import TurboQuantPerTokenBackendPress
    press = TurboQuantPerTokenBackendPress(
        scorer=RiskScorer(n_future_positions=512, n_sink=4, epsilon=1e-2), key_quantizer="mse",
        value_quantizer="mse", bit_levels=(0, 2, 3, 4, 8, 16), target_avg_bits=2.0, sink_tokens=4, layerwise=True,
        buffer_size=16)
    g = torch.Generator().manual_seed(6)
    lv = torch.tensor((0, 2, 3, 4, 8, 16))
    bits = lv[torch.randint(0, 6, (2, 3, 200), generator=g)].int()
    press._record_observed_ratios(5, bits)
    want = ofl.record_observed_ratios(bits, 4, 16)
    for h in range(3):
        got = press._observed_ratios[(5, h)]
        assert [b for b, _ in got] == [b for b, _ in want[h]]
        np.testing.assert_allclose([r for _, r in got], [r for _, r in want[h]], rtol=1e-6)
    B, H, n = 2, 3, 16
    scores = torch.rand(B * H * n, generator=g)
    scores[5] = scores[40]                                           # a tie across batch rows of... some head
    bb, hh, tt = np.meshgrid(np.arange(B), np.arange(H), np.arange(n), indexing="ij")
    pos = np.stack([bb.ravel(), hh.ravel(), tt.ravel()], -1).astype(np.int64)
    allowed = (2, 3, 4, 8, 16)
    want_bits = ofl.cached_ratio_bits(scores, pos, H, want, allowed)
    for batch_size in (B, None):                                     # the one-sort path and the per-head loop
        got_bits = press._allocate_bits_via_cached_ratios(scores, torch.from_numpy(pos), H, 5, set(allowed),
                                                          batch_size=batch_size)
        assert torch.equal(got_bits.cpu(), want_bits)
