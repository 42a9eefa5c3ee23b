"""GPU: the benchmark configurations at their full sizes, through properties that do not need the
CPU oracle to run at that size (it would take minutes): the allocation against the oracle allocator on
the GPU's own scores (bit exact; the oracle allocator is fast), budget and sink/window invariants,
the partition of every position over the levels, and the fused decode attention against dense
attention over the store's own dequantised tensors (<= 1e-3 relative, the stated tolerance).

One kv-head of each configuration is small enough for the oracle (a hundred thousand tokens quantise in seconds in
its fixed-order C restatement): for that head the attention of its query group is compared with the oracle's own
store, built from the same keys, values and stored levels, so the full-size result does not rest on the GPU's own
dequantiser alone.
"""
import numpy as np
import pytest
import torch

import synthetic
from oracle import allocator as oal

pytestmark = pytest.mark.gpu
DEV = "cuda"
LEVELS = (0, 2, 3, 4, 8, 16)
EPS = {0: 1.0, 2: 0.12022445693985273, 3: 0.037507650590957564, 4: 0.012159048378616812,
       8: 0.0011957171333694236, 16: 0.0}
ATTN_RTOL = 1e-3


def _compress(layers, targets, window=128):
    """layers: list of synthetic.Layer (one per sequence).  Returns (state, bits [B,H,T], scores [B,H,T])."""
    from kvquant.allocator import optimal_scores_to_bits_batched
    from kvquant.scorer import _launch_score
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    H, T, _ = layers[0].keys.shape
    k = torch.stack([L.keys for L in layers]).to(DEV)
    v = torch.stack([L.values for L in layers]).to(DEV)
    scores = torch.stack([_launch_score(k[b], v[b], layers[b].mu.to(DEV), None, layers[b].n_q_heads, 4, 1e-2)
                          for b in range(len(layers))])
    bits = optimal_scores_to_bits_batched(scores.reshape(len(layers), -1), LEVELS, list(targets), EPS, n_sink=4,
                                          period=T, eviction_cost=0.5).reshape(len(layers), H, T)
    stored = bits.clone()
    stored[..., -window:] = 16
    st = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=DEV, dtype=torch.float16, key_quantizer="mse",
                                        value_quantizer="mse", seed=42)
    st.prefill(k, v, stored)
    return st, bits, stored, scores


def _dense_attention(st, q, G):
    # dequantised in fp32: the fp16 cast of materialize() would put its own 2^-11 rounding on every
    # key, which large-norm keys (c5 scales four key channels by 20) turn into visible logit errors
    kd = torch.zeros(st.batch_size, st.num_heads, st.seq_len, 128, dtype=torch.float32, device=DEV)
    vd = torch.zeros_like(kd)
    st._dequant_into(kd, vd, True)
    vis = st.visible_mask()
    out = torch.empty(q.shape, dtype=torch.float32, device=DEV)
    for b in range(q.shape[0]):                       # one sequence at a time keeps the temporaries small
        kb = kd[b].float().repeat_interleave(G, dim=0)
        vb = vd[b].float().repeat_interleave(G, dim=0)
        logits = torch.einsum("hd,htd->ht", q[b].float(), kb) / 128 ** 0.5
        logits = logits.masked_fill(~vis[b].repeat_interleave(G, dim=0), float("-inf"))
        out[b] = torch.einsum("ht,htd->hd", torch.softmax(logits, -1), vb)
    return out


def _check_attention(st, layers, G):
    q = torch.stack([L.query for L in layers]).to(DEV)
    fused = st.decode_attention(q)
    dense = _dense_attention(st, q, G)
    err = ((fused - dense).norm(dim=-1) / dense.norm(dim=-1)).max().item()
    assert err < ATTN_RTOL, err
    return err


def _check_attention_against_oracle(st, layers, stored, G, b=0, h=0):
    """The query group of kv-head (b, h): fused attention over the whole store against the oracle's attention over its
    own store of that head alone (fixed-order quantiser, keys and values dequantised in fp32 and then, as the
    reference does, in fp16).  Tokens appended after the prefill are not covered: call before any append."""
    from oracle.attention import decode_attention_state
    from oracle.kvstate import KVState
    L = layers[b]
    k, v = L.keys[None, h:h + 1], L.values[None, h:h + 1]
    bits = stored[b:b + 1, h:h + 1].cpu()
    q = L.query[None, h * G:(h + 1) * G].float()
    fused = st.decode_attention(torch.stack([x.query for x in layers]).to(DEV))[b, h * G:(h + 1) * G].cpu().double()
    errs = {}
    for name, dt in (("fp32", torch.float32), ("fp16", torch.float16)):
        ref = KVState(128, LEVELS, dtype=dt, seed=42, order="canonical")
        ref.prefill(k.to(dt), v.to(dt), bits)
        want = decode_attention_state(q, ref)[0]
        errs[name] = ((fused - want).norm(dim=-1) / want.norm(dim=-1)).max().item()
    assert errs["fp32"] < ATTN_RTOL, errs
    return errs


def _check_levels(st, stored):
    lm = st._level_map
    assert torch.equal(lm.to(torch.int32), stored)
    counts = st.level_counts()
    assert sum(counts.values()) == stored.numel()
    for b in LEVELS:
        assert counts[b] == int((stored == b).sum())


def test_c3_sixteen_sequences_with_cycling_budgets():
    layers = [synthetic.config("c3", seq=s) for s in range(16)]
    targets = [synthetic.C3_TARGETS[s % 3] for s in range(16)]
    st, bits, stored, scores = _compress(layers, targets)
    H, T = 8, 8192
    sink = torch.zeros(H, T, dtype=torch.bool)
    sink[:, :4] = True
    for s in (0, 1, 2, 7, 15):                         # the oracle allocator on the same scores: bit exact
        want = oal.optimal_scores_to_bits(scores[s].cpu(), LEVELS, targets[s], EPS, sink, eviction_cost=0.5)
        assert torch.equal(bits[s].cpu(), want), f"sequence {s}"
    n_active = H * (T - 4)
    for s in range(16):
        got = bits[s, :, 4:].sum().item() / n_active
        assert abs(got - targets[s]) * n_active <= 8, (s, got)
        assert (bits[s, :, :4] == 16).all()
    _check_levels(st, stored)
    _check_attention(st, layers, 4)
    _check_attention_against_oracle(st, layers, stored, 4, b=7, h=3)


def test_c4_long_context_heavy_eviction():
    from kvquant import tq_adaptive_backend as tqa
    L = synthetic.config("c4")
    tqa.release_staging()
    st, bits, stored, scores = _compress([L], [2.0])
    # the first fill of this store went through the staging store (1.2 GB for 8 x 131072 tokens), which a caller can
    # hand back once the prompt is stored
    assert [s.key[:3] for s in tqa._STAGING.values()] == [(1, 8, 131072)]
    held = torch.cuda.memory_allocated()
    tqa.release_staging(DEV)
    assert not tqa._STAGING and held - torch.cuda.memory_allocated() > 1.1e9
    evicted = (bits == 0).float().mean().item()
    assert 0.30 <= evicted <= 0.50, evicted              # the configuration is built to evict about 40 %
    n_active = 8 * (131072 - 4)
    assert abs(bits[0, :, 4:].sum().item() - 2.0 * n_active) <= 8
    sink = torch.zeros(8, 131072, dtype=torch.bool)
    sink[:, :4] = True
    want = oal.optimal_scores_to_bits(scores[0].cpu(), LEVELS, 2.0, EPS, sink, eviction_cost=0.5)
    assert torch.equal(bits[0].cpu(), want)
    _check_levels(st, stored)
    masked = st.masked_key_indices()
    assert masked[0].numel() == int((stored == 0).sum())
    _check_attention(st, [L], 4)
    _check_attention_against_oracle(st, [L], stored, 4, h=5)
    # 128 decode steps keep new tokens exact and visible
    g = torch.Generator().manual_seed(9)
    new_k = torch.randn(128, 1, 8, 1, 128, generator=g).half().to(DEV)
    new_v = torch.randn(128, 1, 8, 1, 128, generator=g).half().to(DEV)
    for step in range(128):
        st.append_all_exact(new_k[step], new_v[step])
        if step in (0, 63):                              # attention stays right while the exact segment grows
            _check_attention(st, [L], 4)
    assert st.seq_len == 131072 + 128
    assert (st._level_map[0, :, 131072:] == 16).all()
    _check_attention(st, [L], 4)


def test_c5_group_of_seven_heavy_tailed_values():
    L = synthetic.config("c5")
    st, bits, stored, scores = _compress([L], [3.0])
    n_active = 4 * (32768 - 4)
    assert abs(bits[0, :, 4:].sum().item() - 3.0 * n_active) <= 8
    sink = torch.zeros(4, 32768, dtype=torch.bool)
    sink[:, :4] = True
    want = oal.optimal_scores_to_bits(scores[0].cpu(), LEVELS, 3.0, EPS, sink, eviction_cost=0.5)
    assert torch.equal(bits[0].cpu(), want)
    used = {b for b in LEVELS if (stored == b).any()}
    assert len(used) >= 4, used                          # a 3-bit budget on heavy tails spreads over the levels
    _check_levels(st, stored)
    _check_attention(st, [L], 7)
    _check_attention_against_oracle(st, [L], stored, 7, h=2)


def test_c2_one_layer_pack_and_decode_at_full_size():
    L = synthetic.config("c2", layer=5)
    st, bits, stored, scores = _compress([L], [2.0])
    n_active = 8 * (32768 - 4)
    assert abs(bits[0, :, 4:].sum().item() - 2.0 * n_active) <= 8
    assert (bits[0, :, :4] == 16).all()
    sink = torch.zeros(8, 32768, dtype=torch.bool)
    sink[:, :4] = True
    want = oal.optimal_scores_to_bits(scores[0].cpu(), LEVELS, 2.0, EPS, sink, eviction_cost=0.5)
    assert torch.equal(bits[0].cpu(), want)
    _check_levels(st, stored)
    _check_attention(st, [L], 4)
    _check_attention_against_oracle(st, [L], stored, 4, h=6)


def test_c2_one_layer_score_matches_oracle_at_full_size():
    from oracle import scorer as osc
    L = synthetic.config("c2", layer=3)
    from kvquant.scorer import _launch_score
    got = _launch_score(L.keys.to(DEV), L.values.to(DEV), L.mu.to(DEV), None, 32, 4, 1e-2).cpu()
    want = osc.risk_score_from_mu(L.keys.float(), L.values.float(), L.mu.unsqueeze(0), 32)
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-3, atol=0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
def test_c2_one_layer_16bit_store_equals_the_exact_quantisers_at_full_size(dtype):
    """fp16 and bf16 tensors are quantised through the matrix-core estimate plus exact codes next to the thresholds,
    fp32 tensors by the exact kernel alone: on a whole 32k-token layer (2.7e8 rotated values, levels
    drawn at random over widths 2, 3 and 4) both must leave the same bytes.  (bf16 rows meet the rotation as two
    bf16 terms: a wider guard band, the same exact codes.)"""
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    L = synthetic.config("c2", layer=9)
    L.keys, L.values = L.keys.to(dtype), L.values.to(dtype)
    g = torch.Generator().manual_seed(9)
    pick = torch.multinomial(torch.tensor([0.02, 0.45, 0.3, 0.2, 0.0, 0.03]), 8 * 32768, replacement=True, generator=g)
    stored = torch.tensor(LEVELS, dtype=torch.int32)[pick].reshape(1, 8, 32768).to(DEV)
    st = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=DEV, dtype=dtype, key_quantizer="mse",
                                        value_quantizer="mse", seed=42)
    st.prefill(L.keys[None].to(DEV), L.values[None].to(DEV), stored)
    counts = st.level_counts()
    assert min(counts[2], counts[3], counts[4]) > 10000 and counts[8] == 0
    ref = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=DEV, dtype=dtype, key_quantizer="mse",
                                         value_quantizer="mse", seed=42)
    ref.prefill(L.keys[None].to(DEV).float(), L.values[None].to(DEV).float(), stored)
    assert np.array_equal(st._seg_tile, ref._seg_tile)
    for li in range(4):
        nt = int(st._seg_tile[li, -1])
        for name, per_tile in (("kcodes", 1024 * (2, 3, 4, 8)[li]), ("vcodes", 1024 * (2, 3, 4, 8)[li]), ("knorm", 64), ("vnorm", 64)):
            a, b = st._bufs[name][li].view(-1)[:nt * per_tile], ref._bufs[name][li].view(-1)[:nt * per_tile]
            if a.dtype == torch.float32:
                a, b = a.view(torch.int32), b.view(torch.int32)
            assert torch.equal(a, b), f"level index {li}, {name}"
