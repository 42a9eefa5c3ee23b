"""CPU: host logic of the press classes and the attention patch (no kernels run)."""
import numpy as np
import pytest
import torch


def _scorer():
    from kvquant import RiskScorer
    return RiskScorer(n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)


def test_package_exports_reference_names():
    import kvquant
    for name in ("scores_to_bits", "ratio_scores_to_bits", "optimal_scores_to_bits", "calibrate_epsilon",
                 "effective_bits", "DEFAULT_BIT_LEVELS", "BaseScorer", "ExpectedAttentionScorer", "RiskScorer",
                 "TurboQuantBackendPress", "TurboQuantPerTokenPress", "TurboQuantPerTokenBackendPress"):
        assert hasattr(kvquant, name), name


def test_constructor_errors_follow_reference():
    from kvquant import TurboQuantPerTokenBackendPress, TurboQuantPerTokenPress
    with pytest.raises(ValueError, match="explicit scorer"):
        TurboQuantPerTokenPress()
    with pytest.raises(ValueError, match="below 2"):
        TurboQuantPerTokenBackendPress(scorer=_scorer(), bit_levels=(0, 1, 2, 16), key_quantizer="prod")
    p = TurboQuantPerTokenBackendPress(scorer=_scorer(), bit_levels=(0, 2, 3, 4, 8, 16), key_quantizer="mse",
                                       value_quantizer="mse", target_avg_bits=2.0)
    assert p._decode_bit_levels == (2, 3, 4, 8, 16) and p.decode_quant and p.buffer_size == 128
    q = TurboQuantPerTokenBackendPress(scorer=_scorer(), bit_levels=(0, 2, 16), key_quantizer="mse",
                                       value_quantizer="mse", allow_decode_eviction=True)
    assert q._decode_bit_levels == (0, 2, 16)


def test_sink_mask_and_uniform_partition():
    from kvquant import TurboQuantPerTokenPress
    p = TurboQuantPerTokenPress(scorer=_scorer(), bit_levels=(0, 2, 4, 16), sink_tokens=4, value_quantizer="mse")
    m = p._build_sink_mask(3, 10, "cpu")
    assert m.shape == (3, 10) and m[:, :4].all() and not m[:, 4:].any()
    assert TurboQuantPerTokenPress(scorer=_scorer(), value_quantizer="mse")._build_sink_mask(2, 5, "cpu") is None
    s = torch.tensor([[0.0, 0.1, 0.3, 0.6, 0.9, 1.0, 0.2, 0.4, 0.7, 0.99]]).repeat(3, 1)
    bits = p._compute_bits(s, m)               # neither ratios nor target: uniform partition, sinks 16
    assert bits[:, :4].eq(16).all()
    assert bits[0, 4:].tolist() == [16, 16, 0, 2, 4, 16]


def test_search_hyperplane_gives_negative_logits():
    from kvquant.attention_patch import search_hyperplane
    g = torch.Generator().manual_seed(0)
    x = torch.randn(6, 12, 128, generator=g) + 0.5
    y = search_hyperplane(x)
    assert y.shape == (6, 128)
    logits = torch.einsum("nmd,nd->nm", x, y)
    assert (logits < -1e3).all()


def test_group_and_scalar_value_quantisers():
    from kvquant.press import _qd_scalar, _qd_values_group
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 128, generator=g)
    for b in (2, 4, 8):
        y = _qd_values_group(x, b, 32)
        xg = x.numpy().reshape(5, 4, 32)
        lo, hi = xg.min(-1, keepdims=True), xg.max(-1, keepdims=True)
        sc = np.maximum((hi - lo) / (2 ** b - 1), 1e-10)
        want = (np.clip(np.round((xg - lo) / sc), 0, 2 ** b - 1) * sc + lo).reshape(5, 128)
        assert np.allclose(y.numpy(), want, atol=1e-6)
        assert (y - x).abs().max() <= (hi - lo).max() / (2 ** b - 1) * 0.5 + 1e-6
        z = _qd_scalar(x, b)
        assert (z - x).abs().max() <= (x.amax(-1) - x.amin(-1)).max() / (2 ** b - 1) * 0.5 + 1e-6
    assert torch.equal(_qd_values_group(x[:, :100], 2, 32), _qd_scalar(x[:, :100], 2))   # d not divisible: per-vector


def test_observed_ratios_and_cached_allocation():
    from kvquant import TurboQuantPerTokenBackendPress
    p = TurboQuantPerTokenBackendPress(scorer=_scorer(), bit_levels=(0, 2, 4, 16), key_quantizer="mse",
                                       value_quantizer="mse", target_avg_bits=2.0, sink_tokens=4, buffer_size=8)
    T = 4 + 40 + 8
    bits = torch.full((1, 2, T), 16, dtype=torch.int32)
    bits[0, 0, 4:44] = torch.tensor([0] * 10 + [2] * 20 + [4] * 10)
    bits[0, 1, 4:44] = torch.tensor([2] * 30 + [4] * 10)
    p._record_observed_ratios(3, bits)
    assert p._observed_ratios[(3, 0)] == ((0, 0.25), (2, 0.5), (4, 0.25))
    assert p._observed_ratios[(3, 1)] == ((2, 0.75), (4, 0.25))
    # flush allocation from the cached ratios, eviction not allowed at decode: level 0 dropped, rest renormalised
    n = 12
    pos = torch.stack([torch.zeros(2 * n, dtype=torch.long), torch.arange(2).repeat_interleave(n),
                       torch.arange(n).repeat(2)], dim=-1)
    scores = torch.linspace(0, 1, 2 * n)
    out = p._allocate_bits_via_cached_ratios(scores, pos, 2, 3, {2, 4, 16})
    assert out[:n].tolist() == [2] * 8 + [4] * 4          # 2/3 and 1/3 of 12
    assert out[n:].tolist() == [2] * 9 + [4] * 3
    assert p._allocate_bits_via_cached_ratios(scores, pos, 2, 5, {2, 4, 16}) is None     # layer without a record
    # the one-sort form taken when the caller vouches for the (batch, head, position) order: same levels
    assert torch.equal(p._allocate_bits_via_cached_ratios(scores, pos, 2, 3, {2, 4, 16}, batch_size=1), out)
    B, H, n = 3, 2, 37
    g = torch.Generator().manual_seed(5)
    scores = torch.rand(B * H * n, generator=g)
    scores[7] = scores[9]                                  # a tie keeps index order in both forms
    pos = torch.stack([torch.arange(B).repeat_interleave(H * n), torch.arange(H).repeat_interleave(n).repeat(B),
                       torch.arange(n).repeat(B * H)], dim=-1)
    for allowed in ({0, 2, 4, 16}, {2, 4}):
        loop = p._allocate_bits_via_cached_ratios(scores, pos, H, 3, allowed)
        assert torch.equal(p._allocate_bits_via_cached_ratios(scores, pos, H, 3, allowed, batch_size=B), loop)


def test_rank_table_follows_the_shares_of_the_latest_prefill():
    """A press object that is used for a second prompt must flush with the second prompt's level shares:
    the expanded rank table is cached, and the cache has to notice that the shares changed."""
    from kvquant import TurboQuantPerTokenBackendPress
    p = TurboQuantPerTokenBackendPress(scorer=_scorer(), bit_levels=(0, 2, 4, 16), key_quantizer="mse",
                                       value_quantizer="mse", target_avg_bits=2.0, sink_tokens=4, buffer_size=8)
    p._decode_bit_levels = {2, 4, 16}
    T = 4 + 40 + 8

    def prompt(n2):
        bits = torch.full((1, 1, T), 16, dtype=torch.int32)
        bits[0, 0, 4:44] = torch.tensor([2] * n2 + [4] * (40 - n2))
        p._record_observed_ratios(0, bits)

    prompt(30)
    table, counts = p._by_rank_table(0, 1, 16, "cpu")
    assert table[0].tolist() == [2] * 12 + [4] * 4 and counts[0].tolist() == [0, 12, 0, 4, 0, 0]
    assert p._by_rank_table(0, 1, 16, "cpu")[0] is table            # same shares: the cached table
    prompt(10)                                                      # the next prompt: 25 % / 75 %
    table2, counts2 = p._by_rank_table(0, 1, 16, "cpu")
    assert table2[0].tolist() == [2] * 4 + [4] * 12 and counts2[0].tolist() == [0, 4, 0, 12, 0, 0]
    p._decode_bit_levels = {4, 16}                                  # and another set of allowed levels
    assert p._by_rank_table(0, 1, 16, "cpu")[0][0].tolist() == [4] * 16


def test_backend_press_rejects_unbuilt_quantisers():
    from kvquant import TurboQuantBackendPress
    with pytest.raises(NotImplementedError):
        TurboQuantBackendPress()                       # min-max values by default
    TurboQuantBackendPress(key_quantizer="mse", value_quantizer="mse")


class _FakeStore:
    """What PackedCacheLayer needs of a packed store: a length, dense rows on request, truncation."""
    def __init__(self, keys, values):
        self.k, self.v = keys.clone(), values.clone()

    @property
    def seq_len(self):
        return self.k.shape[2]

    def append(self, k, v):
        self.k, self.v = torch.cat([self.k, k], 2), torch.cat([self.v, v], 2)

    def materialize(self):
        return self.k, self.v

    def truncate(self, n):
        self.k, self.v = self.k[:, :, :n], self.v[:, :, :n]


def test_packed_cache_layer_aliases_the_newest_token():
    from kvquant.hf_cache import PackedCacheLayer, is_aliased
    g = torch.Generator().manual_seed(0)
    k0, v0 = torch.randn(2, 3, 10, 8, generator=g), torch.randn(2, 3, 10, 8, generator=g)
    store = _FakeStore(k0, v0)
    layer = PackedCacheLayer(store, k0, v0)
    assert layer.get_seq_length() == 10 and layer.get_mask_sizes(1) == (11, 0)
    assert is_aliased(layer.keys) and layer.keys.untyped_storage().nbytes() == 2 * 3 * 8 * 4
    # one token: shapes in step, every position aliases the new token, nothing is concatenated
    k1, v1 = torch.randn(2, 3, 1, 8, generator=g), torch.randn(2, 3, 1, 8, generator=g)
    keys, values = layer.update(k1, v1)
    assert keys.shape == (2, 3, 11, 8) and is_aliased(keys) and torch.equal(keys[:, :, -1:], k1)
    assert torch.equal(values[:, :, -1:], v1) and layer.recent[0] is k1
    store.append(k1, v1)                                   # what the attention path does with the token
    # several tokens: the new tokens alone, tagged with the number of tokens the store holds (the attention patch takes
    # the stored part from the fused kernel: nothing is dequantised), views afterwards
    k2, v2 = torch.randn(2, 3, 4, 8, generator=g), torch.randn(2, 3, 4, 8, generator=g)
    store.materialize = None                               # must not be called
    keys, values = layer.update(k2, v2)
    assert keys is k2 and values is v2 and keys._odmkv_store_len == 11 and values._odmkv_store_len == 11
    assert layer.get_seq_length() == 15 and is_aliased(layer.keys) and torch.equal(layer.recent[0], k2)
    store.append(k2, v2)
    # out of step: refused rather than answered from the wrong rows
    store.truncate(14)
    with pytest.raises(RuntimeError, match="in step"):
        layer.update(k2, v2)
    store.append(k2[:, :, -1:], v2[:, :, -1:])
    # crop, both spellings
    layer.crop(-2)
    assert layer.get_seq_length() == 13 and store.seq_len == 13
    layer.crop(12)
    assert layer.get_seq_length() == 12 and store.seq_len == 12
    layer.crop(40)
    assert layer.get_seq_length() == 12
    with pytest.raises(NotImplementedError):
        layer.reorder_cache(torch.tensor([0, 1]))
    with pytest.raises(ValueError, match="holds"):
        PackedCacheLayer(store, k0, v0)


def test_release_dense_cache_needs_decode_quant():
    from kvquant import TurboQuantPerTokenBackendPress
    with pytest.raises(ValueError, match="release_dense_cache"):
        TurboQuantPerTokenBackendPress(scorer=_scorer(), bit_levels=(0, 2, 4, 16), key_quantizer="mse",
                                       value_quantizer="mse", target_avg_bits=2.0, decode_quant=False,
                                       release_dense_cache=True)
