"""GPU: the press end to end on a small random-init Llama (the counterpart of the reference's
KVPressTextGenerationRunner._run/_decode, benchmark/core/pipeline.py:117-209).

* prefill under the press: the levels it stores equal the oracle allocator's on the same scores
  (bit exact), the window / sink overrides hold, and the HF cache then holds the oracle's
  dequantised values at the quantised positions;
* greedy decode over the packed cache (fused kernel) against the same press decoding over the
  dense re-materialised cache with the HF attention function (what the reference executes):
  same logits within tolerance at every step under teacher forcing, across a buffer flush.
"""
import os

import numpy as np
import pytest
import torch

from oracle import allocator as oal
from oracle import kvstate as okv

pytestmark = pytest.mark.gpu
DEV = "cuda"
LEVELS = (0, 2, 3, 4, 8, 16)
LOGIT_ATOL = 2e-2          # fp16 model: logits are O(1); fused and dense paths differ by fp16 rounding of attention outputs


def _model(seed=0, layers=2):
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(seed)
    cfg = LlamaConfig(hidden_size=512, num_hidden_layers=layers, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=128, intermediate_size=1024, vocab_size=1000, max_position_embeddings=4096,
                      rope_theta=500000.0, attn_implementation="sdpa")
    return LlamaForCausalLM(cfg).to(device=DEV, dtype=torch.float16).eval()


def _press(target=2.5, buffer_size=128, scorer=None, **kw):
    from kvquant import RiskScorer, TurboQuantPerTokenBackendPress
    if scorer is None:
        scorer = RiskScorer(n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)
        scorer.normalize_grain = "global"
    return TurboQuantPerTokenBackendPress(
        scorer=scorer, bit_levels=LEVELS, target_avg_bits=target, eviction_cost=0.5, seed=42, decode_quant=True,
        sink_tokens=4, layerwise=True, key_quantizer="mse", value_quantizer="mse", buffer_size=buffer_size, **kw)


def _ids(T, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, 1000, (1, T), generator=g).to(DEV)


@torch.inference_mode()
def _generate(model, press, ids, n_new, forced=None, fused=True):
    """Prefill under the press, then n_new decode steps; returns (tokens, logits per step)."""
    from transformers import DynamicCache
    from kvquant import attention_patch
    os.environ["ODMKV_FUSED_DECODE"] = "1" if fused else "0"
    before = dict(attention_patch.call_counts)
    try:
        cache = DynamicCache()
        T = ids.shape[1]
        logits, tokens = [], []
        with press(model):
            out = model.model(input_ids=ids, past_key_values=cache)
            last = model.lm_head(out.last_hidden_state[:, -1:, :])[0, -1].float()
            logits.append(last)
            tok = last.argmax() if forced is None else forced[0]
            tokens.append(tok)
            for step in range(n_new - 1):
                pos = T + step
                out = model(input_ids=tokens[-1].view(1, 1), past_key_values=cache,
                            position_ids=torch.tensor([[pos]], device=DEV))
                last = out.logits[0, -1].float()
                logits.append(last)
                tokens.append(last.argmax() if forced is None else forced[step + 1])
            states = dict(press._states)
        n_layers = len(model.model.layers)
        took = {k: attention_patch.call_counts[k] - before[k] for k in before}
        assert took == ({"fused": (n_new - 1) * n_layers, "dense": 0} if fused else
                        {"fused": 0, "dense": (n_new - 1) * n_layers}), took
        return torch.stack(tokens), torch.stack(logits), cache, states
    finally:
        os.environ.pop("ODMKV_FUSED_DECODE", None)


def test_prefill_bits_and_cache_match_oracle():
    from kvquant.allocator import calibrate_epsilon
    model = _model(1)
    ids = _ids(600, 11)
    captured = {}

    def grab(module, args, kwargs, output):
        layer = kwargs["past_key_values"].layers[module.layer_idx]
        captured[module.layer_idx] = (layer.keys.clone(), layer.values.clone())

    hooks = [l.self_attn.register_forward_hook(grab, with_kwargs=True) for l in model.model.layers]
    press = _press(target=2.5)
    seen_scores = {}
    orig = press._score_prefill

    def spy(keys, values, layer_idx, **kw):
        s = orig(keys, values, layer_idx, **kw)
        seen_scores[layer_idx] = s.clone()
        return s

    press._score_prefill = spy
    from transformers import DynamicCache
    cache = DynamicCache()
    with torch.inference_mode(), press(model):
        model.model(input_ids=ids, past_key_values=cache)
        states = dict(press._states)
    for h in hooks:
        h.remove()
    eps = calibrate_epsilon(128, LEVELS, seed=42, device=DEV, value_quantizer="mse")
    for layer_idx, state in states.items():
        scores = seen_scores[layer_idx].float().cpu()
        H, T = scores.shape
        sink = torch.zeros(H, T, dtype=torch.bool); sink[:, :4] = True
        want = oal.optimal_scores_to_bits(scores, LEVELS, 2.5, eps, sink, eviction_cost=0.5).numpy().copy()
        want[:, -128:] = 16
        got = state._level_map[0].cpu().numpy()
        assert np.array_equal(got, want), f"layer {layer_idx}: {int((got != want).sum())} levels differ"
        assert (got[:, :4] == 16).all() and (got[:, -128:] == 16).all()
        # the HF cache now holds the oracle's dequantised values at quantised positions
        k0, v0 = captured[layer_idx]
        ost = okv.KVState(128, LEVELS, dtype=torch.float16, seed=42 + 7 * layer_idx, order="canonical")
        ost.prefill(k0.cpu(), v0.cpu(), torch.from_numpy(want)[None].to(torch.int32))
        wk, wv = ost.materialize()
        gk = cache.layers[layer_idx].keys.float().cpu()
        gv = cache.layers[layer_idx].values.float().cpu()
        vis = torch.from_numpy(want != 0)[None, :, :, None]
        # evicted positions keep their original rows in the dense cache (only quantised rows are overwritten)
        assert torch.allclose(torch.where(vis, gk, torch.zeros(())), torch.where(vis, wk.float(), torch.zeros(())), atol=2e-3, rtol=2e-3)
        assert torch.allclose(torch.where(vis, gv, torch.zeros(())), torch.where(vis, wv.float(), torch.zeros(())), atol=2e-3, rtol=2e-3)
        masked = model.model.layers[layer_idx].self_attn.masked_key_indices
        n_evicted = int((want == 0).sum())
        assert (masked is None and n_evicted == 0) or masked[0].numel() == n_evicted


def test_greedy_decode_fused_matches_dense_path():
    model = _model(2)
    ids = _ids(700, 12)
    n_new = 140                                   # crosses one 128-token buffer flush
    tok_d, log_d, _, _ = _generate(model, _press(), ids, n_new, fused=False)
    tok_f, log_f, cache, states = _generate(model, _press(), ids, n_new, forced=tok_d, fused=True)
    err = (log_f - log_d).abs().max().item()
    assert err < LOGIT_ATOL, err
    agree = (log_f.argmax(-1) == tok_d).float().mean().item()
    assert agree >= 0.97, agree
    # the flush moved the first 128 generated tokens out of the exact segments
    st = states[0]
    assert st.seq_len == 700 + n_new - 1
    lm = st._level_map[0].cpu().numpy()
    assert (lm[:, 700:700 + 128] != 16).any()
    assert (lm[:, 700 + 128:] == 16).all()


def test_free_running_greedy_tokens_agree():
    model = _model(3)
    ids = _ids(500, 13)
    tok_d, _, _, _ = _generate(model, _press(), ids, 24, fused=False)
    tok_f, _, _, _ = _generate(model, _press(), ids, 24, fused=True)
    assert (tok_d == tok_f).float().mean().item() >= 0.9


def _rewind(cache, length):
    """Rewind the way the reference's runner does between questions (benchmark/core/pipeline.py:211-228):
    truncate the store attached to each layer and slice the layer's tensors."""
    for layer in cache.layers:
        store = getattr(layer, "_tq_backend_state", None)
        if store is not None:
            store.truncate(length)
        for name in ("keys", "values"):
            t = getattr(layer, name)
            if t.shape[2] > length:
                setattr(layer, name, t[:, :, :length])


@torch.inference_mode()
def _session(model, press, ids, forced, question):
    """Prefill, teacher-forced single-token steps, a multi-token step, a rewind by three tokens and
    one more step; returns the logits of every call and the cache."""
    from transformers import DynamicCache
    cache = DynamicCache()
    T = ids.shape[1]
    logits = []
    with press(model):
        out = model.model(input_ids=ids, past_key_values=cache)
        logits.append(model.lm_head(out.last_hidden_state[:, -1:, :])[0, -1].float())
        pos = T
        for tok in forced:
            out = model(input_ids=tok.view(1, 1), past_key_values=cache, position_ids=torch.tensor([[pos]], device=DEV))
            logits.append(out.logits[0, -1].float())
            pos += 1
        levels_after_decode = {l: st._level_map.clone() for l, st in press._states.items()}
        mid_layers = [type(layer).__name__ for layer in cache.layers]
        mid_strides = [layer.keys.stride(2) for layer in cache.layers]
        q = question.view(1, -1)
        out = model(input_ids=q, past_key_values=cache,
                    position_ids=torch.arange(pos, pos + q.shape[1], device=DEV).view(1, -1))
        logits.append(out.logits[0, -1].float())
        pos += q.shape[1]
        assert cache.get_seq_length() == pos
        pos -= 2
        _rewind(cache, pos)
        if mid_layers[0] == "PackedCacheLayer":
            cache.crop(-1)                                 # the packed layer truncates its store itself
        else:
            _rewind(cache, pos - 1)
        pos -= 1
        assert cache.get_seq_length() == pos
        assert all(st.seq_len == pos for st in press._states.values())
        out = model(input_ids=forced[0].view(1, 1), past_key_values=cache, position_ids=torch.tensor([[pos]], device=DEV))
        logits.append(out.logits[0, -1].float())
    return torch.stack(logits), cache, mid_layers, mid_strides, levels_after_decode


def test_released_dense_cache_decodes_identically():
    """`release_dense_cache=True` keeps no dense copy of the packed layers (stride-0 views of the
    newest token) and gives the logits of the press that keeps the copy: the same at single-token
    steps (same kernel, same store), within fp16 rounding at the multi-token step (dense attention
    over the dequantised store against dense attention over the kept copy), across a rewind."""
    model = _model(4)
    ids = _ids(600, 21)
    g = torch.Generator().manual_seed(22)
    forced = torch.randint(0, 1000, (140,), generator=g).to(DEV)          # crosses one buffer flush
    question = torch.randint(0, 1000, (5,), generator=g).to(DEV)
    keep, cache_k, layers_k, strides_k, levels_k = _session(model, _press(), ids, forced, question)
    rel, cache_r, layers_r, strides_r, levels_r = _session(model, _press(release_dense_cache=True), ids, forced, question)
    # the released press stores each layer as its own hook fires, the other after the last layer: same levels
    assert levels_k.keys() == levels_r.keys() and all(torch.equal(levels_k[l], levels_r[l]) for l in levels_k)
    assert layers_k == ["DynamicLayer"] * 2 and all(s != 0 for s in strides_k)
    assert layers_r == ["PackedCacheLayer"] * 2 and strides_r == [0, 0]
    n_single = 1 + forced.shape[0]
    assert torch.equal(rel[:n_single], keep[:n_single])
    assert (rel[n_single:] - keep[n_single:]).abs().max().item() < LOGIT_ATOL
    assert torch.isfinite(rel).all()


def test_released_dense_cache_refuses_the_dense_path():
    from transformers import DynamicCache
    model = _model(5)
    ids = _ids(300, 23)
    press = _press(release_dense_cache=True)
    cache = DynamicCache()
    with torch.inference_mode(), press(model):
        model.model(input_ids=ids, past_key_values=cache)
        os.environ["ODMKV_FUSED_DECODE"] = "0"
        try:
            with pytest.raises(RuntimeError, match="dense cache was released"):
                model(input_ids=ids[:, :1], past_key_values=cache, position_ids=torch.tensor([[300]], device=DEV))
        finally:
            os.environ.pop("ODMKV_FUSED_DECODE", None)


@torch.inference_mode()
def test_released_dense_cache_with_a_batch_of_two():
    from transformers import DynamicCache
    model = _model(6)
    g = torch.Generator().manual_seed(31)
    ids = torch.randint(0, 1000, (2, 400), generator=g).to(DEV)
    forced = torch.randint(0, 1000, (12, 2), generator=g).to(DEV)
    runs = []
    for release in (False, True):
        cache, logits = DynamicCache(), []
        with _press(release_dense_cache=release)(model) as _:
            model.model(input_ids=ids, past_key_values=cache)
            for step in range(forced.shape[0]):
                out = model(input_ids=forced[step].view(2, 1), past_key_values=cache,
                            position_ids=torch.full((2, 1), 400 + step, device=DEV))
                logits.append(out.logits[:, -1].float())
        assert cache.get_seq_length() == 400 + forced.shape[0]
        runs.append(torch.stack(logits))
    assert torch.equal(runs[0], runs[1])


@torch.inference_mode()
def test_released_dense_cache_without_a_decode_buffer():
    """buffer_size=0: every decoded token is scored and quantised in the hook; the attention call
    merges the still-dense newest token with the store's partial result.  Same logits with and
    without the dense copy."""
    from transformers import DynamicCache
    model = _model(7)
    ids = _ids(350, 41)
    forced = torch.randint(0, 1000, (10,), generator=torch.Generator().manual_seed(42)).to(DEV)
    runs = []
    for release in (False, True):
        cache, logits = DynamicCache(), []
        press = _press(buffer_size=0, release_dense_cache=release)
        with press(model):
            model.model(input_ids=ids, past_key_values=cache)
            for step in range(forced.shape[0]):
                out = model(input_ids=forced[step].view(1, 1), past_key_values=cache,
                            position_ids=torch.tensor([[350 + step]], device=DEV))
                logits.append(out.logits[0, -1].float())
            assert all(st.seq_len == 350 + forced.shape[0] for st in press._states.values())
            lm = press._states[0]._level_map[0].cpu()
            assert (lm[:, 350:] != 16).any()                   # decoded tokens were quantised, not buffered
        runs.append(torch.stack(logits))
    assert torch.equal(runs[0], runs[1])


def test_bf16_model_fused_matches_dense_path():
    """The same comparison on a bf16 model (exact tokens are then stored as bf16): logits are O(1) and one
    bf16 step near 2 is 0.016, so a few steps of difference between the two attention paths are expected."""
    model = _model(8).to(torch.bfloat16)
    ids = _ids(600, 51)
    n_new = 140                                   # crosses one buffer flush
    tok_d, log_d, _, _ = _generate(model, _press(), ids, n_new, fused=False)
    tok_f, log_f, _, states = _generate(model, _press(), ids, n_new, forced=tok_d, fused=True)
    assert states[0]._exact_torch_dtype == torch.bfloat16
    assert (log_f - log_d).abs().max().item() < 0.06
    assert (log_f.argmax(-1) == tok_d).float().mean().item() >= 0.95


@pytest.mark.parametrize("kind", ["expected_attention", "window_risk"])
def test_press_with_other_scorers(kind):
    """The press with the reference's other scorer class (mean query + query covariance, the default
    layer-wise min-max normalisation) and with the observation-window risk scorer: the budget holds, sinks
    and the window stay exact, the fused decode agrees with the dense path, and a 130-step decode crosses
    a buffer flush."""
    from kvquant import ExpectedAttentionScorer, WindowRiskScorer
    def scorer():
        if kind == "window_risk":
            sc = WindowRiskScorer(window=64, n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)
            sc.normalize_grain = "global"
            return sc
        return ExpectedAttentionScorer(n_future_positions=512, n_sink=4, use_covariance=True, use_vnorm=True, epsilon=1e-2)
    model = _model(5)
    ids = _ids(600, 21)
    n_new = 130
    tok_d, log_d, _, _ = _generate(model, _press(scorer=scorer()), ids, n_new, fused=False)
    tok_f, log_f, cache, states = _generate(model, _press(scorer=scorer()), ids, n_new, forced=tok_d, fused=True)
    assert (log_f - log_d).abs().max().item() < LOGIT_ATOL
    for st in states.values():
        lm = st._level_map[0, :, :600].float()
        assert torch.all(lm[:, :4] == 16) and torch.all(lm[:, 600 - 128:] == 16)
        core = lm[:, 4:600 - 128]
        assert set(core.unique().tolist()) <= set(float(b) for b in LEVELS)
        # the budget is met over all non-sink tokens before the window is forced to 16 bits, so the mean over
        # the tokens in front of the window sits near the target, not exactly under it
        assert abs(core.mean().item() - 2.5) < 0.1


@torch.inference_mode()
@pytest.mark.parametrize("path", ["device", "host"])
def test_flush_levels_match_the_oracle(path):
    """Decode-time flush (reference: kvquant/adaptive_backend_press.py:464-665, 198-241) against
    oracle.flush on the same buffered tokens: attention weights of the current query, normalised risk
    scores, and the levels from the level shares recorded at prefill.  Both ways the press can take: the
    device kernels (odmkv_exact_tail / odmkv_flush_score / odmkv_flush_rank) and the general torch path."""
    from transformers import DynamicCache
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    from oracle import flush as ofl
    model = _model(9)
    T, n_buf = 500, 128
    ids = _ids(T, 61)
    forced = torch.randint(0, 1000, (n_buf + 3,), generator=torch.Generator().manual_seed(62)).to(DEV)
    press = _press(target=2.5)
    press.device_flush = path == "device"
    press.record_flush = True
    rec = {}
    orig_flush, orig_attn, orig_alloc = press._flush_decode_buffer, press._flush_attention, press._allocate_bits_via_cached_ratios

    def spy_flush(state, layer_idx, cache, module, hidden_states=None):
        r = rec.setdefault(layer_idx, {})
        pos, k, v = state.get_buffer_tokens(press._buffer_start_seqs[layer_idx])
        r.update(pos=pos.cpu().numpy(), k=k.float().cpu(), v=v.float().cpu(), hidden=hidden_states.clone(),
                 seq_len=state.seq_len, module=module, observed={h: press._observed_ratios[(layer_idx, h)] for h in range(state.num_heads)})
        press._cur = r
        press.last_flush = None
        orig_flush(state, layer_idx, cache, module, hidden_states)
        r["levels"] = state._level_map[0].cpu().numpy().copy()
        if path == "device":
            lf = press.last_flush
            assert lf is not None and lf["layer"] == layer_idx, "the device path was not taken"
            # the kernels' rows are the buffered tokens in (batch, head, position) order
            assert torch.equal(lf["keys"].reshape(-1, 128).float().cpu(), r["k"]) and torch.equal(lf["values"].reshape(-1, 128).float().cpu(), r["v"])
            raw = lf["scores"].reshape(-1).float()
            lo, hi = raw.min(), raw.max()
            r["attn"] = lf["attn"].reshape(-1).float().cpu()
            r["scores"] = ((raw - lo) / (hi - lo).clamp_min(1e-30)).cpu()      # the normalisation the rank kernel applies
            r["bits"] = lf["bits"].reshape(-1).cpu()

    def spy_attn(*a, **kw):
        out = orig_attn(*a, **kw)
        press._cur["attn"] = out.float().cpu()
        return out

    def spy_alloc(scores, positions, *a, **kw):
        out = orig_alloc(scores, positions, *a, **kw)
        press._cur["scores"] = scores.float().cpu()
        press._cur["bits"] = out.cpu()
        return out

    press._flush_decode_buffer, press._flush_attention, press._allocate_bits_via_cached_ratios = spy_flush, spy_attn, spy_alloc
    cache = DynamicCache()
    with press(model):
        model.model(input_ids=ids, past_key_values=cache)
        for step in range(forced.shape[0]):
            model(input_ids=forced[step].view(1, 1), past_key_values=cache, position_ids=torch.tensor([[T + step]], device=DEV))
    assert sorted(rec) == [0, 1]
    for layer_idx, r in rec.items():
        assert r["pos"].shape[0] == 2 * n_buf and r["seq_len"] == T + n_buf
        # the query of the newest position through the model's own projection and rotary code
        m = r["module"]
        q = m.q_proj(r["hidden"]).view(1, 1, 4, 128).transpose(1, 2)
        cos, sin = model.model.rotary_emb(q, torch.tensor([[r["seq_len"] - 1]], device=DEV))
        q, _ = apply_rotary_pos_emb(q, q, cos, sin)
        q_last = q[:, :, -1, :].float().cpu()
        attn, scores, bits = ofl.flush_levels(q_last, r["k"], r["v"], r["pos"], 2, r["observed"], (2, 3, 4, 8, 16))
        # (1) attention weights: the press works in the model's fp16
        np.testing.assert_allclose(r["attn"].numpy(), attn.numpy(), rtol=2e-2, atol=1e-6)
        # (2) scores on the press's own weights: kernel against the oracle's formula
        want_scores = ofl.flush_scores(r["k"], r["v"], r["attn"], r["pos"], 2)
        np.testing.assert_allclose(r["scores"].numpy(), want_scores.numpy(), rtol=1e-3, atol=1e-6)
        # (3) levels on the press's own scores: bit for bit
        want_bits = ofl.cached_ratio_bits(r["scores"], r["pos"], 2, r["observed"], (2, 3, 4, 8, 16))
        assert torch.equal(r["bits"], want_bits)
        # (4) the whole chain from the oracle's own weights: the same tier sizes, and a different level only
        # for tokens whose score sits at a tier boundary (fp16 rounding of the weights moves the ranks there)
        assert sorted(bits.tolist()) == sorted(r["bits"].tolist())
        assert (bits != r["bits"]).float().mean().item() < 0.05
        # (5) the store took them: buffered positions now hold those levels, later tokens stay exact
        lm = r["levels"]
        assert (lm[r["pos"][:, 1], r["pos"][:, 2]] == r["bits"].numpy()).all()
        assert not (r["bits"] == 0).any()                 # no decode-time eviction


@torch.inference_mode()
def test_second_prompt_through_one_press_flushes_with_its_own_shares():
    """One press object, two prompts with different budgets: the device flush of the second prompt must rank
    with the level shares of the second prefill (the expanded rank table is cached per layer), exactly as
    the oracle does on the same scores and as the general torch path does."""
    from transformers import DynamicCache
    from oracle import flush as ofl
    model = _model(9)
    T, n_buf = 500, 128
    forced = torch.randint(0, 1000, (n_buf + 2,), generator=torch.Generator().manual_seed(72)).to(DEV)
    press = _press(target=2.2)
    press.record_flush = True
    seen = []
    orig_flush = press._flush_decode_buffer

    def spy_flush(state, layer_idx, cache, module, hidden_states=None):
        pos = state.get_buffer_tokens(press._buffer_start_seqs[layer_idx])[0].cpu().numpy()
        observed = {h: press._observed_ratios[(layer_idx, h)] for h in range(state.num_heads)}
        press.last_flush = None
        orig_flush(state, layer_idx, cache, module, hidden_states)
        lf = press.last_flush
        assert lf is not None and lf["layer"] == layer_idx, "the device path was not taken"
        raw = lf["scores"].reshape(-1).float()
        scores = ((raw - raw.min()) / (raw.max() - raw.min()).clamp_min(1e-30)).cpu()
        want = ofl.cached_ratio_bits(scores, pos, 2, observed, (2, 3, 4, 8, 16))
        assert torch.equal(lf["bits"].reshape(-1).cpu(), want), f"layer {layer_idx}, prompt {len(seen) // 2}"
        seen.append((layer_idx, observed, lf["bits"].reshape(-1).cpu()))

    press._flush_decode_buffer = spy_flush
    for prompt, target in enumerate((2.2, 5.0)):
        press.target_avg_bits = target
        cache = DynamicCache()
        with press(model):
            model.model(input_ids=_ids(T, 70 + prompt), past_key_values=cache)
            # the prompt is stored: the press has handed the worst-case staging store of the first fills back
            from kvquant import tq_adaptive_backend as tqa
            assert not tqa._STAGING
            for step in range(forced.shape[0]):
                model(input_ids=forced[step].view(1, 1), past_key_values=cache, position_ids=torch.tensor([[T + step]], device=DEV))
    assert [s[0] for s in seen] == [0, 1, 0, 1]
    for layer in (0, 1):
        first, second = seen[layer], seen[2 + layer]
        assert first[1] != second[1]                              # the two prefills left different shares ...
        assert sorted(first[2].tolist()) != sorted(second[2].tolist())       # ... and the flushes different tier sizes


@torch.inference_mode()
@pytest.mark.parametrize("release", [False, True])
def test_question_block_takes_the_fused_path(release):
    """The reference's runner feeds every question as ONE multi-token forward over the compressed cache
    (benchmark/core/pipeline.py:170-185).  That forward must run on the fused kernel too (stored tokens through
    decode_attention_block, the question's own causal part densely over its few tokens), give the logits of the dense
    path at every question position, and, with the dense copy released, dequantise nothing."""
    from transformers import DynamicCache
    from kvquant import attention_patch
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    model = _model(12)
    T, n_q = 700, 9
    ids = _ids(T, 81)
    question = torch.randint(0, 1000, (1, n_q), generator=torch.Generator().manual_seed(82)).to(DEV)
    pos = torch.arange(T, T + n_q, device=DEV).view(1, -1)
    n_layers = len(model.model.layers)

    def run(fused, released):
        os.environ["ODMKV_FUSED_DECODE"] = "1" if fused else "0"
        try:
            press = _press(release_dense_cache=released)
            cache = DynamicCache()
            with press(model):
                model.model(input_ids=ids, past_key_values=cache)
                before = dict(attention_patch.call_counts)
                out = model(input_ids=question, past_key_values=cache, position_ids=pos)
                took = {k: attention_patch.call_counts[k] - before[k] for k in before}
                # and one ordinary step after the block: the store took the question's tokens
                nxt = model(input_ids=question[:, :1], past_key_values=cache, position_ids=torch.tensor([[T + n_q]], device=DEV))
                assert all(st.seq_len == T + n_q + 1 for st in press._states.values())
            return out.logits[0].float(), nxt.logits[0, -1].float(), took
        finally:
            os.environ.pop("ODMKV_FUSED_DECODE", None)

    dense, dense_next, took_d = run(False, False)
    assert took_d == {"fused": 0, "dense": n_layers}
    orig = TurboQuantAdaptiveKVCacheState.materialize
    if release:
        def refuse(self, *a, **kw):
            raise AssertionError("the store was dequantised for a multi-token step")
        TurboQuantAdaptiveKVCacheState.materialize = refuse
    try:
        fused, fused_next, took_f = run(True, release)
    finally:
        TurboQuantAdaptiveKVCacheState.materialize = orig
    assert took_f == {"fused": n_layers, "dense": 0}
    assert fused.shape == (n_q, 1000)
    assert (fused - dense).abs().max().item() < LOGIT_ATOL
    assert (fused_next - dense_next).abs().max().item() < LOGIT_ATOL
