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


def _press(target=2.5, buffer_size=128, **kw):
    from kvquant import RiskScorer, TurboQuantPerTokenBackendPress
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
