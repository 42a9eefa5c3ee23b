"""GPU: the benchmark's second configuration as a stack (the reference's KVPressTextGenerationRunner over a
Llama-3-8B-shaped model, benchmark/core/pipeline.py:117-209): layers of Llama-3-8B's shape (hidden 4096, 32 query
and 8 KV heads of 128, MLP 14336; two of them, random weights, a small vocabulary), a 32768-token prefill
under the press at 2.0 average bits, then 256 greedy tokens over the packed cache.

* after the prefill every layer's stored levels equal the oracle allocator's on the press's own scores (bit exact),
  with the sink / window overrides and the budget;
* the 256 decode steps over the packed cache (fused kernel) give the logits of the same press decoding over the
  dense re-materialised cache with the model's own attention (what the reference executes), under teacher forcing,
  across a flush of the 128-token decode buffer.
"""
import math

import numpy as np
import pytest
import torch

from oracle import allocator as oal
from test_gpu_press_llama import DEV, LEVELS, LOGIT_ATOL, _generate, _ids, _press

pytestmark = pytest.mark.gpu
T, N_NEW = 32768, 256


def _c2_model(layers=2):
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(5)
    cfg = LlamaConfig(hidden_size=4096, num_hidden_layers=layers, num_attention_heads=32, num_key_value_heads=8,
                      head_dim=128, intermediate_size=14336, vocab_size=1000, max_position_embeddings=T + N_NEW + 8,
                      rope_theta=500000.0, attn_implementation="sdpa")
    default = torch.get_default_dtype()
    torch.set_default_dtype(torch.float16)                 # weights drawn on the device in fp16
    try:
        with torch.device(DEV):
            return LlamaForCausalLM(cfg).eval()
    finally:
        torch.set_default_dtype(default)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
def test_c2_stack_prefill_32k_then_256_greedy_tokens(dtype):
    """bf16 (what Llama-3 checkpoints ship in): exact tokens are stored as bf16 and the model rounds every logit to
    bf16's eight significant bits, so the two attention paths may differ by a few of those steps (three, at the
    largest logit of the run)."""
    from kvquant.allocator import calibrate_epsilon
    model = _c2_model().to(dtype)
    ids = _ids(T, 21)
    # the reference's path first: dense re-materialised cache, the model's own attention
    tok_d, log_d, _, _ = _generate(model, _press(target=2.0), ids, N_NEW, fused=False)
    torch.cuda.empty_cache()
    press = _press(target=2.0)
    seen = {}
    orig = press._score_prefill

    def spy(keys, values, layer_idx, **kw):
        s = orig(keys, values, layer_idx, **kw)
        seen[layer_idx] = s.float().cpu()
        return s

    press._score_prefill = spy
    tok_f, log_f, cache, states = _generate(model, press, ids, N_NEW, forced=tok_d, fused=True)
    err = (log_f - log_d).abs().max().item()
    top = log_d.abs().max().item()
    bf16_step = 2.0 ** (math.floor(math.log2(top)) - 7)
    logit_atol, min_agree = (LOGIT_ATOL, 0.97) if dtype == torch.float16 else (3 * bf16_step, 0.95)
    assert err <= logit_atol, (err, top)
    agree = (log_f.argmax(-1) == tok_d).float().mean().item()
    assert agree >= min_agree, agree

    eps = calibrate_epsilon(128, LEVELS, seed=42, device=DEV, value_quantizer="mse")
    assert sorted(states) == [0, 1]
    for layer_idx, st in states.items():
        assert st._exact_torch_dtype == dtype
        assert st.seq_len == T + N_NEW - 1
        lm = st._level_map[0].cpu().numpy()
        # the prefill's part of the store: the oracle allocator on the same scores, window and sinks exact
        scores = seen[layer_idx]
        H, TT = scores.shape
        assert (H, TT) == (8, T)
        sink = torch.zeros(H, T, dtype=torch.bool)
        sink[:, :4] = True
        want = oal.optimal_scores_to_bits(scores, LEVELS, 2.0, eps, sink, eviction_cost=0.5).numpy().copy()
        n_active = H * (T - 4)
        assert abs(want[:, 4:].sum() - 2.0 * n_active) <= 8          # the budget, before the window override
        want[:, -128:] = 16
        got = lm[:, :T]
        assert np.array_equal(got, want), f"layer {layer_idx}: {int((got != want).sum())} levels differ"
        assert (got[:, :4] == 16).all() and (got[:, -128:] == 16).all()
        # 255 tokens were appended: the first 128 left the exact buffer in a flush, the rest are still exact
        assert (lm[:, T:T + 128] != 16).any()
        assert (lm[:, T + 128:] == 16).all()
        counts = st.level_counts()
        assert sum(counts.values()) == lm.size
        for b in LEVELS:
            assert counts[b] == int((lm == b).sum())
