"""Pins for the oracle's ODM risk score: reference vectors, fp64 brute force, closed forms."""
import types

import numpy as np
import pytest
import torch

from oracle import scorer as sc


class Stub(torch.nn.Module):
    def __init__(self, w, b, n_heads, head_dim):
        super().__init__()
        self.q_proj = torch.nn.Linear(w.shape[1], w.shape[0], bias=True)
        with torch.no_grad():
            self.q_proj.weight.copy_(torch.as_tensor(w))
            self.q_proj.bias.copy_(torch.as_tensor(b))
        self.config = types.SimpleNamespace(num_attention_heads=n_heads, head_dim=head_dim)
        self.head_dim = head_dim


def _stub(golden, name, hq, d, dtype=torch.float32, rotary_cfg=None):
    mod = Stub(golden[f"score_{name}_w"], golden[f"score_{name}_b"], hq, d)
    if rotary_cfg is not None:
        from transformers import LlamaConfig
        from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
        mod.rotary_emb = LlamaRotaryEmbedding(LlamaConfig(**rotary_cfg))
    return mod.to(dtype)


@pytest.mark.parametrize("name,hq,d,nf", [("f32", 4, 16, 512), ("f32_g1", 3, 16, 512), ("f32_d128", 8, 128, 512)])
def test_fp32_matches_reference(golden, name, hq, d, nf):
    k, v, h = (torch.from_numpy(golden[f"score_{name}_{x}"]) for x in "kvh")
    mod = _stub(golden, name, hq, d)
    with torch.no_grad():
        mu = sc.mean_query(mod, h, 4, nf)
        got = sc.risk_score_prefill(k, v, module=mod, hidden_states=h, n_future=nf)
    np.testing.assert_allclose(mu.numpy(), golden[f"score_{name}_mu"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got.numpy(), golden[f"score_{name}_out"], rtol=2e-5)


def test_rope_average_matches_reference(golden):
    cfg = dict(hidden_size=8 * 32, num_attention_heads=8, num_key_value_heads=2, head_dim=32,
               rope_theta=10000.0, max_position_embeddings=4096)
    k, v, h = (torch.from_numpy(golden[f"score_f32_rope_{x}"]) for x in "kvh")
    mod = _stub(golden, "f32_rope", 8, 32, rotary_cfg=cfg)
    with torch.no_grad():
        mu = sc.mean_query(mod, h, 4, 64)
        got = sc.risk_score_prefill(k, v, module=mod, hidden_states=h, n_future=64)
        # closed form: mean cos * mu + mean sin * rotate_half(mu)
        raw = sc.query_states(mod, h[:, 4:]).mean(dim=2)
        cos, sin = mod.rotary_emb(raw, torch.arange(64, 128).unsqueeze(0))
        half = torch.cat([-raw[..., 16:], raw[..., :16]], dim=-1)
        closed = cos[0].mean(0) * raw + sin[0].mean(0) * half
    np.testing.assert_allclose(mu.numpy(), golden["score_f32_rope_mu"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(mu.numpy(), closed.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got.numpy(), golden["score_f32_rope_out"], rtol=2e-5)


def test_fp16_model_dtype_matches_reference(golden):
    k, v, h = (torch.from_numpy(golden[f"score_f16_{x}"]).half() for x in "kvh")
    mod = _stub(golden, "f16", 4, 16, dtype=torch.float16)
    with torch.no_grad():
        got = sc.risk_score_prefill(k, v, module=mod, hidden_states=h)
    np.testing.assert_allclose(got.float().numpy(), golden["score_f16_out"], rtol=5e-3)


MODEL_DTYPE_CASES = {"f16": (torch.float16, 8), "bf16": (torch.bfloat16, 4)}


def model_dtype_case(name):
    """(keys, values, hidden states, module, the reference's mean query and scores) of one case of
    tests/golden/score_model_dtype_d128.npz (written by tests/golden/make_score_model_dtype_vectors.py)."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "score_model_dtype_d128.npz"))
    dt, hq = MODEL_DTYPE_CASES[name]
    k = torch.from_numpy(g[f"{name}_k_bits"]).view(dt)
    v = torch.from_numpy(g[f"{name}_v_bits"]).view(dt)
    h = torch.from_numpy(g[f"{name}_h"]).to(dt)
    mod = Stub(g[f"{name}_w"], g[f"{name}_b"], hq, 128).to(dt)
    return k, v, h, mod, g[f"{name}_mu"], g[f"{name}_out"]


@pytest.mark.parametrize("name", ["f16", "bf16"])
def test_model_dtype_scores_at_head_dim_128_match_reference(name):
    """The scorer on a 16-bit module at the head size the kernels take: the oracle rounds where the reference's
    tensors have the model's dtype, and an fp32 evaluation of the same inputs is measurably elsewhere."""
    k, v, h, mod, mu_ref, out_ref = model_dtype_case(name)
    with torch.no_grad():
        mu = sc.mean_query(mod, h, 4, 512)
        got = sc.risk_score_prefill(k, v, module=mod, hidden_states=h)
    np.testing.assert_array_equal(mu.float().numpy(), mu_ref)
    np.testing.assert_allclose(got.float().numpy(), out_ref, rtol=1e-6)
    fp32 = sc.risk_score_from_mu(k.float(), v.float(), mu.float(), mu.shape[1]).numpy()
    far = np.abs(fp32 - out_ref) / np.abs(out_ref)
    assert far.max() > (1e-3 if name == "f16" else 5e-3)


def test_with_attn_and_fallback_match_reference(golden):
    k, v, a = (torch.from_numpy(golden[f"swa_{x}"]) for x in "kva")
    np.testing.assert_allclose(sc.risk_score_with_attn(k, v, a).numpy(), golden["swa_out"], rtol=1e-5)
    np.testing.assert_allclose(sc.risk_score_prefill(k, v).numpy(), golden["fallback_out"], rtol=1e-6)


def _brute(k, v, mu, g, n_sink=4, eps=1e-2):
    """fp64 loops straight from the formula."""
    k, v, mu = k.double().numpy(), v.double().numpy(), mu.double().numpy()
    h, t, d = k.shape
    out = np.zeros((h, t))
    for hh in range(h):
        p = np.zeros(t - n_sink)
        for gg in range(g):
            logit = np.array([mu[hh * g + gg] @ k[hh, j] / np.sqrt(d) for j in range(n_sink, t)])
            e = np.exp(logit - logit.max())
            p += e / e.sum() / g
        o = sum(p[j] / p.sum() * v[hh, n_sink + j] for j in range(t - n_sink))
        for j in range(t - n_sink):
            vv, kk = v[hh, n_sink + j], k[hh, n_sink + j]
            out[hh, n_sink + j] = (p[j] + eps) ** 2 * (vv @ vv + (kk @ kk) / d * ((vv - o) @ (vv - o)))
    out[:, :n_sink] = out[:, n_sink:].max()
    return out


def test_brute_force_fp64():
    g = torch.Generator().manual_seed(9)
    k = torch.randn(2, 16, 8, generator=g)
    v = torch.randn(2, 16, 8, generator=g)
    mu = torch.randn(4, 8, generator=g)
    got = sc.risk_score_from_mu(k, v, mu.unsqueeze(0), 4)
    np.testing.assert_allclose(got.numpy(), _brute(k, v, mu, 2), rtol=1e-5)


def test_closed_forms_and_invariants():
    g = torch.Generator().manual_seed(10)
    k = torch.randn(2, 40, 8, generator=g)
    v = torch.randn(2, 40, 8, generator=g)
    mu = torch.randn(1, 4, 8, generator=g)
    # attention sums to one over the core tokens
    p = sc.expected_attention(k, mu, 4, 4)
    np.testing.assert_allclose(p.sum(-1).numpy(), 1.0, rtol=1e-6)
    # zero mean query: uniform attention, o-bar is the plain mean of the core values
    s0 = sc.risk_score_from_mu(k, v, torch.zeros(1, 4, 8), 4, epsilon=0.0)
    kc, vc = k[:, 4:], v[:, 4:]
    var = (vc - vc.mean(1, keepdim=True)).pow(2).sum(-1)
    expect = (1 / 36) ** 2 * (vc.pow(2).sum(-1) + kc.pow(2).sum(-1) / 8 * var)
    np.testing.assert_allclose(s0[:, 4:].numpy(), expect.numpy(), rtol=1e-5)
    assert torch.all(s0[:, :4] == s0[:, 4:].max())
    # scaling V by c scales every score by c^2
    s1 = sc.risk_score_from_mu(k, v, mu, 4)
    s3 = sc.risk_score_from_mu(k, 3 * v, mu, 4)
    np.testing.assert_allclose(s3.numpy(), 9 * s1.numpy(), rtol=1e-5)
    # with_attn on the same p (no sinks) reproduces the prefill core
    core = sc.risk_score_with_attn(k[:, 4:], v[:, 4:], p[0])
    np.testing.assert_allclose(core.numpy(), s1[:, 4:].numpy(), rtol=1e-5)
    # short inputs
    assert torch.all(sc.risk_score_from_mu(k[:, :4], v[:, :4], mu, 4) == 1)


# ---- ExpectedAttentionScorer.score_prefill (mean query + query covariance) ---------------------
def _ea_stub(golden, name, hq, d, rotary_cfg=None):
    mod = Stub(golden[f"ea_{name}_w"], golden[f"ea_{name}_b"], hq, d)
    if rotary_cfg is not None:
        from transformers import LlamaConfig
        from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
        mod.rotary_emb = LlamaRotaryEmbedding(LlamaConfig(**rotary_cfg))
    return mod


EA_CASES = {   # name: (hkv, hq, d, use_covariance, use_vnorm, eps, n_future, rotary, grain)
    "cov": (2, 4, 16, True, True, 1e-2, 512, False, "global"),
    "nocov": (2, 4, 16, False, True, 0.0, 512, False, "global"),
    "novnorm": (3, 3, 16, True, False, 0.0, 512, False, "global"),
    "rope": (2, 8, 32, True, True, 1e-2, 64, True, "global"),
    "d128": (2, 8, 128, True, True, 1e-2, 512, False, "global"),
    "d128_rope_layer": (2, 4, 128, True, True, 0.0, 128, True, "layer"),
}


def ea_oracle(golden, name):
    """The oracle's expected-attention score of a recorded case -> (scores, mu, cov)."""
    hkv, hq, d, use_cov, vnorm, eps, nf, rotary, grain = EA_CASES[name]
    cfg = dict(hidden_size=hq * d, num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d,
               rope_theta=10000.0, max_position_embeddings=4096) if rotary else None
    k, v, h = (torch.from_numpy(golden[f"ea_{name}_{x}"]) for x in "kvh")
    mod = _ea_stub(golden, name, hq, d, cfg)
    with torch.no_grad():
        mu, cov = sc.query_statistics(mod, h, 4, nf, use_cov)
        got = sc.expected_attention_score(k, v, mu, cov, hq, n_sink=4, epsilon=eps, use_vnorm=vnorm)
    if grain == "layer":
        got = (got - got.min()) / (got.max() - got.min())
    return got, mu, cov


@pytest.mark.parametrize("name", sorted(EA_CASES))
def test_expected_attention_matches_reference(golden, name):
    got, mu, cov = ea_oracle(golden, name)
    np.testing.assert_allclose(mu.numpy(), golden[f"ea_{name}_mu"], rtol=1e-5, atol=1e-6)
    if EA_CASES[name][3]:
        np.testing.assert_allclose(cov.numpy(), golden[f"ea_{name}_cov"], rtol=1e-4, atol=1e-6)
    else:
        assert cov is None and f"ea_{name}_cov" not in golden
    np.testing.assert_allclose(got.numpy(), golden[f"ea_{name}_out"], rtol=5e-5, atol=1e-7)


def test_expected_attention_closed_forms():
    g = torch.Generator().manual_seed(5)
    hkv, G, T, d = 2, 2, 24, 8
    k = torch.randn(hkv, T, d, generator=g, dtype=torch.float64)
    v = torch.randn(hkv, T, d, generator=g, dtype=torch.float64)
    mu = torch.randn(1, hkv * G, d, generator=g, dtype=torch.float64)
    a = torch.randn(1, hkv * G, d, d, generator=g, dtype=torch.float64)
    cov = a @ a.transpose(-1, -2)
    got = sc.expected_attention_score(k, v, mu, cov, hkv * G, n_sink=4, epsilon=0.5, use_vnorm=True)
    # brute force, one token at a time
    want = torch.zeros(hkv, T, dtype=torch.float64)
    for h in range(hkv):
        p = torch.zeros(T - 4, dtype=torch.float64)
        for gq in range(G):
            q = h * G + gq
            lg = torch.tensor([float(mu[0, q] @ k[h, t]) / d ** 0.5 + float(k[h, t] @ cov[0, q] @ k[h, t]) / (2 * d)
                               for t in range(4, T)], dtype=torch.float64)
            p += torch.exp(lg - lg.max()) / torch.exp(lg - lg.max()).sum() / G
        want[h, 4:] = (p + 0.5) * torch.tensor([float(v[h, t].norm()) for t in range(4, T)], dtype=torch.float64)
    want[:, :4] = want[:, 4:].max()
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-12)
    # a zero covariance is the mean-query score; without the value norm every head's core sums to one
    zero = sc.expected_attention_score(k, v, mu, torch.zeros_like(cov), hkv * G, n_sink=4, use_vnorm=False)
    none = sc.expected_attention_score(k, v, mu, None, hkv * G, n_sink=4, use_vnorm=False)
    np.testing.assert_allclose(zero.numpy(), none.numpy(), rtol=1e-13)
    np.testing.assert_allclose(none[:, 4:].sum(-1).numpy(), 1.0, rtol=1e-12)
    # cov = c I adds c |k|^2 / (2d) to every logit of a head: tokens of equal norm keep their ranks
    kn = k / k.norm(dim=-1, keepdim=True)
    eye = torch.eye(d, dtype=torch.float64).expand(1, hkv * G, d, d) * 3.0
    same = sc.expected_attention_score(kn, v, mu, eye, hkv * G, n_sink=4, use_vnorm=False)
    base = sc.expected_attention_score(kn, v, mu, None, hkv * G, n_sink=4, use_vnorm=False)
    np.testing.assert_allclose(same.numpy(), base.numpy(), rtol=1e-12)


# ---- observation-window attention (no counterpart in the reference: pinned by definition and special cases) ----
def test_window_attention_brute_force_and_special_cases():
    g = torch.Generator().manual_seed(8)
    hkv, G, T, d, W, n_sink = 2, 2, 20, 8, 5, 3
    k = torch.randn(hkv, T, d, generator=g, dtype=torch.float64)
    v = torch.randn(hkv, T, d, generator=g, dtype=torch.float64)
    q = torch.randn(hkv * G, W, d, generator=g, dtype=torch.float64)
    q_pos0 = T - W
    got = sc.window_attention(k, q, n_sink, q_pos0)[0]
    want = torch.zeros(hkv, T - n_sink, dtype=torch.float64)
    for h in range(hkv):
        for gq in range(G):
            for w in range(W):
                last = q_pos0 + w                                     # the query sees keys at positions n_sink .. last
                lg = torch.tensor([float(q[h * G + gq, w] @ k[h, t]) / d ** 0.5 for t in range(n_sink, last + 1)],
                                  dtype=torch.float64)
                pr = torch.exp(lg - lg.max()); pr = pr / pr.sum()
                want[h, : last + 1 - n_sink] += pr / (G * W)
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(got.sum(-1).numpy(), 1.0, rtol=1e-12)                 # a mean of distributions
    assert got[:, -1].max() < 1.0 / W                                                # the last key is seen by one query in W
    # one query at the last position, no key after it: the mean-query attention with that query as the mean
    one = sc.window_attention(k, q[:, -1:], n_sink, T - 1)
    ref = sc.expected_attention(k, q[:, -1].unsqueeze(0), n_sink, hkv * G)
    np.testing.assert_allclose(one.numpy(), ref.numpy(), rtol=1e-12)
    # a window far behind the keys (no causal cut) with identical queries equals that one query's softmax
    same = sc.window_attention(k, q[:, :1].expand(-1, 4, -1), n_sink, T + 10)
    ref = sc.expected_attention(k, q[:, 0].unsqueeze(0), n_sink, hkv * G)
    np.testing.assert_allclose(same.numpy(), ref.numpy(), rtol=1e-12)
    # zero queries: uniform over the keys each query sees
    uni = sc.window_attention(k, torch.zeros_like(q), n_sink, q_pos0)[0]
    cnt = torch.tensor([sum(1.0 / (q_pos0 + w + 1 - n_sink) for w in range(W) if n_sink + t <= q_pos0 + w) / W
                        for t in range(T - n_sink)], dtype=torch.float64)
    np.testing.assert_allclose(uni[0].numpy(), cnt.numpy(), rtol=1e-12)
    # and the score built on it follows the risk formula with that p
    s = sc.window_risk_score(k, v, q, q_pos0, n_sink=n_sink, epsilon=1e-2)
    p = sc.window_attention(k, q, n_sink, q_pos0)
    np.testing.assert_allclose(s[:, n_sink:].numpy(),
                               sc.risk_from_attention(p, k[:, n_sink:], v[:, n_sink:], 1e-2)[0].numpy(), rtol=1e-12)
    assert torch.all(s[:, :n_sink] == s[:, n_sink:].max())
