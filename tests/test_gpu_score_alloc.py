"""GPU parity: risk scorer (<= 1e-3 relative, fp32 accumulate) and Lagrangian allocator (bit exact)."""
import types

import numpy as np
import pytest
import torch

from oracle import allocator as oal
from oracle import scorer as osc

pytestmark = pytest.mark.gpu
DEV = "cuda"
LEVELS = (0, 2, 3, 4, 8, 16)
EPS = {0: 1.0, 2: 0.12022445693985273, 3: 0.037507650590957564, 4: 0.012159048378616812,
       8: 0.0011957171333694236, 16: 0.0}
SCORE_RTOL = 1e-3      # the tolerance the north star states for scores


def _sink(h, t, n=4):
    m = torch.zeros(h, t, dtype=torch.bool)
    m[:, :n] = True
    return m


class Stub(torch.nn.Module):
    def __init__(self, hidden, n_heads, head_dim, seed, rotary=False, n_kv=None):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.q_proj = torch.nn.Linear(hidden, n_heads * head_dim, bias=True)
        with torch.no_grad():
            self.q_proj.weight.copy_(torch.randn(n_heads * head_dim, hidden, generator=g) / hidden ** 0.5)
            self.q_proj.bias.copy_(torch.randn(n_heads * head_dim, generator=g) * 0.1)
        self.config = types.SimpleNamespace(num_attention_heads=n_heads, head_dim=head_dim)
        self.head_dim = head_dim
        if rotary:
            from transformers import LlamaConfig
            from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
            self.rotary_emb = LlamaRotaryEmbedding(LlamaConfig(
                hidden_size=n_heads * head_dim, num_attention_heads=n_heads, num_key_value_heads=n_kv or n_heads,
                head_dim=head_dim, rope_theta=500000.0, max_position_embeddings=8192))


@pytest.mark.parametrize("hkv,hq,T,dtype,rotary", [
    (2, 8, 700, torch.float32, False), (8, 32, 4096, torch.float16, False), (4, 28, 1500, torch.bfloat16, False),
    (2, 4, 300, torch.float32, True), (3, 3, 261, torch.float16, False), (1, 1, 5, torch.float32, False),
    (2, 8, 7, torch.float16, False), (1, 4, 70, torch.bfloat16, False), (2, 16, 5, torch.bfloat16, False)])
def test_score_prefill_matches_oracle(hkv, hq, T, dtype, rotary):
    from kvquant.scorer import RiskScorer
    g = torch.Generator().manual_seed(T)
    k = torch.randn(hkv, T, 128, generator=g); v = torch.randn(hkv, T, 128, generator=g)
    k[:, :4] *= 8; v[:, :4] *= 8
    k, v = k.to(dtype), v.to(dtype)
    h = torch.randn(1, T, 96, generator=g)
    mod = Stub(96, hq, 128, T + 1, rotary=rotary, n_kv=hkv)
    sc = RiskScorer(n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)
    sc.normalize_grain = "global"
    with torch.no_grad():
        # the oracle runs the reference arithmetic on fp32 copies of the same K/V values
        want = osc.risk_score_prefill(k.float(), v.float(), module=mod, hidden_states=h)
        got = sc.score_prefill(k.to(DEV), v.to(DEV), 0, module=mod.to(DEV), hidden_states=h.to(DEV))
    assert got.shape == (hkv, T) and got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=SCORE_RTOL)
    assert torch.all(got[:, :4] == got[:, 4:].max())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mu_scale", [2.0 ** -14, 1.0, 3.0e3])
def test_score_with_mean_queries_far_from_one(dtype, mu_scale):
    """16-bit keys meet the mean query on the matrix cores as 16-bit pieces of it: mean queries thousands of times
    larger or smaller than one (keys scaled the other way, so that the logits are ordinary), heads of different
    magnitude inside one group, one head all zero, a token count that ends inside a block of 16."""
    from kvquant.scorer import _launch_score
    hkv, hq, T = 2, 14, 1003
    g = torch.Generator().manual_seed(int(mu_scale * 7) + 11)
    k = (torch.randn(hkv, T, 128, generator=g) / mu_scale).clamp(-6e4, 6e4).to(dtype)
    v = torch.randn(hkv, T, 128, generator=g).to(dtype)
    mu = torch.randn(hq, 128, generator=g) * mu_scale * 0.3
    mu[1] *= 50.0; mu[2] *= 0.01; mu[5] = 0.0
    want = osc.risk_score_from_mu(k.float(), v.float(), mu.unsqueeze(0), hq)
    got = _launch_score(k.to(DEV), v.to(DEV), mu.to(DEV), None, hq, 4, 1e-2).cpu()
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=SCORE_RTOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_score_reads_keys_where_they_lie(dtype):
    """Keys and values that are views (token-major storage seen as [H, T, d]; the upper half of 256-wide rows; a
    window of a longer cache) are read through their strides, not copied: same scores as for contiguous copies."""
    from kvquant.scorer import _launch_score
    hkv, hq, T = 3, 12, 777
    g = torch.Generator().manual_seed(5)
    mu = torch.randn(hq, 128, generator=g)
    base_k = torch.randn(T + 9, hkv, 256, generator=g).to(dtype)
    base_v = torch.randn(T + 9, hkv, 256, generator=g).to(dtype)
    views = lambda t: t.to(DEV)[5:5 + T, :, 128:].transpose(0, 1)          # noqa: E731
    k, v = views(base_k), views(base_v)
    assert not k.is_contiguous() and k.stride(-1) == 1
    got = _launch_score(k, v, mu.to(DEV), None, hq, 4, 1e-2).cpu()
    want = osc.risk_score_from_mu(k.cpu().float().contiguous(), v.cpu().float().contiguous(), mu.unsqueeze(0), hq)
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=SCORE_RTOL)


@pytest.mark.parametrize("name", ["f16", "bf16"])
def test_model_dtype_rounding_matches_reference_vectors(name):
    """The score with the roundings of a 16-bit model (kvquant/scorer.py:309-315: logits, softmax and group mean
    in the model's dtype) against what the reference returned for the same tensors, from the reference's own mean
    query (the query statistics are torch code on both sides; on the GPU their 16-bit matrix products round
    differently from the CPU's, which is not the kernel's doing).  Most scores agree to fp32 rounding; where an fp32
    sum lands on the other side of a 16-bit rounding boundary than the reference's CPU sum did, p moves by one unit
    of that dtype and the score by about twice that, relatively."""
    from kvquant.scorer import RiskScorer, _launch_score
    from test_oracle_scorer import MODEL_DTYPE_CASES, model_dtype_case
    k, v, h, mod, mu_ref, out_ref = model_dtype_case(name)
    dt, hq = MODEL_DTYPE_CASES[name]
    sc = RiskScorer(n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2, model_dtype_rounding=True)
    sc.normalize_grain = "global"
    mu = torch.from_numpy(mu_ref)[0].to(DEV)
    got = sc._maybe_normalize(_launch_score(k.to(DEV), v.to(DEV), mu, None, hq, 4, 1e-2, round_dtype=dt)).cpu().numpy()
    rel = np.abs(got - out_ref) / np.abs(out_ref)
    ulp = 2.0 ** -10 if name == "f16" else 2.0 ** -7
    assert rel.max() < 4 * ulp, rel.max()
    assert np.median(rel) < 1e-5 and (rel < 1e-4).mean() > 0.9, (np.median(rel), (rel < 1e-4).mean())
    # fp32 arithmetic on the same inputs is measurably further from the 16-bit reference
    far = sc._maybe_normalize(_launch_score(k.to(DEV), v.to(DEV), mu, None, hq, 4, 1e-2)).cpu().numpy()
    assert np.median(np.abs(far - out_ref) / np.abs(out_ref)) > 10 * np.median(rel) + 1e-5
    # the host class passes the flag on: same module on the GPU, scores within a few units of the dtype
    with torch.no_grad():
        e2e = sc.score_prefill(k.to(DEV), v.to(DEV), 0, module=mod.to(DEV), hidden_states=h.to(DEV)).float().cpu().numpy()
    assert (np.abs(e2e - out_ref) / np.abs(out_ref)).max() < 8 * ulp


def test_score_special_cases():
    from kvquant.scorer import RiskScorer
    sc = RiskScorer(n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)
    sc.normalize_grain = "global"
    g = torch.Generator().manual_seed(3)
    k = torch.randn(2, 50, 128, generator=g).half(); v = torch.randn(2, 50, 128, generator=g).half()
    a = torch.softmax(torch.randn(2, 50, generator=g), dim=-1)
    got = sc.score_with_attn(k.to(DEV), v.to(DEV), a.to(DEV))
    np.testing.assert_allclose(got.cpu().numpy(), osc.risk_score_with_attn(k, v, a).numpy(), rtol=SCORE_RTOL)
    # no module: the norm fallback (layer min-max)
    fb = sc.score_prefill(k.to(DEV), v.to(DEV), 0)
    np.testing.assert_allclose(fb.float().cpu().numpy(), osc.risk_score_prefill(k, v).float().numpy(), rtol=2e-3, atol=1e-3)
    # not longer than the sinks: ones
    assert torch.all(sc.score_prefill(k[:, :4].to(DEV), v[:, :4].to(DEV), 0, module=Stub(8, 2, 128, 1),
                                      hidden_states=torch.zeros(1, 4, 8)) == 1)


def _check_alloc(scores, target, sink=None, levels=LEVELS, **kw):
    from kvquant.allocator import optimal_scores_to_bits
    kw.setdefault("eviction_cost", 0.5)
    got = optimal_scores_to_bits(scores.to(DEV), levels, target, EPS, None if sink is None else sink.to(DEV), **kw)
    want = oal.optimal_scores_to_bits(scores, levels, target, EPS, sink, **kw)
    assert got.dtype == torch.int32 and got.shape == scores.shape
    np.testing.assert_array_equal(got.cpu().numpy(), want.numpy())
    return got


@pytest.mark.parametrize("target", [1.5, 2.0, 3.0, 6.5])
def test_allocator_bit_exact_random(target):
    g = torch.Generator().manual_seed(int(target * 10))
    s = torch.exp(2.0 * torch.randn(8, 4096, generator=g))
    s[:, :4] = s.max()
    _check_alloc(s, target, _sink(8, 4096))


@pytest.mark.parametrize("scale,target", [(1e-9, 2.0), (1e-20, 3.0), (1e6, 8.0), (1e12, 2.0), (1.0, 15.9), (1e-30, 2.0)])
def test_allocator_bit_exact_across_score_scales(scale, target):
    """The multiplier bracket reaches neighbouring fp32 numbers after a number of halvings that depends
    on the scale of the scores (24 for large ones, all 64 for tiny ones, never when the bracket was
    widened to its limit): from there the search is resolved without evaluations, and must still land
    on the lambda, and the bits, of the evaluated search."""
    g = torch.Generator().manual_seed(41)
    s = torch.exp(1.5 * torch.randn(4, 3000, generator=g)) * scale
    s[:, :4] = s.max()
    _check_alloc(s, target, _sink(4, 3000))


def test_allocator_bit_exact_edge_cases():
    g = torch.Generator().manual_seed(9)
    vals = torch.exp(torch.linspace(-3, 6, 12))
    ties = vals[torch.randint(0, 12, (4, 900), generator=g)]
    _check_alloc(ties, 2.0, _sink(4, 900))                     # repair inside groups of equal scores
    _check_alloc(ties, 3.0, _sink(4, 900))
    _check_alloc(torch.full((2, 640), 3.0), 2.0)               # all equal
    bad = torch.exp(torch.randn(2, 500, generator=g))
    bad[0, 10] = float("inf"); bad[1, 20] = float("nan"); bad[0, 30] = -5.0; bad[1, 40] = float("-inf")
    _check_alloc(bad, 2.0, _sink(2, 500))
    _check_alloc(torch.full((1, 64), float("nan")), 2.0)
    s = torch.exp(torch.randn(2, 333, generator=g))
    _check_alloc(s, 40.0)                                       # target above the top level
    _check_alloc(s, 0.5, levels=(2, 4, 8), eviction_cost=5.0)   # below the lowest
    _check_alloc(s, 2.0, _sink(2, 333), levels=(4,))            # a single level
    _check_alloc(s, 2.5, levels=(0, 2, 4, 8), eviction_cost=5.0)
    _check_alloc(s, 2.0, _sink(2, 333), above_target_alpha=0.5)
    _check_alloc(s, 2.0, torch.ones(2, 333, dtype=torch.bool))  # nothing but sinks
    for n in (1, 2, 5):
        _check_alloc(torch.exp(torch.randn(1, n, generator=g)), 2.0)
    # an arbitrary (not prefix-shaped) sink mask
    m = torch.rand(2, 333, generator=g) < 0.1
    _check_alloc(s, 2.0, m)


def test_allocator_matches_reference_vectors(golden):
    from kvquant.allocator import optimal_scores_to_bits
    eps = {int(k): float(v) for k, v in zip(golden["alloc_eps_levels"], golden["alloc_eps_values"])}
    for name, kw in {"paper2": dict(target_avg_bits=2.0), "paper15": dict(target_avg_bits=1.5),
                     "paper3": dict(target_avg_bits=3.0), "nonfinite": dict(target_avg_bits=2.0)}.items():
        s = torch.from_numpy(golden[f"alloc_{name}_scores"])
        sink = torch.from_numpy(golden[f"alloc_{name}_sink"])
        got = optimal_scores_to_bits(s.to(DEV), LEVELS, kw["target_avg_bits"], eps, sink.to(DEV), eviction_cost=0.5)
        np.testing.assert_array_equal(got.cpu().numpy(), golden[f"alloc_{name}_bits"])


def test_allocator_batched_rows_with_mixed_budgets():
    from kvquant.allocator import optimal_scores_to_bits_batched
    g = torch.Generator().manual_seed(33)
    H, T = 8, 1024
    s = torch.exp(1.5 * torch.randn(6, H * T, generator=g))
    targets = [1.5, 2.0, 3.0, 1.5, 2.0, 3.0]
    bits, counts, lam = optimal_scores_to_bits_batched(s.to(DEV), LEVELS, targets, EPS, n_sink=4, period=T,
                                                       eviction_cost=0.5, return_stats=True)
    for r in range(6):
        info = {}
        want = oal.optimal_scores_to_bits(s[r].reshape(H, T), LEVELS, targets[r], EPS, _sink(H, T),
                                          eviction_cost=0.5, info=info)
        np.testing.assert_array_equal(bits[r].reshape(H, T).cpu().numpy(), want.numpy())
        assert lam[r].item() == info["lam"]
        hist = [(want[:, 4:] == b).sum().item() for b in LEVELS]
        assert counts[r].cpu().tolist() == hist


def test_calibrate_epsilon_matches_oracle():
    from kvquant.allocator import calibrate_epsilon
    got = calibrate_epsilon(128, LEVELS, device=DEV, value_quantizer="mse")
    want = oal.calibrate_epsilon(128, LEVELS, order="canonical")
    assert set(got) == set(want)
    for b in LEVELS:
        assert abs(got[b] - want[b]) <= 1e-6 * max(want[b], 1e-9) + 1e-12


# ---- ExpectedAttentionScorer: mean query + query covariance (fp32 matrix cores) -----------------
@pytest.mark.parametrize("hkv,hq,T,dtype,use_cov,vnorm", [
    (2, 8, 700, torch.float32, True, True), (8, 32, 2085, torch.float16, True, True),
    (4, 28, 1500, torch.bfloat16, True, True), (3, 3, 261, torch.float16, True, False),
    (2, 16, 517, torch.float16, True, True), (2, 4, 300, torch.float32, False, True), (1, 1, 5, torch.float16, True, True)])
def test_expected_attention_kernel_matches_oracle(hkv, hq, T, dtype, use_cov, vnorm):
    from kvquant.scorer import _launch_score_expected
    g = torch.Generator().manual_seed(T + hq)
    k = torch.randn(hkv, T, 128, generator=g).to(dtype); v = torch.randn(hkv, T, 128, generator=g).to(dtype)
    mu = torch.randn(1, hq, 128, generator=g)
    a = torch.randn(1, hq, 128, 24, generator=g) * 0.2        # low rank + diagonal: a covariance
    cov = a @ a.transpose(-1, -2) + 0.05 * torch.eye(128) if use_cov else None
    want = osc.expected_attention_score(k.double(), v.double(), mu.double(), None if cov is None else cov.double(),
                                        hq, n_sink=4, epsilon=1e-2, use_vnorm=vnorm)
    got = _launch_score_expected(k.to(DEV), v.to(DEV), mu[0].to(DEV), None if cov is None else cov[0].to(DEV),
                                 hq, 4, 1e-2, vnorm)
    assert got.shape == (hkv, T) and got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=SCORE_RTOL)
    assert torch.all(got[:, :4] == got[:, 4:].max())


def test_expected_attention_strided_cache_rows():
    """K/V as slices of a wider buffer (head and token strides differ from the dense ones)."""
    from kvquant.scorer import _launch_score_expected
    g = torch.Generator().manual_seed(77)
    big_k = torch.randn(2, 400, 256, generator=g).half().to(DEV); big_v = torch.randn(2, 400, 256, generator=g).half().to(DEV)
    k, v = big_k[:, 10:350, 128:], big_v[:, 10:350, 128:]
    mu = torch.randn(1, 4, 128, generator=g)
    a = torch.randn(1, 4, 128, 128, generator=g) * 0.05
    cov = a @ a.transpose(-1, -2)
    want = osc.expected_attention_score(k.cpu().double(), v.cpu().double(), mu.double(), cov.double(), 4,
                                        n_sink=4, epsilon=0.0, use_vnorm=True)
    got = _launch_score_expected(k, v, mu[0].to(DEV), cov[0].to(DEV), 4, 4, 0.0, True)
    np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=SCORE_RTOL)


@pytest.mark.parametrize("name", ["d128", "d128_rope_layer"])
def test_expected_attention_scorer_matches_reference_vectors(golden, name):
    """The host class end to end (query statistics, averaged RoPE on mean and covariance, kernel,
    normalisation) against what the reference returned for the same module and tensors."""
    from kvquant.scorer import ExpectedAttentionScorer
    from test_oracle_scorer import EA_CASES, _ea_stub
    hkv, hq, d, use_cov, vnorm, eps, nf, rotary, grain = EA_CASES[name]
    cfg = dict(hidden_size=hq * d, num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d,
               rope_theta=10000.0, max_position_embeddings=4096) if rotary else None
    k, v, h = (torch.from_numpy(golden[f"ea_{name}_{x}"]) for x in "kvh")
    mod = _ea_stub(golden, name, hq, d, cfg).to(DEV)
    sc = ExpectedAttentionScorer(n_future_positions=nf, n_sink=4, use_covariance=use_cov, use_vnorm=vnorm, epsilon=eps)
    sc.normalize_grain = grain
    with torch.no_grad():
        mu, cov = sc._query_statistics(mod, h.to(DEV))
        got = sc.score_prefill(k.to(DEV), v.to(DEV), 0, module=mod, hidden_states=h.to(DEV))
    np.testing.assert_allclose(mu.cpu().numpy(), golden[f"ea_{name}_mu"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(cov.cpu().numpy(), golden[f"ea_{name}_cov"], rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(got.cpu().numpy(), golden[f"ea_{name}_out"], rtol=SCORE_RTOL, atol=1e-6)
    # fp16 model and cache: same scores within the 16-bit rounding of the inputs
    with torch.no_grad():
        got16 = sc.score_prefill(k.half().to(DEV), v.half().to(DEV), 0, module=mod.half(), hidden_states=h.half().to(DEV))
    np.testing.assert_allclose(got16.cpu().numpy(), golden[f"ea_{name}_out"], rtol=2e-2, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("cov_scale", [1e-9, 1.0, 3e3])
def test_expected_attention_covariance_pieces_keep_fp32_accuracy(dtype, cov_scale):
    """16-bit keys take the 16-bit matrix instructions with the covariance split into fp16 / bf16 pieces
    (fp16 after scaling the head's largest entry): whatever the covariance's magnitude, the scores must be
    as close to the fp64 oracle as the fp32 path is, far inside the 1e-3 bar."""
    from kvquant.scorer import _launch_score_expected
    g = torch.Generator().manual_seed(91)
    hkv, hq, T = 2, 8, 900
    k = (torch.randn(hkv, T, 128, generator=g) * (0.02 if cov_scale > 1 else 1.0)).to(dtype)
    v = torch.randn(hkv, T, 128, generator=g).to(dtype)
    mu = torch.randn(1, hq, 128, generator=g)
    a = torch.randn(1, hq, 128, 24, generator=g) * 0.2
    cov = (a @ a.transpose(-1, -2) + 0.05 * torch.eye(128)) * cov_scale
    cov[0, 3] *= 1e-4                                  # heads of very different magnitude
    want = osc.expected_attention_score(k.double(), v.double(), mu.double(), cov.double(), hq, n_sink=4,
                                        epsilon=1e-2, use_vnorm=True)
    got = _launch_score_expected(k.to(DEV), v.to(DEV), mu[0].to(DEV), cov[0].to(DEV), hq, 4, 1e-2, True)
    np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=2e-5)


# ---- observation-window attention on the 16-bit matrix cores --------------------------------------
@pytest.mark.parametrize("hkv,hq,T,W,dtype", [
    (2, 8, 700, 64, torch.float16), (8, 32, 2085, 64, torch.float16), (4, 28, 1500, 32, torch.bfloat16),
    (2, 16, 517, 64, torch.float16), (3, 3, 261, 13, torch.bfloat16), (1, 4, 300, 1, torch.float16),
    (2, 4, 40, 30, torch.float16), (1, 8, 1000, 128, torch.bfloat16)])
def test_window_attention_kernel_matches_oracle(hkv, hq, T, W, dtype):
    from kvquant.scorer import _launch_window_attention
    g = torch.Generator().manual_seed(T + W)
    k = torch.randn(hkv, T, 128, generator=g).to(dtype)
    q = (torch.randn(hq, W, 128, generator=g) * 1.5).to(dtype)
    want = osc.window_attention(k.double(), q.double(), 4, T - W)[0]
    got = _launch_window_attention(k.to(DEV), q.to(DEV), 4, T - W, 128 ** -0.5)
    assert got.shape == (hkv, T - 4) and got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=SCORE_RTOL, atol=1e-12)
    np.testing.assert_allclose(got.sum(-1).cpu().numpy(), 1.0, rtol=1e-4)


def test_window_attention_rejects_fp32_keys():
    from kvquant.scorer import _launch_window_attention
    k = torch.randn(1, 64, 128, device=DEV)
    with pytest.raises(ValueError):
        _launch_window_attention(k, torch.randn(2, 8, 128, device=DEV), 4, 56, 128 ** -0.5)


@pytest.mark.parametrize("dtype,rotary", [(torch.float16, True), (torch.bfloat16, False)])
def test_window_risk_scorer_matches_oracle(dtype, rotary):
    """The host class end to end: the module's own queries of the last `window` positions (RoPE at their
    positions), window attention, risk score, sink padding."""
    from kvquant.scorer import WindowRiskScorer
    from kvquant.attention_utils import _apply_rotary_pos_emb_q
    hkv, hq, T, W = 2, 8, 900, 48
    g = torch.Generator().manual_seed(5)
    k = torch.randn(hkv, T, 128, generator=g).to(dtype); v = torch.randn(hkv, T, 128, generator=g).to(dtype)
    h = torch.randn(1, T, 96, generator=g).to(dtype)
    mod = Stub(96, hq, 128, 17, rotary=rotary, n_kv=hkv).to(dtype)
    sc = WindowRiskScorer(window=W, n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)
    sc.normalize_grain = "global"
    with torch.no_grad():
        got = sc.score_prefill(k.to(DEV), v.to(DEV), 0, module=mod.to(DEV), hidden_states=h.to(DEV))
        # the oracle takes the same 16-bit queries the kernel was given
        mod = mod.cpu()
        q = osc.query_states(mod, h[:, T - W:])
        if rotary:
            cos, sin = mod.rotary_emb(q, torch.arange(T - W, T).unsqueeze(0))
            q = _apply_rotary_pos_emb_q(q, cos.to(q.dtype), sin.to(q.dtype))
        want = osc.window_risk_score(k.double(), v.double(), q[0].to(dtype).double(), T - W, n_sink=4, epsilon=1e-2)
    assert got.shape == (hkv, T) and got.dtype == torch.float32
    # the queries come out of a 16-bit GEMM on either side (CPU and GPU round differently): 16-bit tolerance
    np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=3e-2)
    assert torch.all(got[:, :4] == got[:, 4:].max())
