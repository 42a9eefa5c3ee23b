"""Writes tests/golden/reference_vectors.npz: small input/output vectors of the reference.

Run once, in the build container, where the reference checkout is mounted read-only:

    python tests/golden/make_reference_vectors.py /root/reference

It imports the reference's own modules and records what they return for seeded inputs, for
the points of the path that reading the code cannot settle: the exact fp64 codebook tables,
the allocator's choices (including which of several equal scores its unstable argsort moves),
the scorer in fp32 and in fp16, the container bytes of the bit packer, the rank-ratio
allocator.  The quantiser itself cannot be recorded: the reference imports a module it does
not ship (kvquant.tq_triton) inside TurboQuantMSE.quantize.

Only data is stored (numpy arrays); no reference source text.
"""
from __future__ import annotations

import os
import sys
import types

import numpy as np
import torch


def main(ref_root: str) -> None:
    sys.path.insert(0, ref_root)
    import codebook as ref_codebook                                   # noqa: E402
    from kvquant import allocator as ref_alloc                        # noqa: E402
    from kvquant import scorer as ref_scorer                          # noqa: E402
    from kvquant import tq_backend as ref_tq                          # noqa: E402

    out: dict[str, np.ndarray] = {}

    # ---- codebooks -------------------------------------------------------------------
    for d in (128, 64):
        for b in (1, 2, 3, 4, 8):
            if d == 64 and b > 4:
                continue
            out[f"codebook_d{d}_b{b}"] = ref_codebook.compute_codebook(2 ** b, d)

    # ---- bit packer ------------------------------------------------------------------
    g = torch.Generator().manual_seed(7)
    for b in (1, 2, 3, 4, 8):
        codes = torch.randint(0, 2 ** b, (5, 128), generator=g, dtype=torch.int64)
        out[f"pack_b{b}_codes"] = codes.numpy().astype(np.uint8)
        packed = ref_tq._pack_indices(codes, b)
        out[f"pack_b{b}_bytes"] = packed.numpy()
        back = ref_tq._unpack_indices(packed, b, 128)
        out[f"pack_b{b}_roundtrip"] = back.numpy().astype(np.uint8)

    # ---- dequantise (rotation + centroid gather + norm) ------------------------------
    pi = ref_tq.random_rotation(128, torch.device("cpu"), torch.float32, seed=42)
    out["pi_seed42"] = pi.numpy()
    q4 = ref_tq.TurboQuantMSE(128, 4, device=torch.device("cpu"), dtype=torch.float16, seed=42)
    codes = torch.randint(0, 16, (6, 128), generator=g, dtype=torch.int64)
    norms = torch.rand(6, generator=g) * 10 + 0.5
    deq = q4.dequantize(ref_tq.MSEQuantized(indices=ref_tq._pack_indices(codes, 4), norms=norms, bits=4))
    out["deq_b4_codes"] = codes.numpy().astype(np.uint8)
    out["deq_b4_norms"] = norms.numpy()
    out["deq_b4_out"] = deq.numpy()
    out["deq_b4_centroids"] = q4.centroids.numpy()

    # ---- allocator -------------------------------------------------------------------
    eps = {0: 1.0, 2: 0.1175, 3: 0.0345, 4: 0.0095, 8: 4.0e-5, 16: 0.0}
    levels = (0, 2, 3, 4, 8, 16)

    def alloc_case(name, scores, sink_mask, **kw):
        res = ref_alloc.optimal_scores_to_bits(scores, sink_mask=sink_mask, **kw)
        out[f"alloc_{name}_scores"] = scores.numpy()
        if sink_mask is not None:
            out[f"alloc_{name}_sink"] = sink_mask.numpy()
        out[f"alloc_{name}_bits"] = res.numpy()

    def sink(h, t, n=4):
        m = torch.zeros(h, t, dtype=torch.bool)
        m[:, :n] = True
        return m

    g = torch.Generator().manual_seed(11)
    s = torch.exp(2.0 * torch.randn(8, 512, generator=g))
    s[:, :4] = s.max()
    alloc_case("paper2", s, sink(8, 512), bit_levels=levels, target_avg_bits=2.0, epsilon=eps, eviction_cost=0.5)
    alloc_case("paper15", s, sink(8, 512), bit_levels=levels, target_avg_bits=1.5, epsilon=eps, eviction_cost=0.5)
    alloc_case("paper3", s, sink(8, 512), bit_levels=levels, target_avg_bits=3.0, epsilon=eps, eviction_cost=0.5)
    alloc_case("default_evict", s, None, bit_levels=(0, 2, 4, 8), target_avg_bits=2.5, epsilon=eps)
    alloc_case("alpha", s, sink(8, 512), bit_levels=levels, target_avg_bits=2.0, epsilon=eps,
               eviction_cost=0.5, above_target_alpha=0.5)
    # heavy ties: scores drawn from 12 distinct values
    vals = torch.exp(torch.linspace(-3, 6, 12))
    st = vals[torch.randint(0, 12, (4, 300), generator=g)]
    alloc_case("ties", st, sink(4, 300), bit_levels=levels, target_avg_bits=2.0, epsilon=eps, eviction_cost=0.5)
    alloc_case("allequal", torch.full((2, 64), 3.0), None, bit_levels=levels, target_avg_bits=2.0,
               epsilon=eps, eviction_cost=0.5)
    # non-finite and negative entries
    sb = torch.exp(torch.randn(2, 200, generator=g))
    sb[0, 10] = float("inf"); sb[1, 20] = float("nan"); sb[0, 30] = -5.0; sb[1, 40] = float("-inf")
    alloc_case("nonfinite", sb, sink(2, 200), bit_levels=levels, target_avg_bits=2.0, epsilon=eps, eviction_cost=0.5)
    # clamps and single level
    alloc_case("target_hi", s[:2, :64], None, bit_levels=levels, target_avg_bits=40.0, epsilon=eps, eviction_cost=0.5)
    alloc_case("target_lo", s[:2, :64], None, bit_levels=(2, 4, 8), target_avg_bits=0.5, epsilon=eps)
    alloc_case("single", s[:2, :64], sink(2, 64), bit_levels=(4,), target_avg_bits=2.0, epsilon=eps)
    # tiny problems
    for n in (1, 2, 5):
        alloc_case(f"tiny{n}", torch.exp(torch.randn(1, n, generator=g)), None, bit_levels=levels,
                   target_avg_bits=2.0, epsilon=eps, eviction_cost=0.5)
    out["alloc_eps_levels"] = np.asarray(sorted(eps), np.int32)
    out["alloc_eps_values"] = np.asarray([eps[k] for k in sorted(eps)], np.float64)

    # ---- rank-ratio and uniform allocators -------------------------------------------
    sr = torch.rand(3, 128, generator=g)
    out["ratio_scores"] = sr.numpy()
    out["ratio_bits"] = ref_alloc.ratio_scores_to_bits(sr, (2, 3, 4, 8, 16), (0.5, 0.2, 0.15, 0.1, 0.05)).numpy()
    out["ratio_bits_flat"] = ref_alloc.ratio_scores_to_bits(sr, (2, 4, 8), (0.6, 0.3, 0.1), per_head=False).numpy()
    out["uniform_bits"] = ref_alloc.scores_to_bits(sr, (2, 3, 4, 8, 16)).numpy()

    # ---- scorer ----------------------------------------------------------------------
    class Stub(torch.nn.Module):
        def __init__(self, hidden, n_heads, head_dim, seed):
            super().__init__()
            gg = torch.Generator().manual_seed(seed)
            self.q_proj = torch.nn.Linear(hidden, n_heads * head_dim, bias=True)
            with torch.no_grad():
                self.q_proj.weight.copy_(torch.randn(n_heads * head_dim, hidden, generator=gg) / hidden ** 0.5)
                self.q_proj.bias.copy_(torch.randn(n_heads * head_dim, generator=gg) * 0.1)
            self.config = types.SimpleNamespace(num_attention_heads=n_heads, head_dim=head_dim)
            self.head_dim = head_dim

    def score_case(name, hkv, hq, t, d, hidden, seed, dtype, rotary=False, n_future=512):
        gg = torch.Generator().manual_seed(seed)
        k = torch.randn(hkv, t, d, generator=gg)
        v = torch.randn(hkv, t, d, generator=gg)
        k[:, :4] *= 8
        v[:, :4] *= 8
        h = torch.randn(1, t, hidden, generator=gg)
        mod = Stub(hidden, hq, d, seed + 1)
        if rotary:
            from transformers import LlamaConfig
            from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
            cfg = LlamaConfig(hidden_size=hq * d, num_attention_heads=hq, num_key_value_heads=hkv,
                              head_dim=d, rope_theta=10000.0, max_position_embeddings=4096)
            mod.rotary_emb = LlamaRotaryEmbedding(cfg)
        mod = mod.to(dtype)
        sc = ref_scorer.RiskScorer(n_future_positions=n_future, n_sink=4, use_vnorm=True, epsilon=1e-2)
        sc.normalize_grain = "global"
        with torch.no_grad():
            res = sc.score_prefill(k.to(dtype), v.to(dtype), 0, module=mod, hidden_states=h.to(dtype))
            mu = sc._query_statistics(mod, h.to(dtype))[0]
        out[f"score_{name}_k"] = k.numpy()
        out[f"score_{name}_v"] = v.numpy()
        out[f"score_{name}_h"] = h.numpy()
        out[f"score_{name}_w"] = mod.q_proj.weight.detach().float().numpy()
        out[f"score_{name}_b"] = mod.q_proj.bias.detach().float().numpy()
        out[f"score_{name}_mu"] = mu.float().numpy()
        out[f"score_{name}_out"] = res.float().numpy()

    score_case("f32", 2, 4, 48, 16, 24, 21, torch.float32)
    score_case("f32_g1", 3, 3, 40, 16, 24, 22, torch.float32)
    score_case("f32_rope", 2, 8, 64, 32, 40, 23, torch.float32, rotary=True, n_future=64)
    score_case("f16", 2, 4, 48, 16, 24, 21, torch.float16)
    score_case("f32_d128", 2, 8, 160, 128, 64, 24, torch.float32)

    # ExpectedAttentionScorer.score_prefill: covariance on/off, value norm on/off, RoPE, GQA
    def ea_case(name, hkv, hq, t, d, hidden, seed, *, cov=True, vnorm=True, eps=0.0, rotary=False, n_future=512,
                grain="global"):
        gg = torch.Generator().manual_seed(seed)
        k = torch.randn(hkv, t, d, generator=gg)
        v = torch.randn(hkv, t, d, generator=gg)
        h = torch.randn(1, t, hidden, generator=gg)
        mod = Stub(hidden, hq, d, seed + 1)
        if rotary:
            from transformers import LlamaConfig
            from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
            cfg = LlamaConfig(hidden_size=hq * d, num_attention_heads=hq, num_key_value_heads=hkv,
                              head_dim=d, rope_theta=10000.0, max_position_embeddings=4096)
            mod.rotary_emb = LlamaRotaryEmbedding(cfg)
        sc = ref_scorer.ExpectedAttentionScorer(n_future_positions=n_future, n_sink=4, use_covariance=cov,
                                                use_vnorm=vnorm, epsilon=eps)
        sc.normalize_grain = grain
        with torch.no_grad():
            res = sc.score_prefill(k, v, 0, module=mod, hidden_states=h)
            mu, cv = sc._query_statistics(mod, h)
        out[f"ea_{name}_k"], out[f"ea_{name}_v"], out[f"ea_{name}_h"] = k.numpy(), v.numpy(), h.numpy()
        out[f"ea_{name}_w"] = mod.q_proj.weight.detach().numpy()
        out[f"ea_{name}_b"] = mod.q_proj.bias.detach().numpy()
        out[f"ea_{name}_mu"] = mu.numpy()
        if cv is not None:
            out[f"ea_{name}_cov"] = cv.numpy()
        out[f"ea_{name}_out"] = res.numpy()

    ea_case("cov", 2, 4, 48, 16, 24, 41, eps=1e-2)
    ea_case("nocov", 2, 4, 48, 16, 24, 42, cov=False)
    ea_case("novnorm", 3, 3, 40, 16, 24, 43, vnorm=False)
    ea_case("rope", 2, 8, 64, 32, 40, 44, rotary=True, n_future=64, eps=1e-2)
    ea_case("d128", 2, 8, 300, 128, 64, 45, eps=1e-2)
    ea_case("d128_rope_layer", 2, 4, 200, 128, 64, 46, rotary=True, n_future=128, grain="layer")

    # score_with_attn and the norm fallback
    gg = torch.Generator().manual_seed(31)
    k = torch.randn(3, 20, 16, generator=gg); v = torch.randn(3, 20, 16, generator=gg)
    a = torch.softmax(torch.randn(3, 20, generator=gg), dim=-1)
    sc = ref_scorer.RiskScorer(n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)
    sc.normalize_grain = "global"
    out["swa_k"], out["swa_v"], out["swa_a"] = k.numpy(), v.numpy(), a.numpy()
    out["swa_out"] = sc.score_with_attn(k, v, a).numpy()
    out["fallback_out"] = sc.score_prefill(k, v, 0).numpy()

    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")
    np.savez_compressed(dst, **out)
    print(f"wrote {dst}: {len(out)} arrays, {os.path.getsize(dst)} bytes")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
