"""Writes tests/golden/score_model_dtype_d128.npz: the reference's RiskScorer.score_prefill on a module whose
weights, hidden states, keys and values are fp16 / bf16 (the scorer then rounds the logits, the softmax and the
group mean to that type), at head_dim 128, the only one the HIP kernels take.

Run once, in the build container, where the reference checkout is mounted read-only:

    python tests/golden/make_score_model_dtype_vectors.py /root/reference

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
    from kvquant import scorer as ref_scorer                          # noqa: E402

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

    out: dict[str, np.ndarray] = {}
    for name, dtype, hkv, hq, t, hidden, seed in (("f16", torch.float16, 2, 8, 800, 64, 31),
                                                  ("bf16", torch.bfloat16, 2, 4, 700, 64, 32)):
        gg = torch.Generator().manual_seed(seed)
        k = torch.randn(hkv, t, 128, generator=gg)
        v = torch.randn(hkv, t, 128, generator=gg)
        k[:, :4] *= 8
        v[:, :4] *= 8
        h = torch.randn(1, t, hidden, generator=gg)
        mod = Stub(hidden, hq, 128, seed + 1).to(dtype)
        sc = ref_scorer.RiskScorer(n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)
        sc.normalize_grain = "global"
        with torch.no_grad():
            res = sc.score_prefill(k.to(dtype), v.to(dtype), 0, module=mod, hidden_states=h.to(dtype))
            mu = sc._query_statistics(mod, h.to(dtype))[0]
        # keys and values as the bit patterns of the 16-bit values the scorer saw
        out[f"{name}_k_bits"] = k.to(dtype).view(torch.int16).numpy()
        out[f"{name}_v_bits"] = v.to(dtype).view(torch.int16).numpy()
        out[f"{name}_h"] = h.to(dtype).float().numpy()
        out[f"{name}_w"] = mod.q_proj.weight.detach().float().numpy()
        out[f"{name}_b"] = mod.q_proj.bias.detach().float().numpy()
        out[f"{name}_mu"] = mu.float().numpy()
        out[f"{name}_out"] = res.float().numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "score_model_dtype_d128.npz")
    np.savez_compressed(path, **out)
    print(path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
