"""Pins for the two oracle modules the GPU tests use as yardsticks for the packed store and the
fused decode attention: ``oracle.attention`` and ``oracle.kvstate``.

Nothing here retypes the oracle's formula: the attention oracle is checked against torch's own
scaled_dot_product_attention, against cases whose answer is known without any formula (one visible
token, a permutation of the tokens, a split of the token axis merged by log-sum-exp), and the store
against its partition invariants and against ``oracle.quantizer.dequantize`` (itself pinned by the
reference's own output vectors in tests/golden).

Reference: kvquant/attention_patch.py:30-55, kvquant/tq_adaptive_backend.py:350-374, 380-464, 481-541.
"""
import math

import numpy as np
import pytest
import torch

from oracle import attention as oat
from oracle.kvstate import KVState
from oracle.quantizer import Quantized, dequantize, quantize

LEVELS = (0, 2, 3, 4, 8, 16)


def _rand(seed, *shape, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float64).to(dtype)


# ----------------------------------------------------------------------------------------------
# oracle.attention.decode_attention
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("G", [1, 4, 7])
def test_attention_equals_torch_sdpa_in_fp64(G):
    B, Hkv, T, d = 2, 3, 37, 16
    q = _rand(1 + G, B, Hkv * G, d)
    k = _rand(2 + G, B, Hkv, T, d)
    v = _rand(3 + G, B, Hkv, T, d)
    got = oat.decode_attention(q, k, v)
    want = torch.nn.functional.scaled_dot_product_attention(
        q[:, :, None, :], k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1))[:, :, 0, :]
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)
    # an explicit scale and a boolean mask go the same way
    vis = torch.rand(B, Hkv, T, generator=torch.Generator().manual_seed(9)) > 0.3
    vis[:, :, 0] = True
    got = oat.decode_attention(q, k, v, vis, scaling=0.37)
    want = torch.nn.functional.scaled_dot_product_attention(
        q[:, :, None, :], k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1),
        attn_mask=vis.repeat_interleave(G, dim=1)[:, :, None, :], scale=0.37)[:, :, 0, :]
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)


def test_attention_single_visible_token_returns_its_value():
    B, Hkv, G, T, d = 1, 2, 4, 9, 8
    q, k, v = _rand(1, B, Hkv * G, d), _rand(2, B, Hkv, T, d), _rand(3, B, Hkv, T, d)
    vis = torch.zeros(B, Hkv, T, dtype=torch.bool)
    vis[0, 0, 5] = True
    vis[0, 1, 2] = True
    out = oat.decode_attention(q, k, v, vis)
    for h in range(Hkv * G):
        want = v[0, h // G, 5 if h < G else 2]
        torch.testing.assert_close(out[0, h], want, rtol=0, atol=1e-15)


def test_attention_is_invariant_under_token_permutation_and_split_merge():
    B, Hkv, G, T, d = 2, 2, 4, 41, 16
    q, k, v = _rand(4, B, Hkv * G, d), _rand(5, B, Hkv, T, d), _rand(6, B, Hkv, T, d)
    vis = torch.rand(B, Hkv, T, generator=torch.Generator().manual_seed(7)) > 0.25
    vis[:, :, -1] = True
    base = oat.decode_attention(q, k, v, vis)
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(8))
    torch.testing.assert_close(oat.decode_attention(q, k[:, :, perm], v[:, :, perm], vis[:, :, perm]), base,
                               rtol=1e-12, atol=1e-13)
    # evicted tokens are absent: dropping them from the tensors changes nothing
    for b in range(B):
        for h in range(Hkv):
            keep = vis[b, h]
            part = oat.decode_attention(q[b:b + 1, h * G:(h + 1) * G], k[b:b + 1, h:h + 1, keep], v[b:b + 1, h:h + 1, keep])
            torch.testing.assert_close(part[0], base[b, h * G:(h + 1) * G], rtol=1e-12, atol=1e-13)
    # split of the token axis: out = sum_i w_i out_i with w_i = exp(lse_i - lse), lse over the scaled logits
    cut = 17
    scale = 1.0 / math.sqrt(d)
    outs, lses = [], []
    for sl in (slice(0, cut), slice(cut, T)):
        vv = vis[:, :, sl]
        if not vv.any(dim=-1).all():
            pytest.skip("a half has no visible token for some head")
        outs.append(oat.decode_attention(q, k[:, :, sl], v[:, :, sl], vv))
        logits = torch.einsum("bhd,bhtd->bht", q, k[:, :, sl].repeat_interleave(G, dim=1)) * scale
        logits = logits.masked_fill(~vv.repeat_interleave(G, dim=1), float("-inf"))
        lses.append(torch.logsumexp(logits, dim=-1))
    tot = torch.logsumexp(torch.stack(lses), dim=0)
    merged = sum(o * torch.exp(l - tot)[..., None] for o, l in zip(outs, lses))
    torch.testing.assert_close(merged, base, rtol=1e-12, atol=1e-13)


# ----------------------------------------------------------------------------------------------
# oracle.kvstate.KVState
# ----------------------------------------------------------------------------------------------
def _layer(seed, B=2, H=3, T=50, d=128):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, H, T, d, generator=g).half()
    v = torch.randn(B, H, T, d, generator=g).half()
    bits = torch.tensor(LEVELS)[torch.randint(0, len(LEVELS), (B, H, T), generator=g)].int()
    return k, v, bits


@pytest.mark.parametrize("order", ["blas", "canonical"])
def test_state_partitions_positions_and_materializes_through_the_pinned_dequantizer(order):
    k, v, bits = _layer(11)
    st = KVState(128, LEVELS, seed=42, order=order)
    st.prefill(k, v, bits)
    B, H, T, d = k.shape
    # every position in exactly one level, and it is the level that was asked for
    seen = np.zeros((B, H, T), np.int32)
    for pos in [st.masked, st.exact.pos] + [b.pos for b in st.banks.values()]:
        if pos.shape[0]:
            np.add.at(seen, (pos[:, 0], pos[:, 1], pos[:, 2]), 1)
    assert (seen == 1).all()
    assert (st.level_map() == bits.numpy()).all()
    # bank order is the row-major (b, h, t) order of nonzero (tq_adaptive_backend.py:356-361)
    for bank in st.banks.values():
        key = (bank.pos[:, 0] * H + bank.pos[:, 1]) * T + bank.pos[:, 2]
        assert (np.diff(key) > 0).all()
    mk, mv = st.materialize()
    assert mk.dtype == torch.float16 and mk.shape == k.shape
    for lvl in LEVELS:
        m = bits == lvl
        if lvl == 0:
            assert (mk[m] == 0).all() and (mv[m] == 0).all()
            assert (st.visible_mask() == (bits != 0)).all()
        elif lvl == 16:
            assert torch.equal(mk[m], k[m]) and torch.equal(mv[m], v[m])
        else:
            # the golden-pinned quantiser applied to the same rows, rounded to the cache dtype once
            kq = quantize(k[m], st.pi_k, lvl, order=order)
            vq = quantize(v[m], st.pi_v, lvl, order=order)
            assert torch.equal(mk[m], dequantize(kq, st.pi_k).half())
            assert torch.equal(mv[m], dequantize(vq, st.pi_v).half())
    # the key and the value rotation differ (seed and seed + 2000) and are orthogonal
    assert not torch.allclose(st.pi_k, st.pi_v)
    torch.testing.assert_close(st.pi_v @ st.pi_v.T, torch.eye(128), atol=1e-5, rtol=0)
    # masked_key_indices lists exactly the evicted positions
    mi = st.masked_key_indices()
    got = torch.zeros(B, H, T, dtype=torch.bool)
    got[mi[0], mi[1], mi[2]] = True
    assert torch.equal(got, bits == 0)


def test_materialize_quantized_into_leaves_exact_and_evicted_positions_alone():
    k, v, bits = _layer(12)
    st = KVState(128, LEVELS, seed=5)
    st.prefill(k, v, bits)
    fk = torch.full_like(k, 7.0)
    fv = torch.full_like(v, -3.0)
    st.materialize_quantized_into(fk, fv)
    mk, mv = st.materialize()
    quant = (bits != 0) & (bits != 16)
    assert torch.equal(fk[quant], mk[quant]) and torch.equal(fv[quant], mv[quant])
    assert (fk[~quant] == 7.0).all() and (fv[~quant] == -3.0).all()


def test_truncate_drops_exactly_the_positions_behind_the_cut():
    k, v, bits = _layer(13, T=60)
    st = KVState(128, LEVELS, seed=3)
    st.prefill(k, v, bits)
    full_k, full_v = st.materialize()
    for cut in (47, 47, 20, 0):
        st.truncate(cut)
        assert st.seq_len == cut
        mk, mv = st.materialize()
        assert torch.equal(mk, full_k[:, :, :cut]) and torch.equal(mv, full_v[:, :, :cut])
        assert (st.level_map() == bits[:, :, :cut].numpy()).all()
    st.truncate(100)                       # never grows
    assert st.seq_len == 0


def test_append_all_exact_and_flush_buffer_reroute_only_the_buffered_tokens():
    k, v, bits = _layer(14, T=40)
    nb = 12
    g = torch.Generator().manual_seed(15)
    kn = torch.randn(2, 3, nb, 128, generator=g).half()
    vn = torch.randn(2, 3, nb, 128, generator=g).half()
    st = KVState(128, LEVELS, seed=9)
    st.prefill(k, v, bits)
    before_k, before_v = st.materialize()
    for t in range(nb):                    # one token at a time, as a decode loop does
        st.append_all_exact(kn[:, :, t:t + 1], vn[:, :, t:t + 1])
    assert st.seq_len == 40 + nb
    pos, bk, bv = st.get_buffer_tokens(40)
    assert pos.shape[0] == 2 * 3 * nb and (pos[:, 2] >= 40).all()
    # buffered tokens come back as they went in, whatever their order
    assert torch.equal(bk, kn[pos[:, 0], pos[:, 1], pos[:, 2] - 40])
    assert torch.equal(bv, vn[pos[:, 0], pos[:, 1], pos[:, 2] - 40])
    new_bits = torch.tensor((2, 3, 4, 8, 16, 0))[torch.randint(0, 6, (pos.shape[0],), generator=g)].int()
    st.flush_buffer(40, new_bits)
    mk, mv = st.materialize()
    # what was stored before the buffer is untouched
    assert torch.equal(mk[:, :, :40], before_k) and torch.equal(mv[:, :, :40], before_v)
    lm = st.level_map()
    assert (lm[:, :, :40] == bits.numpy()).all()
    assert (lm[pos[:, 0], pos[:, 1], pos[:, 2]] == new_bits.numpy()).all()
    for lvl in (2, 3, 4, 8):
        m = (new_bits == lvl).numpy()
        if not m.any():
            continue
        rows = torch.from_numpy(m)
        want_k = dequantize(quantize(bk[rows], st.pi_k, lvl), st.pi_k).half()
        want_v = dequantize(quantize(bv[rows], st.pi_v, lvl), st.pi_v).half()
        p = pos[m]
        # the bank is dequantised whole (one matrix product over old and new rows): the library may sum
        # in another order than for these rows alone, so the last fp16 bit is free
        torch.testing.assert_close(mk[p[:, 0], p[:, 1], p[:, 2]], want_k, rtol=2e-3, atol=1e-6)
        torch.testing.assert_close(mv[p[:, 0], p[:, 1], p[:, 2]], want_v, rtol=2e-3, atol=1e-6)
    m16 = (new_bits == 16).numpy()
    p = pos[m16]
    assert torch.equal(mk[p[:, 0], p[:, 1], p[:, 2]], bk[torch.from_numpy(m16)])
    m0 = (new_bits == 0).numpy()
    p = pos[m0]
    assert (mk[p[:, 0], p[:, 1], p[:, 2]] == 0).all()
    assert not st.visible_mask()[p[:, 0], p[:, 1], p[:, 2]].any()
    # a second flush with nothing behind the mark changes nothing
    st.flush_buffer(st.seq_len, torch.zeros(0, dtype=torch.int32))
    mk2, _ = st.materialize()
    assert torch.equal(mk2, mk)


def test_packed_bytes_counts_true_widths_norms_and_exact_rows():
    k, v, bits = _layer(16, B=1, H=2, T=30)
    st = KVState(128, LEVELS, seed=1)
    st.prefill(k, v, bits)
    n = {lvl: int((bits == lvl).sum()) for lvl in LEVELS}
    want = n[16] * 512 + sum(n[b] * (2 * b * 16 + 8) for b in (2, 3, 4, 8))
    assert st.packed_bytes() == want


def test_attention_over_a_state_is_attention_over_its_dense_cache_without_evicted_tokens():
    k, v, bits = _layer(17, B=1, H=2, T=33)
    st = KVState(128, LEVELS, seed=2)
    st.prefill(k, v, bits)
    q = _rand(18, 1, 8, 128)
    mk, mv = st.materialize()
    got = oat.decode_attention_state(q, st)
    for h in range(2):
        keep = bits[0, h] != 0
        kk = mk[0, h][keep].double().repeat(4, 1, 1)       # the four query heads of the group
        vv = mv[0, h][keep].double().repeat(4, 1, 1)
        want = torch.nn.functional.scaled_dot_product_attention(q[0, 4 * h:4 * h + 4, None, :], kk, vv)[:, 0]
        torch.testing.assert_close(got[0, 4 * h:4 * h + 4], want, rtol=1e-12, atol=1e-13)
