"""GPU: the device kernels of the decode-time flush through the C ABI (odmkv_exact_tail, odmkv_flush_score,
odmkv_flush_rank) against oracle.flush (reference: kvquant/adaptive_backend_press.py:198-241, 464-665) and the
state's own general gather: attention and scores within 1e-3, levels bit for bit on the kernel's own scores,
ties and a degenerate score range included."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import flush as ofl

pytestmark = pytest.mark.gpu
DEV = "cuda"
LEVELS = (0, 2, 3, 4, 8, 16)


def _positions(B, H, n, start=100):
    bb, hh, tt = np.meshgrid(np.arange(B), np.arange(H), np.arange(n) + start, indexing="ij")
    return np.stack([bb.ravel(), hh.ravel(), tt.ravel()], -1).astype(np.int64)


def _score(k, v, q, eps, mode, want_attn=True):
    from kvquant import _lib
    B, H, n, d = k.shape
    attn = torch.empty(B * H, n, dtype=torch.float32, device=DEV) if want_attn else None
    scores = torch.empty(B * H, n, dtype=torch.float32, device=DEV)
    minmax = torch.empty(B * H, 2, dtype=torch.float32, device=DEV)
    q32 = q.reshape(B * H, d).float().contiguous()
    _lib.check(_lib.lib.odmkv_flush_score(k.data_ptr(), v.data_ptr(), _lib.dtype_code(k), B * H, n, q32.data_ptr(),
                                          d ** -0.5, eps, mode, _lib.ptr(attn), scores.data_ptr(), minmax.data_ptr(),
                                          _lib.stream_ptr(k.device)))
    return attn, scores, minmax


@pytest.mark.parametrize("B,H,n,dtype", [(1, 8, 128, torch.float16), (3, 2, 37, torch.bfloat16), (2, 4, 700, torch.float16),
                                         (1, 1, 1, torch.float16), (1, 2, 2048, torch.float32)])
def test_flush_score_matches_oracle(B, H, n, dtype):
    g = torch.Generator().manual_seed(B * 1000 + n)
    k = torch.randn(B, H, n, 128, generator=g).to(dtype)
    v = torch.randn(B, H, n, 128, generator=g).to(dtype)
    q = (torch.randn(B, H, 128, generator=g) * 1.5).to(dtype)
    pos = _positions(B, H, n)
    fk, fv = k.reshape(-1, 128).float(), v.reshape(-1, 128).float()
    want_attn = ofl.flush_attention(q.float(), fk, pos, H)                      # one query head per kv-head: the mean is the query
    attn, scores, minmax = _score(k.to(DEV), v.to(DEV), q.to(DEV), 1e-2, 0)
    np.testing.assert_allclose(attn.reshape(-1).cpu().numpy(), want_attn.numpy(), rtol=1e-3, atol=1e-9)
    np.testing.assert_allclose(attn.sum(-1).cpu().numpy(), 1.0, atol=1e-5)
    raw = scores.reshape(-1).cpu()
    lo, hi = minmax[:, 0].min().item(), minmax[:, 1].max().item()
    assert lo == raw.min().item() and hi == raw.max().item()
    want = ofl.flush_scores(fk, fv, attn.reshape(-1).cpu(), pos, H, epsilon=1e-2)   # normalised over the whole flush
    got = ofl.minmax(raw) if n * B * H > 1 else torch.full_like(raw, 0.5)
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-3, atol=1e-6)
    # without a scorer: attn^2 |v|^2
    _, plain, _ = _score(k.to(DEV), v.to(DEV), q.to(DEV), 0.0, 1, want_attn=False)
    want_plain = attn.reshape(-1).cpu().pow(2) * fv.pow(2).sum(-1)
    np.testing.assert_allclose(plain.reshape(-1).cpu().numpy(), want_plain.numpy(), rtol=1e-4, atol=1e-12)


@pytest.mark.parametrize("mode", [0, 1])
def test_flush_score_range_carries_a_nan(mode):
    """A NaN among the buffered values gives NaN scores; the range the kernel reports for that head must say so
    (torch's min() / max() in the reference's normalisation return NaN then), and the ranking that follows must
    still give every token a level: the whole chain on one poisoned buffer."""
    g = torch.Generator().manual_seed(31)
    B, H, n = 1, 2, 64
    k = torch.randn(B, H, n, 128, generator=g).half()
    v = torch.randn(B, H, n, 128, generator=g).half()
    v[0, 1, 7, 3] = float("nan")
    q = torch.randn(B, H, 128, generator=g).half()
    _, scores, minmax = _score(k.to(DEV), v.to(DEV), q.to(DEV), 1e-2, mode)
    mm = minmax.cpu()
    assert torch.isnan(scores.reshape(B, H, n)[0, 1]).any()
    assert torch.isnan(mm[1]).all() and torch.isfinite(mm[0]).all()
    observed = {h: ((2, 0.5), (4, 0.5)) for h in range(H)}
    got = _rank(scores, minmax, B, H, n, observed, {2, 4, 16}).cpu()
    want = ofl.cached_ratio_bits(ofl.minmax(scores.reshape(-1).cpu()), _positions(B, H, n), H, observed, (2, 4, 16))
    assert torch.equal(got.reshape(-1), want)                # all keys 0.5: index order, the first half 2 bits
    assert got[0, 0].tolist() == [2] * 32 + [4] * 32


def _rank(scores, minmax, B, H, n, observed, allowed):
    from kvquant import _lib
    from kvquant.adaptive_backend_press import _levels_by_rank
    rows = []
    for h in range(H):
        kept = [(b, r) for b, r in observed[h] if b in allowed and r > 0]
        total = sum(r for _, r in kept)
        levels, ratios = zip(*[(b, r / total) for b, r in kept])
        rows.append(_levels_by_rank(levels, ratios, B * n))
    by_rank = torch.from_numpy(np.stack(rows)).to(DEV)
    bits = torch.empty(B, H, n, dtype=torch.int32, device=DEV)
    _lib.check(_lib.lib.odmkv_flush_rank(scores.data_ptr(), minmax.data_ptr(), B, H, n, by_rank.data_ptr(), bits.data_ptr(),
                                         _lib.stream_ptr(scores.device)))
    return bits


@pytest.mark.parametrize("B,H,n,kind", [(1, 8, 128, "random"), (4, 3, 100, "random"), (2, 2, 64, "ties"), (1, 2, 33, "flat"),
                                        (8, 1, 512, "random"), (1, 1, 1, "random"), (2, 2, 37, "nan"), (1, 3, 100, "inf"),
                                        (2, 2, 37, "neginf"), (1, 2, 3, "inf")])
def test_flush_rank_matches_oracle_bit_for_bit(B, H, n, kind):
    g = torch.Generator().manual_seed(B * 77 + n)
    scores = torch.rand(B, H, n, generator=g) * 3.0 + 0.5
    if kind == "ties":
        scores = (scores * 4).round() / 4                                       # many equal scores across sequences
    if kind == "flat":
        scores = torch.full((B, H, n), 2.0) + torch.rand(B, H, n, generator=g) * 1e-9      # range below the 1e-8 floor
    # scores that are not finite (a NaN or inf in the buffered rows or the query): torch's min / max / sort set the rule
    # (a NaN makes every normalised score 0.5, an inf makes its own NaN and the finite ones 0, NaN sorts last), and
    # every token still gets a level of its head's table
    if kind == "nan":
        scores[0, 1, 5] = float("nan")
        scores[-1, 0, n - 1] = float("nan")
    if kind == "inf":
        scores[0, 0, 1] = float("inf")
        scores[0, H - 1, 0] = float("inf")
        scores[0, H - 1, n - 1] = float("inf")
    if kind == "neginf":
        scores[0, 0, 3] = float("-inf")
    observed = {h: ((0, 0.3), (2, 0.4), (3, 0.1 + 0.01 * h), (4, 0.15), (8, 0.05)) for h in range(H)}
    allowed = (2, 3, 4, 8, 16)
    s_dev = scores.to(DEV).contiguous()
    minmax = torch.stack([s_dev.reshape(B * H, n).min(-1).values, s_dev.reshape(B * H, n).max(-1).values], -1).contiguous()
    got = _rank(s_dev, minmax, B, H, n, observed, set(allowed)).cpu()
    norm = ofl.minmax(scores.reshape(-1))                                       # what the press hands to the ranking
    want = ofl.cached_ratio_bits(norm, _positions(B, H, n), H, observed, allowed)
    assert torch.equal(got.reshape(-1), want)
    assert not (got == 0).any()


def test_exact_tail_is_the_buffer_gather():
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    g = torch.Generator().manual_seed(5)
    B, H, T, n = 2, 3, 300, 70
    k = torch.randn(B, H, T, 128, generator=g).half().to(DEV)
    v = torch.randn(B, H, T, 128, generator=g).half().to(DEV)
    bits = torch.full((B, H, T), 2, dtype=torch.int32)
    bits[..., :4] = 16
    bits[..., -20:] = 16
    st = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=DEV, dtype=torch.float16, key_quantizer="mse",
                                        value_quantizer="mse", seed=42)
    st.prefill(k, v, bits.to(DEV))
    new_k = torch.randn(n, B, H, 1, 128, generator=g).half().to(DEV)
    new_v = torch.randn(n, B, H, 1, 128, generator=g).half().to(DEV)
    for i in range(n):
        st.append_all_exact(new_k[i], new_v[i])
    pos, rows_k, rows_v = st.get_buffer_tokens(T)                               # the general gather (reads positions back)
    tk, tv = st.exact_tail(n)
    assert torch.equal(tk.reshape(-1, 128), rows_k) and torch.equal(tv.reshape(-1, 128), rows_v)
    assert torch.equal(tk, new_k[:, :, :, 0].permute(1, 2, 0, 3))
    assert (pos.cpu().numpy() == _positions(B, H, n, start=T)).all()
    assert st.exact_tail(n + 25) is None                                        # more than the shortest exact segment holds
    # a flush handed the rows and (one sequence or not) no counts stores the same as the general one
    lv = torch.tensor((2, 3, 4, 8), dtype=torch.int32)[torch.randint(0, 4, (B, H, n), generator=g)].to(DEV)
    st.flush_buffer(T, lv, rows=(tk, tv))
    assert torch.equal(st._level_map[:, :, T:].to(torch.int32), lv) and st.seq_len == T + n
