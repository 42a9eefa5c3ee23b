"""GPU parity: TurboQuant-MSE quantiser, packed store, dequantise (through the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import quantizer as oq
from oracle.codebook import codebook_f32
from oracle.kvstate import KVState

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand_bits(g, shape, levels=(0, 2, 3, 4, 8, 16), probs=(0.25, 0.4, 0.12, 0.1, 0.08, 0.05)):
    idx = torch.multinomial(torch.tensor(probs), int(np.prod(shape)), replacement=True, generator=g)
    return torch.tensor(levels, dtype=torch.int32)[idx].reshape(shape)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_quantize_rows_bit_exact(bits, dtype):
    from kvquant.tq_backend import TurboQuantMSE
    g = torch.Generator().manual_seed(100 + bits)
    x = (torch.randn(1000, 128, generator=g) * torch.exp(torch.randn(1000, 1, generator=g))).to(dtype)
    x[5] = 0                                                   # a zero row must not blow up
    q = TurboQuantMSE(128, bits, device=DEV, dtype=dtype, seed=42)
    np.testing.assert_array_equal(q.centroids.cpu().numpy(), codebook_f32(bits, 128))
    codes, norms = q.quantize_codes(x.to(DEV))
    ref = oq.quantize(x, q.pi.cpu(), bits, order="canonical")
    np.testing.assert_array_equal(norms.cpu().numpy(), ref.norms)          # same fp32 bits
    np.testing.assert_array_equal(codes.cpu().numpy(), ref.codes)          # every code identical
    # against the library-ordered (BLAS) statement: only coordinates on a cell boundary may move
    blas = oq.quantize(x, q.pi.cpu(), bits, order="blas")
    diff = blas.codes != codes.cpu().numpy()
    assert diff.mean() < 2e-3
    assert np.all(np.abs(blas.codes[diff].astype(int) - codes.cpu().numpy()[diff].astype(int)) == 1)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_container_roundtrip_and_dequantize(bits):
    from kvquant.tq_backend import TurboQuantMSE, _unpack_indices
    g = torch.Generator().manual_seed(1007)      # not the rotation's seed: see calibrate_epsilon's quirk
    x = torch.randn(300, 128, generator=g).half()
    q = TurboQuantMSE(128, bits, device=DEV, dtype=torch.float16, seed=7)
    mq = q.quantize(x.to(DEV))
    codes, _ = q.quantize_codes(x.to(DEV))
    np.testing.assert_array_equal(mq.indices.cpu().numpy(), oq.pack_codes(codes.cpu().numpy(), bits))
    assert torch.equal(_unpack_indices(mq.indices, bits, 128), codes.long())
    rec = q.dequantize(mq).cpu()
    ref = oq.dequantize(oq.Quantized(codes.cpu().numpy(), mq.norms.cpu().numpy(), bits), q.pi.cpu())
    # fp32 with a different summation order: 1e-5 relative to the row norm
    err = (rec - ref).norm(dim=-1) / ref.norm(dim=-1)
    assert err.max() < 1e-5
    rel = ((x.float() - rec) ** 2).sum() / (x.float() ** 2).sum()
    assert rel < {2: 0.13, 3: 0.04, 4: 0.011, 8: 1e-4}[bits]


def _state(levels=(0, 2, 3, 4, 8, 16), dtype=torch.float16, seed=42):
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    return TurboQuantAdaptiveKVCacheState(128, levels, device=DEV, dtype=dtype, key_quantizer="mse",
                                          value_quantizer="mse", seed=seed)


def _check_store_against_oracle(state, ref: KVState):
    from packed_layout import decode_exact, decode_level
    H = state.num_heads
    for li, w in enumerate((2, 3, 4, 8)):
        bank = ref.banks.get(w)
        got = decode_level(state, li)
        n_ref = 0 if bank is None else bank.size
        assert len(got["pos"]) == n_ref, f"level {w}: {len(got['pos'])} stored, oracle {n_ref}"
        if n_ref == 0:
            continue
        # oracle banks are in (b, h, t) order within an append; sort both by (bh, pos)
        key_ref = bank.pos[:, 0] * H * 10 ** 7 + bank.pos[:, 1] * 10 ** 7 + bank.pos[:, 2]
        key_got = got["bh"].astype(np.int64) * 10 ** 7 + got["pos"]
        o_ref, o_got = np.argsort(key_ref, kind="stable"), np.argsort(key_got, kind="stable")
        np.testing.assert_array_equal(key_got[o_got], key_ref[o_ref])
        np.testing.assert_array_equal(got["kcodes"][o_got], bank.kc[o_ref])
        np.testing.assert_array_equal(got["vcodes"][o_got], bank.vc[o_ref])
        np.testing.assert_array_equal(got["knorm"][o_got], bank.kn[o_ref])
        np.testing.assert_array_equal(got["vnorm"][o_got], bank.vn[o_ref])
        # ascending positions inside every segment
        for s in np.unique(got["bh"]):
            assert np.all(np.diff(got["pos"][got["bh"] == s]) > 0)
    ex = decode_exact(state)
    assert len(ex["pos"]) == ref.exact.size
    if ref.exact.size:
        key_ref = ref.exact.pos[:, 0] * H * 10 ** 7 + ref.exact.pos[:, 1] * 10 ** 7 + ref.exact.pos[:, 2]
        key_got = ex["bh"].astype(np.int64) * 10 ** 7 + ex["pos"]
        o_ref, o_got = np.argsort(key_ref, kind="stable"), np.argsort(key_got, kind="stable")
        np.testing.assert_array_equal(key_got[o_got], key_ref[o_ref])
        np.testing.assert_array_equal(ex["k"][o_got], ref.exact.k.view(torch.int16).numpy()[o_ref])
        np.testing.assert_array_equal(ex["v"][o_got], ref.exact.v.view(torch.int16).numpy()[o_ref])


def _ulp_close_fp16(a: torch.Tensor, b: torch.Tensor, max_ulp=1, max_frac=0.02, sum_noise=1e-6):
    """a equals b up to how an fp32 sum of 128 terms depends on its order (the oracle sums in the canonical
    order, the kernel on the matrix cores): `sum_noise` of the row's norm before the rounding to fp16, hence at
    most one fp16 step, or that noise where it is larger than a step (elements near zero), and few such."""
    ai, bi = a.view(torch.int16).int(), b.view(torch.int16).int()
    ai = torch.where(ai < 0, -32768 - ai, ai)          # map sign-magnitude to a monotone scale
    bi = torch.where(bi < 0, -32768 - bi, bi)
    d = (ai - bi).abs()
    small = (a.float() - b.float()).abs() <= sum_noise * b.float().norm(dim=-1, keepdim=True)
    assert int(d[~small].max() if (~small).any() else 0) <= max_ulp, f"max fp16 ulp distance {int(d[~small].max())}"
    assert float((d > 0).float().mean()) <= max_frac


@pytest.mark.parametrize("B,H,T", [(1, 2, 300), (2, 3, 129), (1, 8, 1000)])
def test_prefill_codes_positions_and_materialize(B, H, T):
    g = torch.Generator().manual_seed(B * 1000 + T)
    k = torch.randn(B, H, T, 128, generator=g).half()
    v = (torch.randn(B, H, T, 128, generator=g) * 2).half()
    bits = _rand_bits(g, (B, H, T))
    bits[..., -5:] = 16
    state = _state()
    state.prefill(k.to(DEV), v.to(DEV), bits.to(DEV))
    ref = KVState(128, (0, 2, 3, 4, 8, 16), seed=42, order="canonical")
    ref.prefill(k, v, bits)
    assert state.seq_len == T and state.batch_size == B and state.num_heads == H
    _check_store_against_oracle(state, ref)
    assert state.packed_bytes() == ref.packed_bytes()
    # dense read-back
    km, vm = state.materialize()
    kr, vr = ref.materialize()
    _ulp_close_fp16(km.cpu(), kr)
    _ulp_close_fp16(vm.cpu(), vr)
    evicted = torch.from_numpy(ref.level_map() == 0)
    assert torch.all(km.cpu()[evicted] == 0) and torch.all(vm.cpu()[evicted] == 0)
    exact = torch.from_numpy(ref.level_map() == 16)
    assert torch.equal(km.cpu()[exact], k[exact]) and torch.equal(vm.cpu()[exact], v[exact])
    # in-place variant leaves exact and evicted positions untouched
    k2, v2 = k.clone().to(DEV), v.clone().to(DEV)
    state.materialize_quantized_into(k2, v2)
    untouched = evicted | exact
    assert torch.equal(k2.cpu()[untouched], k[untouched])
    assert torch.equal(k2.cpu()[~untouched], km.cpu()[~untouched])
    # evicted index lists agree
    mi, ri = state.masked_key_indices(), ref.masked_key_indices()
    assert (mi is None) == (ri is None)
    if mi is not None:
        for a, b in zip(mi, ri):
            assert torch.equal(a.cpu(), b)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_dequantise_into_other_cache_dtypes(out_dtype):
    """The dense read-back into fp32 and bf16 tensors (the store itself holds fp16 exact rows):
    quantised positions equal the oracle's fp32 dequantisation (to the output type's rounding),
    exact positions are the stored fp16 rows converted, evicted ones are left alone."""
    g = torch.Generator().manual_seed(31)
    B, H, T = 2, 3, 257
    k = torch.randn(B, H, T, 128, generator=g).half(); v = (torch.randn(B, H, T, 128, generator=g) * 3).half()
    bits = _rand_bits(g, (B, H, T)); bits[..., :2] = 16
    state = _state()
    state.prefill(k.to(DEV), v.to(DEV), bits.to(DEV))
    ref = KVState(128, (0, 2, 3, 4, 8, 16), dtype=torch.float32, seed=42, order="canonical")
    ref.prefill(k.float(), v.float(), bits)
    kr, vr = ref.materialize()
    kd = torch.full((B, H, T, 128), 7.0, dtype=out_dtype, device=DEV); vd = torch.full_like(kd, 7.0)
    state._dequant_into(kd, vd, True)
    lm = torch.from_numpy(ref.level_map())
    quant = (lm != 0) & (lm != 16)
    tol = 2e-5 if out_dtype == torch.float32 else 2 ** -8
    for got, want in ((kd, kr), (vd, vr)):
        got = got.float().cpu()
        err = (got[quant] - want[quant]).norm(dim=-1) / want[quant].norm(dim=-1)
        assert err.max() < tol, float(err.max())
        assert torch.equal(got[lm == 16], want[lm == 16].to(out_dtype).float())
        assert torch.all(got[lm == 0] == 7.0)


def test_append_truncate_and_flush_follow_the_oracle():
    g = torch.Generator().manual_seed(77)
    B, H, D = 1, 4, 128
    k0 = torch.randn(B, H, 200, D, generator=g).half(); v0 = torch.randn(B, H, 200, D, generator=g).half()
    bits0 = _rand_bits(g, (B, H, 200)); bits0[..., -16:] = 16
    state, ref = _state(), KVState(128, (0, 2, 3, 4, 8, 16), seed=42, order="canonical")
    state.prefill(k0.to(DEV), v0.to(DEV), bits0.to(DEV)); ref.prefill(k0, v0, bits0)
    # a second block with its own bits (tail tiles are partially filled: read-modify-write on V)
    k1 = torch.randn(B, H, 70, D, generator=g).half(); v1 = torch.randn(B, H, 70, D, generator=g).half()
    bits1 = _rand_bits(g, (B, H, 70))
    state.append(k1.to(DEV), v1.to(DEV), bits1.to(DEV)); ref.append(k1, v1, bits1)
    _check_store_against_oracle(state, ref)
    # 40 single-token decode steps into the exact segments
    for _ in range(40):
        kn = torch.randn(B, H, 1, D, generator=g).half(); vn = torch.randn(B, H, 1, D, generator=g).half()
        state.append_all_exact(kn.to(DEV), vn.to(DEV)); ref.append_all_exact(kn, vn)
    assert state.seq_len == ref.seq_len == 310
    _check_store_against_oracle(state, ref)
    # flush the 40 buffered tokens to new levels
    pos, bk, bv = state.get_buffer_tokens(270)
    rpos, rk, rv = ref.get_buffer_tokens(270)
    assert pos.shape[0] == rpos.shape[0] == H * 40
    new_bits = _rand_bits(g, (H * 40,), probs=(0.0, 0.5, 0.2, 0.15, 0.1, 0.05))
    # the oracle's buffer order is step-major; ours is (b, h, t): map one onto the other
    key_ours = (pos[:, 1] * 10 ** 6 + pos[:, 2]).cpu().numpy()
    key_ref = rpos[:, 1] * 10 ** 6 + rpos[:, 2]
    lookup = {kk: i for i, kk in enumerate(key_ours)}
    perm = np.asarray([lookup[kk] for kk in key_ref])
    assert torch.equal(bk.cpu()[perm], rk) and torch.equal(bv.cpu()[perm], rv)
    state.flush_buffer(270, new_bits.to(DEV)); ref.flush_buffer(270, new_bits[perm])
    _check_store_against_oracle(state, ref)
    km, vm = state.materialize(); kr, vr = ref.materialize()
    _ulp_close_fp16(km.cpu(), kr); _ulp_close_fp16(vm.cpu(), vr)
    # rewind
    state.truncate(150); ref.truncate(150)
    assert state.seq_len == 150
    _check_store_against_oracle(state, ref)
    km, vm = state.materialize(); kr, vr = ref.materialize()
    assert km.shape == kr.shape
    _ulp_close_fp16(km.cpu(), kr)


def test_a_store_with_room_for_flushes_holds_the_same_tokens_and_does_not_move():
    """quant_headroom=True (what the press asks for when it will flush decode-time tokens into the quantised levels):
    the first fill, staged (T >= 256) or not, leaves a sixteenth more tiles (two at least) in every quantised
    segment; the stored tokens are the oracle's, and the tokens of a flush fit without the store being laid out again."""
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    g = torch.Generator().manual_seed(123)
    for T in (200, 700):
        B, H, D = 1, 3, 128
        k = torch.randn(B, H, T, D, generator=g).half(); v = torch.randn(B, H, T, D, generator=g).half()
        bits = _rand_bits(g, (B, H, T)); bits[..., -8:] = 16
        state = TurboQuantAdaptiveKVCacheState(128, (0, 2, 3, 4, 8, 16), device=DEV, dtype=torch.float16, key_quantizer="mse",
                                               value_quantizer="mse", seed=42, quant_headroom=True)
        plain = _state()
        ref = KVState(128, (0, 2, 3, 4, 8, 16), seed=42, order="canonical")
        state.prefill(k.to(DEV), v.to(DEV), bits.to(DEV)); plain.prefill(k.to(DEV), v.to(DEV), bits.to(DEV)); ref.prefill(k, v, bits)
        have, base = np.diff(state._seg_tile, axis=1), np.diff(plain._seg_tile, axis=1)
        assert np.array_equal(have[:4], base[:4] + np.maximum(base[:4] // 16, 2)) and np.array_equal(have[4], base[4])
        _check_store_against_oracle(state, ref)
        assert state.packed_bytes() == ref.packed_bytes()
        arena, tiles = state._bufs.arena.data_ptr(), state._seg_tile.copy()
        # 100 more tokens per head at the quantised levels: inside the room left
        k1 = torch.randn(B, H, 100, D, generator=g).half(); v1 = torch.randn(B, H, 100, D, generator=g).half()
        bits1 = _rand_bits(g, (B, H, 100), probs=(0.0, 0.4, 0.25, 0.2, 0.15, 0.0))
        state.append(k1.to(DEV), v1.to(DEV), bits1.to(DEV)); ref.append(k1, v1, bits1)
        assert state._bufs.arena.data_ptr() == arena and np.array_equal(state._seg_tile, tiles)
        _check_store_against_oracle(state, ref)
        km, vm = state.materialize(); kr, vr = ref.materialize()
        _ulp_close_fp16(km.cpu(), kr); _ulp_close_fp16(vm.cpu(), vr)


def test_edge_cases_and_errors():
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    g = torch.Generator().manual_seed(5)
    k = torch.randn(1, 2, 64, 128, generator=g).half().to(DEV)
    # everything evicted / everything exact / a single level
    for fill in (0, 16, 4):
        st = _state()
        st.prefill(k, k, torch.full((1, 2, 64), fill, dtype=torch.int32, device=DEV))
        km, _ = st.materialize()
        if fill == 0:
            assert torch.all(km == 0) and st.packed_bytes() == 0
        if fill == 16:
            assert torch.equal(km, k)
    st = _state()
    with pytest.raises(ValueError):
        st.prefill(k, k[:, :1], torch.zeros(1, 2, 64, dtype=torch.int32, device=DEV))
    with pytest.raises(ValueError):
        st.prefill(k, k, torch.zeros(1, 2, 63, dtype=torch.int32, device=DEV))
    with pytest.raises(ValueError):
        st.prefill(k, k, torch.full((1, 2, 64), 5, dtype=torch.int32, device=DEV))
    # the same on a first fill long enough to go through the staging store (its level counts come from the compaction's
    # chunk counts): a value that is no level, a level the store was not built for; the store stays usable afterwards
    k2 = torch.randn(1, 2, 2048 + 70, 128, generator=g).half().to(DEV)
    good = torch.full((1, 2, 2048 + 70), 2, dtype=torch.int32, device=DEV)
    good[0, 0, 100:300] = 4; good[0, 1, 2048:] = 16; good[0, 1, :9] = 0
    for bad_value, levels in ((5, (0, 2, 3, 4, 8, 16)), (3, (0, 2, 4, 16))):
        st = TurboQuantAdaptiveKVCacheState(128, levels, device=DEV, dtype=torch.float16, key_quantizer="mse", value_quantizer="mse", seed=42)
        bad = good.clone(); bad[0, 1, 2050] = bad_value
        with pytest.raises(ValueError):
            st.prefill(k2, k2, bad)
        st.prefill(k2, k2, good)
        assert st.level_counts() == {0: 9, 2: 2 * 2118 - 200 - 70 - 9, 3: 0, 4: 200, 8: 0, 16: 70}
        km, _ = st.materialize()
        assert torch.equal(km[0, 1, 2048:], k2[0, 1, 2048:]) and torch.all(km[0, 1, :9] == 0)
    with pytest.raises(ValueError):
        TurboQuantAdaptiveKVCacheState(128, (0, 1, 4), device=DEV, key_quantizer="prod", value_quantizer="mse")
    with pytest.raises(NotImplementedError):
        TurboQuantAdaptiveKVCacheState(128, (0, 2, 4), device=DEV)      # defaults are prod / minmax
    with pytest.raises(ValueError):
        TurboQuantAdaptiveKVCacheState(64, (0, 2, 4), device=DEV, key_quantizer="mse", value_quantizer="mse")


# ---- 16-bit tensors: the matrix-core estimate with exact codes next to the decision thresholds ----------
# fp16 and bf16 rows are quantised by a kernel that estimates the rotation on the 16-bit matrix cores and
# recomputes, by the definition's own chain, only the values within a guard band of a threshold; fp32 rows
# (and what that kernel hands over) go through the exact kernel alone.  The same numbers given in either
# type must therefore come out as the same bytes.
def _handed_over(state, B, H, T):
    import ctypes as C
    import os
    from kvquant import _lib
    blib = C.CDLL(os.path.join(os.path.dirname(_lib.__file__), "..", "lib", "libodmkv_bench.so"))
    ws = _lib.workspace(state.device, _lib.lib.odmkv_pack_workspace_bytes(B, H, T), "pack")     # the buffer the state's call used
    out = (C.c_int32 * 2)()
    blib.odmkv_bench_pack_handed_over.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int32), C.c_void_p]
    rc = blib.odmkv_bench_pack_handed_over(ws.data_ptr(), B, H, T, out, _lib.stream_ptr(state.device))
    assert rc == 0
    return int(out[0]), int(out[1])


def _same_bytes_in_both_types(k16, v16, bits):
    """Prefill the 16-bit tensors and their fp32 copies; compare every quantised level's buffers bit for bit.
    Returns the tiles the 16-bit call handed to the exact kernel (keys, values)."""
    B, H, T, _ = k16.shape
    s16, s32 = _state(dtype=k16.dtype), _state(dtype=k16.dtype)
    s16.prefill(k16, v16, bits)
    handed = _handed_over(s16, B, H, T)
    s32.prefill(k16.float(), v16.float(), bits)
    assert np.array_equal(s16._seg_tile, s32._seg_tile) and np.array_equal(s16._counts, s32._counts)
    for li in range(4):
        nt = int(s16._seg_tile[li, -1])
        if nt == 0:
            continue
        for name, per_tile in (("kcodes", 64 * 16 * (2, 3, 4, 8)[li]), ("vcodes", 64 * 16 * (2, 3, 4, 8)[li]),
                               ("knorm", 64), ("vnorm", 64), ("pos", 64)):
            a, b = s16._bufs[name][li].view(-1), s32._bufs[name][li].view(-1)
            n = nt * per_tile
            if a.dtype == torch.float32:
                a, b = a.view(torch.int32), b.view(torch.int32)
            bad = (a[:n] != b[:n]).nonzero()
            assert bad.numel() == 0, f"level index {li}, {name}: {bad.numel()} of {n} differ, first at {int(bad[0])}"
    return handed


def _rows_on_thresholds(state, pi, n_rows, per_row, width, g, dtype=torch.float16):
    """16-bit rows whose rotated unit vectors have `per_row` entries on decision thresholds of `width` bits
    (up to fp16 rounding of the row: a few 1e-5, well inside the guard band)."""
    cb = state.codebooks.cpu()
    off = {2: 0, 3: 4, 4: 12}[width]
    c = cb[off:off + (1 << width)].double()
    thr = (c[:-1] + c[1:]) / 2
    if per_row > 20:
        thr = thr[thr.abs() < 0.09]                                        # many entries: inner thresholds, so that the row stays a unit vector
    y = torch.randn(n_rows, 128, generator=g, dtype=torch.float64) / 128 ** 0.5
    for r in range(n_rows):
        idx = torch.randperm(128, generator=g)[:per_row]
        y[r, idx] = thr[torch.randint(len(thr), (per_row,), generator=g)]
        rest = torch.ones(128, dtype=torch.bool); rest[idx] = False
        left = 1.0 - float((y[r, idx] ** 2).sum())
        assert left > 0
        y[r, rest] *= (left / float((y[r, rest] ** 2).sum())) ** 0.5       # unit norm keeps the chosen entries where they are
    x = y @ pi.cpu().double()                                              # y = Pi x
    scale = torch.rand(n_rows, 1, generator=g, dtype=torch.float64) * 20 + 0.05
    return (x * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("per_row", [2, 100])
def test_fp16_rows_next_to_thresholds_get_the_exact_codes(per_row, dtype):
    g = torch.Generator().manual_seed(per_row)
    B, H, T = 1, 2, 1024
    probe = _state()
    bits = torch.tensor([2, 3, 4], dtype=torch.int32)[torch.randint(3, (B, H, T), generator=g)]
    k = torch.empty(B, H, T, 128, dtype=dtype)
    v = torch.empty(B, H, T, 128, dtype=dtype)
    for w in (2, 3, 4):
        m = bits == w
        n = int(m.sum())
        k[m] = _rows_on_thresholds(probe, probe.pi_k, n, per_row, w, g, dtype)
        v[m] = _rows_on_thresholds(probe, probe.pi_v, n, per_row, w, g, dtype)
    hk, hv = _same_bytes_in_both_types(k.to(DEV), v.to(DEV), bits.to(DEV))
    if per_row == 2:
        assert (hk, hv) == (0, 0)          # a couple of hundred listed values per tile: worked off in the kernel
    elif dtype == torch.float16:
        assert hk > 0 and hv > 0           # thousands per tile: the tiles go to the exact kernel
    # (bf16 rounds the rows a hundred times more coarsely than the guard band is wide: few entries stay inside it)
    # and the oracle agrees on a sample of the rows
    ref = KVState(128, (0, 2, 3, 4, 8, 16), dtype=dtype, seed=42, order="canonical")
    ref.prefill(k[:, :, :192], v[:, :, :192], bits[:, :, :192])
    st = _state(dtype=dtype)
    st.prefill(k[:, :, :192].to(DEV), v[:, :, :192].to(DEV), bits[:, :, :192].to(DEV))
    _check_store_against_oracle(st, ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fp16_special_rows_and_ordinary_ones(dtype):
    g = torch.Generator().manual_seed(11)
    B, H, T = 2, 2, 1500
    big, small = (65504.0, 6e-8) if dtype == torch.float16 else (1e18, 1e-10)
    k = torch.randn(B, H, T, 128, generator=g).to(dtype)
    v = (torch.randn(B, H, T, 128, generator=g) * 3).to(dtype)
    bits = _rand_bits(g, (B, H, T), levels=(0, 2, 3, 4, 16), probs=(0.1, 0.45, 0.25, 0.15, 0.05))
    hk, hv = _same_bytes_in_both_types(k.to(DEV), v.to(DEV), bits.to(DEV))
    assert (hk, hv) == (0, 0)              # no 8-bit tiles, ordinary rows: nothing for the exact kernel
    # rows of zeros, the largest and the smallest fp16 numbers, a huge outlier, infinities and NaNs
    k2, v2 = k.clone(), v.clone()
    k2[0, 0, 5] = 0; v2[0, 0, 5] = 0
    k2[0, 1, 70:80] = big; v2[0, 1, 70:80] = -big
    k2[1, 0, 200:210] = small; v2[1, 0, 200:210] *= 1e-4
    k2[1, 1, 300, 7] = 30000.0; v2[1, 1, 300, 90] = -30000.0
    k2[0, 0, 900, 3] = float("inf"); v2[0, 0, 901, 4] = float("nan")
    k2[1, 1, 1400, 0] = float("-inf"); v2[1, 1, 1400, 127] = float("inf")
    odd_k, odd_v = [(0, 0, 900), (1, 1, 1400)], [(0, 0, 901), (1, 1, 1400)]
    if dtype == torch.bfloat16:            # rows whose squares vanish in fp32 although the row is not zero
        k2[0, 1, 1000] = 1e-20; v2[0, 1, 1001] = -3e-21
        odd_k.append((0, 1, 1000)); odd_v.append((0, 1, 1001))
    hk, hv = _same_bytes_in_both_types(k2.to(DEV), v2.to(DEV), bits.to(DEV))
    lvl = bits.numpy()
    expect_k = sum(int(lvl[i] in (2, 3, 4)) for i in odd_k)
    expect_v = sum(int(lvl[i] in (2, 3, 4)) for i in odd_v)
    assert hk <= expect_k and hv <= expect_v       # (two such rows can share a tile)
    assert (hk > 0) == (expect_k > 0) and (hv > 0) == (expect_v > 0)
    # 8-bit tiles always go to the exact kernel
    bits8 = _rand_bits(g, (B, H, T))
    hk, hv = _same_bytes_in_both_types(k.to(DEV), v.to(DEV), bits8.to(DEV))
    n8 = sum(-(-int((bits8[b, h] == 8).sum()) // 64) for b in range(B) for h in range(H))
    assert (hk, hv) == (n8, n8)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 8])
def test_lloyd_max_on_the_device_gives_the_reference_tables(golden, bits):
    """odmkv_lloyd_max against the fp64 centroids the reference's compute_codebook returned (fixture) and against the
    host routine of the product: the same numbers to 1e-13 relative to the table's scale, and the same fp32 tables
    bit for bit (only the order of the additions inside a cell differs)."""
    from codebook import compute_codebook
    from kvquant.tq_backend import lloyd_max_on_device
    got = lloyd_max_on_device(2 ** bits, 128, DEV)
    ref = golden[f"codebook_d128_b{bits}"]
    host = compute_codebook(2 ** bits, 128)
    assert got.dtype == np.float64 and got.shape == ref.shape and np.all(np.diff(got) > 0)
    scale = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-13 * scale, np.abs(got - ref).max() / scale
    assert np.array_equal(got.astype(np.float32), ref.astype(np.float32))
    assert np.array_equal(got.astype(np.float32), host.astype(np.float32))
    # the argument checks: too many levels, a dimension whose density is not the normal one
    from kvquant import _lib
    out = torch.empty(512, dtype=torch.float64, device=DEV)
    assert _lib.lib.odmkv_lloyd_max(512, 128, 500, 1e-10, 5.0, out.data_ptr(), None, None) == -1
    assert _lib.lib.odmkv_lloyd_max(4, 64, 500, 1e-10, 5.0, out.data_ptr(), None, None) == -1
