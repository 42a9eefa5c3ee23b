"""Pins for the oracle's codebook, bit packer, rotation and (de)quantiser."""
import numpy as np
import pytest
import torch

from oracle import codebook as cb
from oracle import quantizer as qz

SIGMA = 1 / np.sqrt(128)


@pytest.mark.parametrize("d,b", [(128, 1), (128, 2), (128, 3), (128, 4), (128, 8), (64, 2), (64, 4)])
def test_codebook_bits_match_reference(golden, d, b):
    ref = golden[f"codebook_d{d}_b{b}"]
    mine = cb.lloyd_max_codebook(2 ** b, d)
    assert mine.dtype == np.float64
    np.testing.assert_array_equal(mine, ref)          # same doubles, not just close


def test_codebook_textbook_levels():
    # Max (1960), unit-variance Gaussian
    book = {1: [0.7979], 2: [0.4528, 1.510], 3: [0.2451, 0.7560, 1.344, 2.152]}
    for b, levels in book.items():
        c = cb.lloyd_max_codebook(2 ** b, 128) / SIGMA
        np.testing.assert_allclose(c[len(c) // 2:], levels, rtol=4e-3)
        np.testing.assert_allclose(c, -c[::-1], atol=1e-9)          # symmetric
        assert np.all(np.diff(c) > 0)


def test_codebook_distortion_table_and_bound():
    expect = {1: 0.3634, 2: 0.1175, 3: 0.03454, 4: 0.009497}
    for b, dist in expect.items():
        c = cb.lloyd_max_codebook(2 ** b, 128)
        got = cb.distortion(c, 128) / SIGMA ** 2
        assert abs(got - dist) / dist < 2e-3
        assert got <= np.sqrt(3) * np.pi / 2 / 4 ** b          # Panter-Dite high-resolution constant


def test_pdf_matches_scipy():
    from scipy import stats
    x = np.linspace(-5 * SIGMA, 5 * SIGMA, 1001)
    np.testing.assert_array_equal(cb.coordinate_pdf(x, 128), stats.norm.pdf(x, loc=0, scale=SIGMA))


@pytest.mark.parametrize("b", [1, 2, 3, 4, 8])
def test_pack_bytes_match_reference(golden, b):
    codes = golden[f"pack_b{b}_codes"]
    np.testing.assert_array_equal(qz.pack_codes(codes, b), golden[f"pack_b{b}_bytes"])
    np.testing.assert_array_equal(qz.unpack_codes(golden[f"pack_b{b}_bytes"], b, 128), codes)
    np.testing.assert_array_equal(golden[f"pack_b{b}_roundtrip"], codes)


def test_pack_layout_by_hand():
    # 2-bit: value i of a byte sits at bit 2*i; 3- and 4-bit ride in nibbles
    assert qz.pack_codes(np.array([[1, 2, 3, 0]]), 2).tolist() == [[1 | 2 << 2 | 3 << 4]]
    assert qz.pack_codes(np.array([[5, 7]]), 3).tolist() == [[5 | 7 << 4]]
    assert qz.pack_codes(np.array([[9, 15]]), 4).tolist() == [[9 | 15 << 4]]
    assert qz.pack_codes(np.array([[1, 0, 1, 1, 0, 0, 0, 1]]), 1).tolist() == [[0b10001101]]
    assert qz.pack_codes(np.array([[200, 3]]), 8).tolist() == [[200, 3]]
    # ragged tail is zero padded
    assert qz.pack_codes(np.array([[3, 1, 2]]), 2).tolist() == [[3 | 1 << 2 | 2 << 4]]


def test_rotation_matches_reference_and_is_orthogonal(golden):
    pi = qz.random_rotation(128, 42)
    np.testing.assert_allclose(pi.numpy(), golden["pi_seed42"], atol=1e-6)
    eye = (pi.double() @ pi.double().T).numpy()
    np.testing.assert_allclose(eye, np.eye(128), atol=1e-5)


def test_dequantize_matches_reference(golden):
    pi = torch.from_numpy(golden["pi_seed42"])
    np.testing.assert_array_equal(cb.codebook_f32(4, 128), golden["deq_b4_centroids"])
    q = qz.Quantized(golden["deq_b4_codes"], golden["deq_b4_norms"], 4)
    np.testing.assert_allclose(qz.dequantize(q, pi).numpy(), golden["deq_b4_out"], rtol=1e-6, atol=1e-7)


def test_nearest_centroid_is_brute_force_argmin():
    rng = np.random.default_rng(0)
    for b in (2, 3, 4, 8):
        c = cb.codebook_f32(b, 128)
        y = (rng.standard_normal(20000) * SIGMA * 1.5).astype(np.float32)
        y[:4] = [c[0] - 1, c[-1] + 1, c[0], c[-1]]
        brute = np.abs(y[:, None] - c[None, :]).argmin(axis=1)
        np.testing.assert_array_equal(qz.nearest_centroid(y, c), brute)
    # exactly on a midpoint the lower index is kept
    c = np.array([-1.0, 0.0, 2.0], np.float32)
    assert qz.nearest_centroid(np.array([-0.5, 1.0], np.float32), c).tolist() == [0, 1]


def test_quantize_identity_rotation_two_levels_is_sign():
    x = torch.tensor([[3.0, -4.0, 0.5, -0.25]])
    c = cb.codebook_f32(1, 4)           # two centroids, symmetric
    q = qz.quantize(x, torch.eye(4), 1)
    assert q.codes.tolist() == [[1, 0, 1, 0]]
    np.testing.assert_allclose(q.norms, [np.sqrt(9 + 16 + 0.25 + 0.0625)], rtol=1e-6)
    back = qz.dequantize(q, torch.eye(4)).numpy()
    np.testing.assert_allclose(np.abs(back), abs(c[1]) * q.norms[0], rtol=1e-6)
    assert (np.sign(back) == np.sign(x.numpy())).all()


def test_roundtrip_mse_matches_lloyd_max_table():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2048, 128, generator=g).half()
    pi = qz.random_rotation(128, 42)
    expect = {2: 0.1175, 3: 0.03454, 4: 0.009497}
    for b, dist in expect.items():
        rec = qz.dequantize(qz.quantize(x, pi, b), pi)
        rel = ((x.float() - rec) ** 2).sum() / (x.float() ** 2).sum()
        assert abs(rel.item() - dist) / dist < 0.03


@pytest.mark.parametrize("b", [2, 3, 4, 8])
def test_canonical_order_agrees_with_blas_except_near_midpoints(b):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(512, 128, generator=g).half()
    pi = qz.random_rotation(128, 42)
    (qa, ya), (qb, yb) = qz.quantize(x, pi, b, want_y=True), qz.quantize(x, pi, b, order="canonical", want_y=True)
    np.testing.assert_allclose(qa.norms, qb.norms, rtol=3e-7)
    diff = qa.codes != qb.codes
    assert diff.mean() < 2e-3
    if diff.any():
        c = cb.codebook_f32(b, 128)
        mids = (c[:-1] + c[1:]) / 2
        assert np.all(np.abs(qa.codes[diff].astype(int) - qb.codes[diff].astype(int)) == 1)
        dist = np.abs(ya[diff][:, None] - mids[None, :]).min(axis=1)
        assert dist.max() < 1e-6
    # the canonical y itself is the sequential-fma dot product
    u = (x[0].float() / (qb.norms[0] + np.float32(1e-10))).numpy()
    acc = np.float32(0)
    row = pi.numpy()[7]
    for j in range(128):
        acc = np.float32(np.float64(u[j]) * np.float64(row[j]) + np.float64(acc))   # one rounding = fma
    assert acc == yb[0, 7]
