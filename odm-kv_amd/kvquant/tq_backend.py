"""TurboQuant-MSE quantiser front end: rotation, codebooks, quantise / dequantise on the GPU.

Mirrors the names of the reference's kvquant/tq_backend.py that the hot path uses:
``random_rotation`` (:25-36), ``_load_or_compute_codebook`` (:39-46), ``MSEQuantized`` (:49-53),
``_pack_indices`` / ``_unpack_indices`` (:103-145), ``TurboQuantMSE`` (:165-203) and the two
``normalize_*_quantizer`` helpers (:72-100).  The arithmetic runs in libodmkv (HIP).

Differences that are deliberate and documented:
  * the rotation is always drawn from the CPU generator and then moved to the device, so a
    given seed names the same matrix on every machine (the reference draws it on whatever
    device it is asked for, and CPU and GPU streams differ);
  * only key/value quantiser "mse" and widths 2, 3, 4, 8 are implemented (the paper
    configuration); "prod" keys and min-max values raise ``NotImplementedError``.
"""
from __future__ import annotations

from typing import NamedTuple, Optional

import numpy as np
import torch

from codebook import compute_codebook

from . import _lib
from ._lib import lib

_CODEBOOK_CACHE: dict[tuple[int, int], torch.Tensor] = {}
_TABLE_CACHE: dict[tuple[int, str], torch.Tensor] = {}
_ROTATION_CACHE: dict[tuple[int, int, str], torch.Tensor] = {}

SUPPORTED_WIDTHS = _lib.WIDTHS


def random_rotation(dim: int, device, dtype: torch.dtype = torch.float32,
                    seed: Optional[int] = None) -> torch.Tensor:
    """Pi = Q * sign(diag R) from the QR factorisation of a seeded Gaussian matrix."""
    gen = None
    if seed is not None:
        gen = torch.Generator(device="cpu")
        gen.manual_seed(int(seed))
    mat = torch.randn(dim, dim, dtype=torch.float32, generator=gen)
    q, r = torch.linalg.qr(mat)
    diag = torch.diag(r)
    signs = torch.where(diag >= 0, torch.ones_like(diag), -torch.ones_like(diag))
    return (q * signs.unsqueeze(0)).to(device=device, dtype=dtype)


def cached_rotation(dim: int, device, seed: int) -> torch.Tensor:
    key = (dim, int(seed), str(device))
    pi = _ROTATION_CACHE.get(key)
    if pi is None:
        pi = random_rotation(dim, device, torch.float32, seed).contiguous()
        _ROTATION_CACHE[key] = pi
    return pi


def lloyd_max_on_device(k: int, dim: int, device, n_iter: int = 500, tol: float = 1e-10,
                        x_range: float = 5.0) -> np.ndarray:
    """compute_codebook(k, dim) run by the GPU (odmkv_lloyd_max): fp64 centroids, ascending."""
    dev = torch.device(device)
    out = torch.empty(k, dtype=torch.float64, device=dev)
    _lib.check(lib.odmkv_lloyd_max(int(k), int(dim), int(n_iter), float(tol), float(x_range), out.data_ptr(), None,
                                   _lib.stream_ptr(dev)))
    return out.cpu().numpy()


def _load_or_compute_codebook(bits: int, dim: int, device, dtype: torch.dtype) -> torch.Tensor:
    """The 2^bits centroids as a tensor on `device` (kvquant/tq_backend.py:39-46).  Built once per (bits, dim): by
    the GPU when `device` is one and the density is the normal one (dim >= 100; 0.6 s of host time for the 8-bit
    table otherwise), by codebook.compute_codebook on the host else.  The two give the same fp32 numbers."""
    key = (bits, dim)
    cached = _CODEBOOK_CACHE.get(key)
    if cached is None:
        if torch.device(device).type == "cuda" and dim >= 100 and bits <= 8:
            c64 = lloyd_max_on_device(2 ** bits, dim, device)
        else:
            c64 = compute_codebook(2 ** bits, dim)
        cached = torch.from_numpy(c64.astype(np.float32))
        _CODEBOOK_CACHE[key] = cached
    return cached.to(device=device, dtype=dtype)


def codebook_table(dim: int, device) -> torch.Tensor:
    """The 2-, 3-, 4- and 8-bit tables back to back (4 + 8 + 16 + 256 fp32), on `device`."""
    key = (dim, str(device))
    tab = _TABLE_CACHE.get(key)
    if tab is None:
        parts = [_load_or_compute_codebook(b, dim, device, torch.float32) for b in SUPPORTED_WIDTHS]
        tab = torch.cat(parts).contiguous()
        _TABLE_CACHE[key] = tab
    return tab


_DECODE_TABLE_CACHE: dict[tuple[int, str], tuple[torch.Tensor, list[float]]] = {}


def _fp16_friendly_scale(c: np.ndarray, n_candidates: int = 100_000) -> float:
    """A scale S in [1, 2) for which every S * c_k is as close as possible to an fp16 number.

    The decode kernel keeps centroid tables in fp16.  Rounding c_k itself costs up to 2^-11
    relative per entry; rounding S * c_k for a well chosen S costs far less when the table has
    few distinct magnitudes (2 for the 2-bit table, 4 for the 3-bit one), and the common factor
    S is divided out of the per-token norm in fp32."""
    mags = np.unique(np.abs(c.astype(np.float64)))
    mags = mags[mags > 0]
    cand = np.exp2(np.linspace(0.0, 1.0, n_candidates, endpoint=False))
    prod = cand[:, None] * mags[None, :]
    err = np.abs(prod.astype(np.float16).astype(np.float64) - prod) / prod
    return float(cand[int(np.argmin(err.max(axis=1)))])


def decode_tables(dim: int, device) -> tuple[torch.Tensor, list[float]]:
    """(scaled centroid tables [284] on `device`, reciprocal scales per width) for the fused
    decode kernel."""
    key = (dim, str(device))
    got = _DECODE_TABLE_CACHE.get(key)
    if got is None:
        parts, inv = [], []
        for b in SUPPORTED_WIDTHS:
            c = _load_or_compute_codebook(b, dim, device, torch.float32).cpu().numpy()
            s = _fp16_friendly_scale(c)
            parts.append(torch.from_numpy((c.astype(np.float64) * s).astype(np.float32)))
            inv.append(float(np.float32(1.0 / s)))
        got = (torch.cat(parts).to(device).contiguous(), inv)
        _DECODE_TABLE_CACHE[key] = got
    return got


class MSEQuantized(NamedTuple):
    indices: torch.Tensor     # container bytes as the reference packs them
    norms: torch.Tensor
    bits: int


def normalize_value_quantizer(name: str) -> str:
    aliases = {"group": "minmax", "group_minmax": "minmax", "minmax": "minmax",
               "mse": "mse", "turboquant": "mse", "turboquant_mse": "mse"}
    key = str(name).strip().lower()
    if key not in aliases:
        raise ValueError(f"Unsupported value quantizer: {name!r}")
    return aliases[key]


def normalize_key_quantizer(name: str) -> str:
    aliases = {"prod": "prod", "turboquant_prod": "prod", "turboquantprod": "prod",
               "mse": "mse", "turboquant_mse": "mse", "turboquantmse": "mse"}
    key = str(name).strip().lower()
    if key not in aliases:
        raise ValueError(f"Unsupported key quantizer: {name!r}")
    return aliases[key]


def _container(bits: int) -> tuple[int, int]:
    if bits == 1:
        return 8, 1
    if bits == 2:
        return 4, 2
    if bits <= 4:
        return 2, 4
    return 1, 8


def _pack_indices(indices: torch.Tensor, bits: int) -> torch.Tensor:
    """One code per element -> the reference's container bytes (value i at bit i*eff of its byte;
    3-bit codes ride in nibbles)."""
    per, eff = _container(bits)
    idx = indices.to(torch.uint8)
    if per == 1:
        return idx
    d = idx.shape[-1]
    pad = (-d) % per
    if pad:
        idx = torch.nn.functional.pad(idx, (0, pad), value=0)
    grouped = idx.reshape(*idx.shape[:-1], -1, per).to(torch.int32)
    shifts = torch.arange(per, device=idx.device, dtype=torch.int32) * eff
    return (grouped << shifts).sum(dim=-1).to(torch.uint8)


def _unpack_indices(packed: torch.Tensor, bits: int, dim: int) -> torch.Tensor:
    per, eff = _container(bits)
    if per == 1:
        return packed.long()
    shifts = torch.arange(per, device=packed.device, dtype=torch.int32) * eff
    vals = (packed.to(torch.int32).unsqueeze(-1) >> shifts) & ((1 << eff) - 1)
    return vals.reshape(*packed.shape[:-1], -1)[..., :dim].long()


class TurboQuantMSE:
    """Unit-normalise, rotate by Pi, snap every coordinate to a Lloyd-Max centroid."""

    def __init__(self, dim: int, bits: int, *, device, dtype: torch.dtype, seed: int = 42):
        if dim != _lib.HEAD_DIM:
            raise ValueError(f"the HIP kernels are written for head_dim {_lib.HEAD_DIM}, got {dim}")
        if bits not in SUPPORTED_WIDTHS:
            raise ValueError(f"bit width {bits} is not one of {SUPPORTED_WIDTHS}")
        self.dim, self.bits = dim, bits
        self.device = torch.device(device)
        self.dtype = dtype
        self.compute_dtype = torch.float32
        self.pi = cached_rotation(dim, self.device, seed)
        self.centroids = _load_or_compute_codebook(bits, dim, self.device, torch.float32).contiguous()

    def quantize_codes(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """x [..., d] -> (codes uint8 [..., d] one per byte, norms fp32 [...])."""
        _lib.require_gpu(x, "x")
        flat = x.reshape(-1, self.dim)
        if flat.stride(-1) != 1:
            flat = flat.contiguous()
        n = flat.shape[0]
        codes = torch.empty(n, self.dim, dtype=torch.uint8, device=x.device)
        norms = torch.empty(n, dtype=torch.float32, device=x.device)
        _lib.check(lib.odmkv_quantize_rows(
            flat.data_ptr(), _lib.dtype_code(flat), n, flat.stride(0), self.bits,
            self.pi.data_ptr(), self.centroids.data_ptr(), codes.data_ptr(), norms.data_ptr(),
            _lib.stream_ptr(x.device)))
        return codes.reshape(*x.shape), norms.reshape(x.shape[:-1])

    def quantize(self, x: torch.Tensor) -> MSEQuantized:
        codes, norms = self.quantize_codes(x)
        return MSEQuantized(indices=_pack_indices(codes, self.bits), norms=norms, bits=self.bits)

    def dequantize(self, q: MSEQuantized) -> torch.Tensor:
        codes = _unpack_indices(q.indices, q.bits, self.dim).to(torch.uint8)
        flat = codes.reshape(-1, self.dim).contiguous()
        norms = q.norms.float().reshape(-1).contiguous()
        out = torch.empty(flat.shape[0], self.dim, dtype=torch.float32, device=flat.device)
        _lib.check(lib.odmkv_dequantize_rows(
            flat.data_ptr(), norms.data_ptr(), flat.shape[0], q.bits, self.pi.data_ptr(),
            self.centroids.data_ptr(), out.data_ptr(), _lib.stream_ptr(flat.device)))
        return out.reshape(*codes.shape)
