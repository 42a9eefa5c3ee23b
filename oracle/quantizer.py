"""Oracle: TurboQuant-MSE quantise / pack / dequantise on the CPU.

Follows /root/reference/kvquant/tq_backend.py:
  random_rotation            :25-36
  _pack_indices              :103-125
  _unpack_indices            :128-145
  TurboQuantMSE.quantize     :185-197
  TurboQuantMSE.dequantize   :199-203

``quantize(..., order="blas")`` runs the reference's op sequence on torch CPU
kernels (summation order left to the library, as in the reference).
``order="canonical"`` runs the fixed-order C restatement in ``canon.c`` that the
HIP kernel mirrors operation for operation; codes from the two agree except where
a rotated coordinate falls within rounding distance of a cell midpoint.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import NamedTuple

import numpy as np
import torch

from .codebook import codebook_f32

_HERE = os.path.dirname(os.path.abspath(__file__))
_CANON_SO = os.path.join(_HERE, "_build", "libodmkv_canon.so")
_canon = None


def build_canon(force: bool = False) -> str:
    """Compile ``canon.c`` with gcc into ``oracle/_build`` (fmaf kept, no contraction)."""
    src = os.path.join(_HERE, "canon.c")
    if force or not os.path.exists(_CANON_SO) or os.path.getmtime(_CANON_SO) < os.path.getmtime(src):
        os.makedirs(os.path.dirname(_CANON_SO), exist_ok=True)
        subprocess.check_call([
            "gcc", "-O2", "-mfma", "-ffp-contract=off", "-fno-fast-math", "-shared", "-fPIC",
            "-o", _CANON_SO, src, "-lm",
        ])
    return _CANON_SO


def _load_canon():
    global _canon
    if _canon is None:
        if not os.path.exists(_CANON_SO):
            build_canon()
        lib = ctypes.CDLL(_CANON_SO)
        lib.odmkv_canon_quantize.argtypes = [
            ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p,
            ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        lib.odmkv_canon_quantize.restype = None
        lib.odmkv_canon_nearest.argtypes = [
            ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        lib.odmkv_canon_nearest.restype = None
        _canon = lib
    return _canon


# ---------------------------------------------------------------------------
# rotation (tq_backend.py:25-36) -- always from the CPU generator
# ---------------------------------------------------------------------------

def random_rotation(dim: int, seed: int) -> torch.Tensor:
    """Pi = Q * sign(diag R) of a seeded Gaussian matrix; fp32 [dim, dim]."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    mat = torch.randn(dim, dim, dtype=torch.float32, generator=gen)
    q, r = torch.linalg.qr(mat)
    diag = torch.diag(r)
    signs = torch.where(diag >= 0, torch.ones_like(diag), -torch.ones_like(diag))
    return q * signs.unsqueeze(0)


# ---------------------------------------------------------------------------
# container bytes of the reference (tq_backend.py:103-145)
# ---------------------------------------------------------------------------

def _container(bits: int) -> tuple[int, int]:
    """(values per byte, bits per value) of the reference's container."""
    if bits == 1:
        return 8, 1
    if bits == 2:
        return 4, 2
    if bits <= 4:
        return 2, 4          # 3-bit codes ride in nibbles
    return 1, 8


def pack_codes(codes: np.ndarray, bits: int) -> np.ndarray:
    """uint8 codes [..., d] -> reference container bytes (value i at bit i*eff of its byte)."""
    per, eff = _container(bits)
    codes = np.asarray(codes, dtype=np.uint8)
    if per == 1:
        return codes.copy()
    d = codes.shape[-1]
    pad = (-d) % per
    if pad:
        codes = np.concatenate([codes, np.zeros(codes.shape[:-1] + (pad,), np.uint8)], axis=-1)
    grouped = codes.reshape(codes.shape[:-1] + (-1, per)).astype(np.uint16)
    shifts = (np.arange(per) * eff).astype(np.uint16)
    return (grouped << shifts).sum(axis=-1).astype(np.uint8)


def unpack_codes(packed: np.ndarray, bits: int, d: int) -> np.ndarray:
    per, eff = _container(bits)
    packed = np.asarray(packed, dtype=np.uint8)
    if per == 1:
        return packed.copy()
    shifts = (np.arange(per) * eff).astype(np.uint8)
    vals = (packed[..., None] >> shifts) & np.uint8((1 << eff) - 1)
    return vals.reshape(packed.shape[:-1] + (-1,))[..., :d]


# ---------------------------------------------------------------------------
# nearest centroid -- the reference's routine is not shipped (tq_backend.py:195);
# this is the op sequence its comment names (tq_backend.py:191-194)
# ---------------------------------------------------------------------------

def nearest_centroid(y: np.ndarray, c: np.ndarray) -> np.ndarray:
    y = np.asarray(y, dtype=np.float32)
    c = np.asarray(c, dtype=np.float32)
    pos = np.searchsorted(c, y, side="left")
    pos = np.clip(pos, 1, len(c) - 1)
    dl = np.abs(y - c[pos - 1])
    dh = np.abs(y - c[pos])
    return np.where(dh < dl, pos, pos - 1).astype(np.uint8)


class Quantized(NamedTuple):
    codes: np.ndarray     # uint8 [N, d], one code per byte (the unpacked indices)
    norms: np.ndarray     # fp32 [N]
    bits: int


def quantize(x: torch.Tensor, pi: torch.Tensor, bits: int, *, order: str = "blas",
             want_y: bool = False):
    """x [N, d] (any float dtype) -> Quantized (tq_backend.py:185-197)."""
    d = x.shape[-1]
    c = codebook_f32(bits, d)
    xf = x.detach().cpu().float().contiguous()
    if order == "blas":
        norms = xf.norm(dim=-1)
        unit = xf / (norms.unsqueeze(-1) + 1e-10)
        y = (unit @ pi.float().T).numpy()
        q = Quantized(nearest_centroid(y, c), norms.numpy().copy(), bits)
        return (q, y) if want_y else q
    if order != "canonical":
        raise ValueError(order)
    lib = _load_canon()
    n = xf.shape[0]
    xin = xf.numpy()
    pin = np.ascontiguousarray(pi.detach().cpu().float().numpy())
    norms = np.empty(n, np.float32)
    codes = np.empty((n, d), np.uint8)
    y = np.empty((n, d), np.float32) if want_y else None
    lib.odmkv_canon_quantize(xin.ctypes.data, n, d, pin.ctypes.data, c.ctypes.data, len(c),
                             norms.ctypes.data, codes.ctypes.data,
                             y.ctypes.data if want_y else None)
    q = Quantized(codes, norms, bits)
    return (q, y) if want_y else q


def dequantize(q: Quantized, pi: torch.Tensor) -> torch.Tensor:
    """x_hat = (centroids[codes] @ Pi) * norm, fp32 (tq_backend.py:199-203)."""
    d = q.codes.shape[-1]
    c = torch.from_numpy(codebook_f32(q.bits, d))
    y_hat = c[torch.from_numpy(q.codes.astype(np.int64))]
    x_hat = y_hat @ pi.float()
    return x_hat * torch.from_numpy(q.norms).float().unsqueeze(-1)
