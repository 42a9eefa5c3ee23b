"""ctypes binding of libodmkv.so, the C ABI declared in include/odmkv.h.

The HIP library is the only compute path: importing this module fails if the library
has not been built (``python odm-kv_amd/build.py``), and nothing falls back to PyTorch.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("ODMKV_LIB") or os.path.join(os.path.dirname(_HERE), "lib", "libodmkv.so")

F16, BF16, F32 = 0, 1, 2
HEAD_DIM = 128
TILE = 64
WIDTHS = (2, 3, 4, 8)                 # level index 0..3
LEVEL_ORDER = (0, 2, 3, 4, 8, 16)     # order of odmkv_level_counts columns
CODEBOOK_OFFSETS = (0, 4, 12, 28)
CODEBOOK_FLOATS = 284

_DT = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}


class Packed(C.Structure):
    """struct odmkv_packed of include/odmkv.h."""
    _fields_ = [
        ("B", C.c_int32), ("Hkv", C.c_int32), ("exact_dtype", C.c_int32),
        ("n_tiles", C.c_int32 * 5),
        ("kcodes", C.c_void_p * 4), ("vcodes", C.c_void_p * 4),
        ("knorm", C.c_void_p * 4), ("vnorm", C.c_void_p * 4),
        ("pos", C.c_void_p * 5), ("seg_tile", C.c_void_p * 5), ("seg_count", C.c_void_p * 5),
        ("kexact", C.c_void_p), ("vexact", C.c_void_p),
    ]


class Worklist(C.Structure):
    """struct odmkv_worklist of include/odmkv.h."""
    _fields_ = [
        ("items", C.c_void_p), ("item_range", C.c_void_p), ("dispatch_order", C.c_void_p),
        ("n_items", C.c_int32), ("wavefronts", C.c_int32), ("n_workgroups", C.c_int32), ("two_per_cu", C.c_int32),
    ]


class Step(C.Structure):
    """struct odmkv_step of include/odmkv.h."""
    _fields_ = [
        ("store", C.POINTER(Packed)), ("work", C.POINTER(Worklist)), ("pi_k_ops", C.c_void_p), ("pi_v", C.c_void_p),
        ("codebooks", C.c_void_p), ("codebooks_host", C.POINTER(C.c_float)), ("inv_scales", C.POINTER(C.c_float)),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t), ("B", C.c_int32), ("Hq", C.c_int32),
        ("q_dtype", C.c_int32), ("out_dtype", C.c_int32), ("scaling", C.c_float),
    ]


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build the HIP kernels first (python odm-kv_amd/build.py). "
            "There is no PyTorch fallback for the ODM-KV kernels.")
    lib = C.CDLL(LIB_PATH)
    i32, i64, vp, f32, sz = C.c_int, C.c_int64, C.c_void_p, C.c_float, C.c_size_t
    sig = {
        "odmkv_version": (C.c_int, []),
        "odmkv_last_error": (C.c_char_p, []),
        "odmkv_score_workspace_bytes": (sz, [i32, i32, i32]),
        "odmkv_score": (C.c_int, [vp, vp, i32, i32, i32, i64, i64, vp, i32, vp, i32, f32, vp, vp, sz, vp]),
        "odmkv_score_model_dtype": (C.c_int, [vp, vp, i32, i32, i32, i64, i64, vp, i32, vp, i32, f32, i32, vp, vp, sz, vp]),
        "odmkv_score_expected": (C.c_int, [vp, vp, i32, i32, i32, i64, i64, vp, vp, i32, i32, f32, i32, vp, vp, sz, vp]),
        "odmkv_window_attention_workspace_bytes": (sz, [i32, i32, i32, i32]),
        "odmkv_window_attention": (C.c_int, [vp, i32, i32, i32, i64, i64, vp, i32, i32, i32, i32, f32, vp, vp, sz, vp]),
        "odmkv_allocate_workspace_bytes": (sz, [i32, i32]),
        "odmkv_allocate": (C.c_int, [vp, i32, i32, vp, i32, i32, i32, C.POINTER(C.c_int32), i32,
                                     C.POINTER(C.c_double), vp, vp, vp, vp, vp, sz, vp]),
        "odmkv_level_counts": (C.c_int, [vp, i32, i32, i32, vp, vp]),
        "odmkv_store_init": (C.c_int, [vp, vp, i32, i32, vp, C.c_uint64, C.c_uint64, C.c_uint64, vp]),
        "odmkv_store_gather": (C.c_int, [C.POINTER(Packed), C.POINTER(Packed), vp]),
        "odmkv_quant_pack_staged": (C.c_int, [vp, vp, i32, i32, i32, i32, i64, i64, i64, vp, i32, vp, vp, vp,
                                              C.POINTER(Packed), vp, vp, vp, C.c_uint64, C.c_uint64, vp, vp, vp, vp, sz, vp]),
        "odmkv_store_layout": (C.c_int, [vp, i32, vp, vp, vp]),
        "odmkv_store_bind": (C.c_int, [vp, vp, vp, i32, i32, i32, i32, C.POINTER(Packed)]),
        "odmkv_pack_workspace_bytes": (sz, [i32, i32, i32]),
        "odmkv_quant_pack": (C.c_int, [vp, vp, i32, i32, i32, i32, i64, i64, i64, vp, i32, vp, vp, vp,
                                       C.POINTER(Packed), vp, sz, vp]),
        "odmkv_quantize_rows": (C.c_int, [vp, i32, i64, i64, i32, vp, vp, vp, vp, vp]),
        "odmkv_dequantize_rows": (C.c_int, [vp, vp, i64, i32, vp, vp, vp, vp]),
        "odmkv_lloyd_max": (C.c_int, [i32, i32, i32, C.c_double, C.c_double, vp, vp, vp]),
        "odmkv_rotation_operands": (C.c_int, [vp, vp, vp]),
        "odmkv_pack_count_chunks": (C.c_int, [i32]),
        "odmkv_store_finish_staged": (C.c_int, [vp, i32, i32, i32, i32, i32, i32, i32, vp, C.c_uint64, C.POINTER(Packed), vp, vp,
                                                vp, vp, vp, C.POINTER(Packed), vp, vp]),
        "odmkv_dequant": (C.c_int, [C.POINTER(Packed), vp, vp, i32, i32, i64, i64, i64, vp, vp, vp, i32, vp]),
        "odmkv_dequant_from": (C.c_int, [C.POINTER(Packed), vp, vp, i32, i32, i32, i64, i64, i64, vp, vp, vp, i32, vp]),
        "odmkv_append_exact": (C.c_int, [C.POINTER(Packed), vp, vp, i64, i64, i32, vp]),
        "odmkv_decode_workspace_bytes": (sz, [i32, i32, i32]),
        "odmkv_decode_attn": (C.c_int, [vp, i32, i32, i32, f32, C.POINTER(Packed), C.POINTER(Worklist), vp, vp, vp,
                                        C.POINTER(C.c_float), C.POINTER(C.c_float), vp, i32, vp, vp, sz, vp]),
        "odmkv_decode_attn_static": (C.c_int, [vp, i32, i32, i32, f32, C.POINTER(Packed), C.POINTER(Worklist), vp, vp, vp,
                                               C.POINTER(C.c_float), C.POINTER(C.c_float), vp, i32, vp, vp]),
        "odmkv_decode_step": (C.c_int, [C.POINTER(Step), vp, vp, vp, i64, i64, i32, vp, vp, vp]),
        "odmkv_exact_tail": (C.c_int, [C.POINTER(Packed), i32, vp, vp, vp]),
        "odmkv_flush_score": (C.c_int, [vp, vp, i32, i32, i32, vp, f32, f32, i32, vp, vp, vp, vp]),
        "odmkv_flush_rank": (C.c_int, [vp, vp, i32, i32, i32, vp, vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()
EXPORTS = ("odmkv_version", "odmkv_last_error", "odmkv_score_workspace_bytes", "odmkv_score", "odmkv_score_model_dtype", "odmkv_score_expected",
           "odmkv_window_attention_workspace_bytes", "odmkv_window_attention",
           "odmkv_allocate_workspace_bytes", "odmkv_allocate", "odmkv_level_counts",
           "odmkv_store_init", "odmkv_store_gather", "odmkv_quant_pack_staged", "odmkv_store_layout", "odmkv_store_bind", "odmkv_pack_workspace_bytes", "odmkv_pack_count_chunks", "odmkv_store_finish_staged", "odmkv_quant_pack", "odmkv_quantize_rows",
           "odmkv_dequantize_rows", "odmkv_lloyd_max", "odmkv_dequant", "odmkv_dequant_from", "odmkv_append_exact",
           "odmkv_decode_workspace_bytes", "odmkv_rotation_operands", "odmkv_decode_attn", "odmkv_decode_attn_static",
           "odmkv_decode_step", "odmkv_exact_tail", "odmkv_flush_score", "odmkv_flush_rank")


def check(rc: int) -> None:
    """0 -> ok; EINVAL / ENOSPACE -> ValueError (as the reference raises on bad shapes and levels);
    anything else -> RuntimeError."""
    if rc == 0:
        return
    msg = lib.odmkv_last_error().decode("utf-8", "replace")
    if rc in (-1, -2):
        raise ValueError(f"odmkv: {msg}")
    raise RuntimeError(f"odmkv: {msg} (code {rc})")


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}; expected float16, bfloat16 or float32") from None


def require_gpu(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{what} must live on the GPU: the ODM-KV kernels have no CPU path")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device) -> int:
    """The current stream of `device` as a raw handle (called twice per layer and decode step: the raw
    query is several times cheaper than building a torch.cuda.Stream object)."""
    if _raw_stream is not None:
        idx = getattr(device, "index", None)
        if idx is None:
            idx = torch.device(device).index
        if idx is None:
            idx = torch.cuda.current_device()
        return _raw_stream(idx)
    return torch.cuda.current_stream(device).cuda_stream


def ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


_ws_cache: dict[tuple, torch.Tensor] = {}


def workspace(device, nbytes: int, tag: str = "") -> torch.Tensor:
    """A reusable scratch buffer per (device, stream, tag); grown, never shrunk."""
    key = (str(device), stream_ptr(device), tag)
    buf = _ws_cache.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        _ws_cache[key] = buf
    return buf
