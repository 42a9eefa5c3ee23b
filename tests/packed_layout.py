"""Test helper: decode the packed KV store's buffers with numpy, from the layout as documented in
include/odmkv.h (independent of the kernels' own indexing code)."""
import numpy as np

TILE, HD = 64, 128
WIDTHS = (2, 3, 4, 8)


def _bits_to_codes(byte_rows: np.ndarray, w: int) -> np.ndarray:
    """[..., nbytes] little-endian bit streams -> [..., nbytes*8/w] codes."""
    bits = np.unpackbits(byte_rows, axis=-1, bitorder="little")
    bits = bits.reshape(bits.shape[:-1] + (bits.shape[-1] // w, w)).astype(np.uint16)     # also for zero rows
    return (bits << np.arange(w, dtype=np.uint16)).sum(axis=-1).astype(np.uint8)


def decode_level(state, li: int):
    """-> dict(bh, pos, kcodes [N,128], vcodes [N,128], knorm, vnorm) over the stored tokens."""
    w = WIDTHS[li]
    b = state._bufs
    nt = int(state._seg_tile[li, -1])
    kc = b["kcodes"][li].cpu().numpy()[: nt * TILE * 16 * w].reshape(nt, w, TILE, 16)
    k_rows = kc.transpose(0, 2, 1, 3).reshape(nt, TILE, 16 * w)               # token-major streams
    kcodes = _bits_to_codes(k_rows, w)                                        # [nt, 64, 128]
    U = 8 if w == 3 else 16
    nu = 8 * w // U
    vc = b["vcodes"][li].cpu().numpy()[: nt * HD * 8 * w].reshape(nt, nu, HD, U)
    v_rows = vc.transpose(0, 2, 1, 3).reshape(nt, HD, 8 * w)                  # dim-major streams
    vcodes = _bits_to_codes(v_rows, w).transpose(0, 2, 1)                     # [nt, 64 tokens, 128 dims]
    kn = b["knorm"][li].cpu().numpy()[: nt * TILE].reshape(nt, TILE)
    vn = b["vnorm"][li].cpu().numpy()[: nt * TILE].reshape(nt, TILE)
    pos = b["pos"][li].cpu().numpy()[: nt * TILE].reshape(nt, TILE)
    out = {k: [] for k in ("bh", "pos", "kcodes", "vcodes", "knorm", "vnorm")}
    for s in range(state._nseg):
        c = int(state._counts[li, s])
        t0 = int(state._seg_tile[li, s])
        for i in range(c):
            t, l = t0 + i // TILE, i % TILE
            out["bh"].append(s); out["pos"].append(pos[t, l])
            out["kcodes"].append(kcodes[t, l]); out["vcodes"].append(vcodes[t, l])
            out["knorm"].append(kn[t, l]); out["vnorm"].append(vn[t, l])
    return {k: np.asarray(v) for k, v in out.items()}


def decode_exact(state):
    b = state._bufs
    nt = int(state._seg_tile[4, -1])
    ke = b["kexact"].view(-1).cpu().view(dtype=__import__("torch").int16).numpy()[: nt * TILE * HD]
    ve = b["vexact"].view(-1).cpu().view(dtype=__import__("torch").int16).numpy()[: nt * TILE * HD]
    krows = ke.reshape(nt, 16, TILE, 8).transpose(0, 2, 1, 3).reshape(nt, TILE, HD)
    vrows = ve.reshape(nt, 16, HD, 4).transpose(0, 1, 3, 2).reshape(nt, TILE, HD)
    pos = b["pos"][4].cpu().numpy()[: nt * TILE].reshape(nt, TILE)
    out = {k: [] for k in ("bh", "pos", "k", "v")}
    for s in range(state._nseg):
        c = int(state._counts[4, s])
        t0 = int(state._seg_tile[4, s])
        for i in range(c):
            t, l = t0 + i // TILE, i % TILE
            out["bh"].append(s); out["pos"].append(pos[t, l]); out["k"].append(krows[t, l]); out["v"].append(vrows[t, l])
    return {k: np.asarray(v) for k, v in out.items()}
