"""Test helper: decode the packed KV store's buffers with numpy, from the layout as documented in
include/odmkv.h (independent of the kernels' own indexing code)."""
import numpy as np

TILE, HD = 64, 128
WIDTHS = (2, 3, 4, 8)
# slot of key block b (0..3), column n (0..15) of a tile: [n, b]
KEY_SLOT = np.array([[32 * (b >> 1) + 8 * (n >> 2) + 2 * (n & 3) + (b & 1) for b in range(4)] for n in range(16)])


def _bits_to_codes(byte_rows: np.ndarray, w: int) -> np.ndarray:
    """[..., nbytes] little-endian bit streams -> [..., nbytes*8/w] codes."""
    bits = np.unpackbits(byte_rows, axis=-1, bitorder="little")
    bits = bits.reshape(bits.shape[:-1] + (bits.shape[-1] // w, w)).astype(np.uint16)     # also for zero rows
    return (bits << np.arange(w, dtype=np.uint16)).sum(axis=-1).astype(np.uint8)


def _lane_streams(buf: np.ndarray, nt: int, w: int) -> np.ndarray:
    """Tile buffer -> [nt, 64 lanes, 128 codes]: chunk c of lane l sits at byte (c*64 + l)*16 of its tile."""
    chunks = buf[: nt * TILE * 16 * w].reshape(nt, w, TILE, 16)
    return _bits_to_codes(chunks.transpose(0, 2, 1, 3).reshape(nt, TILE, 16 * w), w)


def decode_level(state, li: int):
    """-> dict(bh, pos, kcodes [N,128], vcodes [N,128], knorm, vnorm) over the stored tokens."""
    w = WIDTHS[li]
    b = state._bufs
    nt = int(state._seg_tile[li, -1])
    # keys: lane 16j+n, code 32b+i = dim 32j+i of slot key_slot(n, b)
    ks = _lane_streams(b["kcodes"][li].cpu().numpy(), nt, w).reshape(nt, 4, 16, 4, 32)        # [t, j, n, b, i]
    kcodes = np.empty((nt, TILE, HD), np.uint8)
    kcodes[:, KEY_SLOT.reshape(-1)] = ks.transpose(0, 2, 3, 1, 4).reshape(nt, TILE, HD)       # rows (n, b) -> their slots
    # values: lane 16j+n, code 64k+8m+e = slot 32k+8j+e of dim 16m+n
    vs = _lane_streams(b["vcodes"][li].cpu().numpy(), nt, w).reshape(nt, 4, 16, 2, 8, 8)      # [t, j, n, k, m, e]
    vcodes = vs.transpose(0, 3, 1, 5, 4, 2).reshape(nt, TILE, HD)                             # [t, slot=32k+8j+e, dim=16m+n]
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
    # keys: chunk 4b+k of lane 16j+n = dims 32j+8k..+7 of slot key_slot(n, b)
    krows = np.empty((nt, TILE, HD), ke.dtype)
    krows[:, KEY_SLOT.reshape(-1)] = ke.reshape(nt, 4, 4, 4, 16, 8).transpose(0, 4, 1, 3, 2, 5).reshape(nt, TILE, HD)  # [t,b,k,j,n,e] -> [t, (n, b), (j, k, e)]
    # values: chunk 8k+m of lane 16j+n = slots 32k+8j..+7 of dim 16m+n
    vrows = ve.reshape(nt, 2, 8, 4, 16, 8).transpose(0, 1, 3, 5, 2, 4).reshape(nt, TILE, HD)  # [t,k,m,j,n,e] -> [t, k, j, e, m, n]
    pos = b["pos"][4].cpu().numpy()[: nt * TILE].reshape(nt, TILE)
    out = {k: [] for k in ("bh", "pos", "k", "v")}
    for s in range(state._nseg):
        c = int(state._counts[4, s])
        t0 = int(state._seg_tile[4, s])
        for i in range(c):
            t, l = t0 + i // TILE, i % TILE
            out["bh"].append(s); out["pos"].append(pos[t, l]); out["k"].append(krows[t, l]); out["v"].append(vrows[t, l])
    return {k: np.asarray(v) for k, v in out.items()}
