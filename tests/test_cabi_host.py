"""CPU-only checks of the C ABI: the library loads, exports every declared symbol, and rejects
bad arguments with an error code and a message before touching a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "odm-kv_amd", "lib", "libodmkv.so")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail("libodmkv.so is not built: run python odm-kv_amd/build.py")
    return C.CDLL(LIB)


def test_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "odmkv.h")).read()
    declared = set(re.findall(r"\b(odmkv_[a-z_]+)\s*\(", header))
    assert len(declared) >= 15
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in odmkv.h but not exported"
    from kvquant import _lib
    assert set(_lib.EXPORTS) == declared
    # the measurement entry points live in a library of their own and are not part of the product ABI
    bench_header = open(os.path.join(ROOT, "include", "odmkv_bench.h")).read()
    bench_declared = set(re.findall(r"\b(odmkv_bench_[a-z_]+)\s*\(", bench_header))
    assert len(bench_declared) >= 5
    blib = C.CDLL(os.path.join(ROOT, "odm-kv_amd", "lib", "libodmkv_bench.so"))
    for name in bench_declared:
        assert hasattr(blib, name) and not hasattr(lib, name)
    for name in declared:
        assert hasattr(blib, name)
    # and nothing else is a dynamic symbol of the product library: no C++ helper, no kernel stub, no measurement door
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", LIB], capture_output=True, text=True, check=True).stdout
    exported = {ln.split()[-1] for ln in out.splitlines() if len(ln.split()) == 3 and ln.split()[1] in "TDBRW"}
    assert exported == declared, sorted(exported ^ declared)


def test_version_and_error_slot(lib):
    assert lib.odmkv_version() == 1
    lib.odmkv_last_error.restype = C.c_char_p
    lib.odmkv_score.restype = C.c_int
    rc = lib.odmkv_score(None, None, 0, 8, 100, C.c_int64(0), C.c_int64(0), None, 32, None, 4,
                         C.c_float(0.01), None, None, C.c_size_t(0), None)
    assert rc == -1 and b"null" in lib.odmkv_last_error()


def test_argument_checks_without_a_gpu(lib):
    lib.odmkv_last_error.restype = C.c_char_p
    buf = C.create_string_buffer(4096)
    p = C.cast(buf, C.c_void_p)
    # head counts that do not divide
    rc = lib.odmkv_score(p, p, 0, 3, 100, C.c_int64(128 * 100), C.c_int64(128), p, 8, None, 4,
                         C.c_float(0.01), p, p, C.c_size_t(1 << 30), None)
    assert rc == -1 and b"head counts" in lib.odmkv_last_error()
    # T <= n_sink
    rc = lib.odmkv_score(p, p, 0, 2, 4, C.c_int64(512), C.c_int64(128), p, 4, None, 4,
                         C.c_float(0.01), p, p, C.c_size_t(1 << 30), None)
    assert rc == -1 and b"n_sink" in lib.odmkv_last_error()
    # workspace too small
    lib.odmkv_score_workspace_bytes.restype = C.c_size_t
    assert lib.odmkv_score_workspace_bytes(8, 32, 4096) > 0
    # descending levels
    levels = (C.c_int32 * 3)(4, 2, 8)
    eps = (C.c_double * 3)(0.1, 0.2, 0.3)
    rc = lib.odmkv_allocate(p, 1, 64, None, 64, 4, 16, levels, 3, eps, p, p, None, None, p, C.c_size_t(1 << 30), None)
    assert rc == -1 and b"ascending" in lib.odmkv_last_error()
    # unsupported width
    rc = lib.odmkv_quantize_rows(p, 0, C.c_int64(4), C.c_int64(128), 5, p, p, p, p, None)
    assert rc == -1 and b"width" in lib.odmkv_last_error()
    rc = lib.odmkv_decode_attn(None, 2, 1, 8, C.c_float(1.0), None, None, None, None, None, None, None,
                               None, 2, None, None, C.c_size_t(0), None)
    assert rc == -1
    rc = lib.odmkv_decode_attn(p, 7, 1, 8, C.c_float(1.0), None, None, None, None, None, None, None,
                               p, 2, None, None, C.c_size_t(0), None)
    assert rc == -1 and b"query dtype" in lib.odmkv_last_error()
    rc = lib.odmkv_decode_attn_static(p, 0, 1, 8, C.c_float(1.0), None, None, None, None, None, None, None, p, 2, None, None)
    assert rc == -1 and b"work list" in lib.odmkv_last_error()
    # a work list that asks for two workgroups per compute unit with sixteen wavefronts each, or without a dispatch
    # order, or for more workgroups than items, is refused before anything is launched
    from kvquant._lib import Packed, Worklist
    store, cbh, inv = Packed(), (C.c_float * 284)(), (C.c_float * 4)()
    def decode(work):
        return lib.odmkv_decode_attn(p, 0, 1, 8, C.c_float(1.0), C.byref(store), C.byref(work), p, p, p, cbh, inv,
                                     p, 2, None, p, C.c_size_t(1 << 20), None)
    w = Worklist(); w.items, w.item_range, w.dispatch_order, w.n_items = 4096, 4096, 4096, 3
    w.wavefronts, w.two_per_cu = 16, 1
    assert decode(w) == -1 and b"two workgroups per compute unit" in lib.odmkv_last_error()
    w.wavefronts, w.dispatch_order = 8, None
    assert decode(w) == -1 and b"two workgroups per compute unit" in lib.odmkv_last_error()
    w.two_per_cu, w.n_workgroups = 0, 5
    assert decode(w) == -1 and b"workgroups for" in lib.odmkv_last_error()


def test_host_modules_import_and_validate():
    import torch
    from kvquant import RiskScorer, effective_bits, ratio_scores_to_bits, scores_to_bits
    from kvquant.tq_backend import _pack_indices, _unpack_indices, random_rotation
    assert effective_bits(2, 8, 128, 4) == 2 + 8 * 2 / 128
    codes = torch.randint(0, 8, (3, 128))
    assert torch.equal(_unpack_indices(_pack_indices(codes, 3), 3, 128), codes)
    pi = random_rotation(128, "cpu", torch.float32, seed=42)
    assert torch.allclose(pi @ pi.T, torch.eye(128), atol=1e-5)
    s = torch.rand(2, 40)
    assert set(scores_to_bits(s, (2, 4, 8)).unique().tolist()) <= {2, 4, 8}
    assert ratio_scores_to_bits(s, (2, 4), (0.5, 0.5)).shape == s.shape
    sc = RiskScorer(n_future_positions=512, n_sink=4, epsilon=1e-2)
    # CPU tensors have no kernel path: asking for it is an error, not a silent fallback
    with pytest.raises(RuntimeError):
        sc.score_with_attn(torch.zeros(1, 8, 128), torch.zeros(1, 8, 128), torch.ones(1, 8) / 8)


def test_host_ratio_and_container_match_reference(golden):
    import torch
    from kvquant.allocator import ratio_scores_to_bits, scores_to_bits
    from kvquant.tq_backend import _pack_indices
    sr = torch.from_numpy(golden["ratio_scores"])
    assert (ratio_scores_to_bits(sr, (2, 3, 4, 8, 16), (0.5, 0.2, 0.15, 0.1, 0.05)).numpy() == golden["ratio_bits"]).all()
    assert (scores_to_bits(sr, (2, 3, 4, 8, 16)).numpy() == golden["uniform_bits"]).all()
    for b in (1, 2, 3, 4, 8):
        codes = torch.from_numpy(golden[f"pack_b{b}_codes"])
        assert (_pack_indices(codes, b).numpy() == golden[f"pack_b{b}_bytes"]).all()


def test_product_rotation_is_the_reference_matrix(golden):
    """The product's own random_rotation (not the oracle's copy) against the matrix the reference
    drew for seed 42 on the CPU generator (kvquant/tq_backend.py:25-36)."""
    import torch
    from kvquant.tq_backend import cached_rotation, random_rotation
    pi = random_rotation(128, "cpu", torch.float32, seed=42)
    assert pi.dtype == torch.float32 and (pi.numpy() == golden["pi_seed42"]).all()
    assert (cached_rotation(128, "cpu", 42).numpy() == golden["pi_seed42"]).all()
    # another seed is another matrix; the value rotation of a state is seed + 2000
    assert not (random_rotation(128, "cpu", torch.float32, seed=2042).numpy() == golden["pi_seed42"]).all()


def test_store_layout_and_bind_are_host_arithmetic(lib):
    """odmkv_store_layout / odmkv_store_bind touch no GPU: 33 buffers in the documented order, each on a multiple
    of 256 bytes and as large as its level's tiles need, the marks between the groups, and a descriptor whose
    pointers are the allocation's base plus those offsets."""
    import numpy as np
    from kvquant._lib import Packed
    nseg, B, H = 6, 2, 3
    rng = np.random.default_rng(5)
    cap = rng.integers(0, 9, size=(5, nseg))
    cap[1] = 0                                             # a level nobody uses keeps one tile of room
    seg_tile = np.zeros((5, nseg + 1), np.int32)
    seg_tile[:, 1:] = np.cumsum(cap, axis=1)
    off, size, marks = (C.c_uint64 * 33)(), (C.c_uint64 * 33)(), (C.c_uint64 * 5)()
    lib.odmkv_store_layout.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    assert lib.odmkv_store_layout(seg_tile.ctypes.data, nseg, off, size, marks) == 0
    off, size, marks = list(off), list(size), list(marks)
    nt = [max(int(t), 1) for t in seg_tile[:, -1]]
    widths = (2, 3, 4, 8)
    want = ([(nseg + 1) * 4] * 5 + [nseg * 4] * 5 + [nt[li] * 64 * 4 for li in range(4) for _ in (0, 1)]
            + [nt[4] * 64 * 128 * 2] * 2 + [nt[li] * 64 * 4 for li in range(5)]
            + [nt[li] * 64 * 16 * widths[li] for li in range(4) for _ in (0, 1)])
    assert size == want
    assert off[0] == 0 and all(o % 256 == 0 for o in off)
    assert all(off[i + 1] == off[i] + -(-size[i] // 256) * 256 for i in range(32))
    assert marks == [off[5], off[10], off[20], off[25], off[32] + -(-size[32] // 256) * 256]
    p = Packed()
    base = 0x7000_0000_0000
    lib.odmkv_store_bind.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(Packed)]
    assert lib.odmkv_store_bind(base, (C.c_uint64 * 33)(*off), seg_tile.ctypes.data, nseg, B, H, 0, C.byref(p)) == 0
    assert (p.B, p.Hkv, p.exact_dtype) == (B, H, 0) and list(p.n_tiles) == [int(t) for t in seg_tile[:, -1]]
    for li in range(5):
        assert p.seg_tile[li] == base + off[li] and p.seg_count[li] == base + off[5 + li] and p.pos[li] == base + off[20 + li]
    for li in range(4):
        assert (p.knorm[li], p.vnorm[li]) == (base + off[10 + 2 * li], base + off[11 + 2 * li])
        assert (p.kcodes[li], p.vcodes[li]) == (base + off[25 + 2 * li], base + off[26 + 2 * li])
    assert (p.kexact, p.vexact) == (base + off[18], base + off[19])
    lib.odmkv_last_error.restype = C.c_char_p
    assert lib.odmkv_store_bind(base, (C.c_uint64 * 33)(*off), seg_tile.ctypes.data, nseg, B, H + 1, 0, C.byref(p)) == -1
    assert b"store_bind" in lib.odmkv_last_error()


def test_store_finish_staged_sizes_the_store_without_a_gpu(lib):
    """With no allocation to lay the store out in, odmkv_store_finish_staged launches nothing: it adds up the chunk
    counts, sizes the segments (a tile per 64 tokens, the exact segments with room to grow), reports the bytes the
    layout needs and returns ODMKV_ENOSPACE; counts that do not add up to every token are refused."""
    import numpy as np
    from kvquant._lib import Packed
    B, H, T, n_chunks, slack = 1, 3, 5000, 3, 256
    nseg = B * H
    rng = np.random.default_rng(9)
    per_seg = np.zeros((nseg, 6), np.int64)
    for s in range(nseg):
        cut = np.sort(rng.integers(0, T + 1, size=5))
        per_seg[s] = np.diff(np.concatenate([[0], cut, [T]]))
    per_seg[1, 2] += per_seg[1, 3]; per_seg[1, 3] = 0                 # a level nobody uses in one segment
    chunks = np.zeros((nseg, n_chunks, 6), np.int32)
    for s in range(nseg):
        for k in range(6):
            parts = rng.multinomial(per_seg[s, k], [1 / n_chunks] * n_chunks)
            chunks[s, :, k] = parts
    counts = np.zeros((nseg, 6), np.int32)
    seg_tile = np.zeros((5, nseg + 1), np.int32)
    off, size, marks = (C.c_uint64 * 33)(), (C.c_uint64 * 33)(), (C.c_uint64 * 5)()
    staging, store, need = Packed(), Packed(), C.c_uint64(0)
    f = lib.odmkv_store_finish_staged
    f.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_uint64, C.POINTER(Packed),
                  C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Packed), C.c_void_p, C.c_void_p]
    rc = f(chunks.ctypes.data, n_chunks, B, H, T, slack, 0, 0, None, 0, C.byref(staging), counts.ctypes.data,
           seg_tile.ctypes.data, off, size, marks, C.byref(store), C.byref(need), None)
    assert rc == -2 and b"needs" in lib.odmkv_last_error()
    assert np.array_equal(counts, per_seg)
    want = (per_seg[:, 1:].T + 63) // 64
    want[4] = (per_seg[:, 5] + slack + 63) // 64
    assert np.array_equal(np.diff(seg_tile, axis=1), want) and np.all(seg_tile[:, 0] == 0)
    assert need.value == marks[4] > 0
    plain = need.value
    # with head-room for later flushes: a sixteenth more tiles, two at least, in every quantised segment
    rc = f(chunks.ctypes.data, n_chunks, B, H, T, slack, 1, 0, None, 0, C.byref(staging), counts.ctypes.data,
           seg_tile.ctypes.data, off, size, marks, C.byref(store), C.byref(need), None)
    assert rc == -2
    roomy = want.copy()
    roomy[:4] += np.maximum(roomy[:4] // 16, 2)
    assert np.array_equal(np.diff(seg_tile, axis=1), roomy) and need.value > plain
    chunks[2, 1, 4] += 1                                               # one token too many
    rc = f(chunks.ctypes.data, n_chunks, B, H, T, slack, 0, 0, None, 0, C.byref(staging), counts.ctypes.data,
           seg_tile.ctypes.data, off, size, marks, C.byref(store), C.byref(need), None)
    assert rc == -1 and b"must take values" in lib.odmkv_last_error()
