"""GPU: the decode entry point that allocates nothing (odmkv_decode_attn_static: its scratch is a
fixed array inside the library's device image) against odmkv_decode_attn with a caller workspace,
through the C ABI, on two calls in a row, the second with a smaller input; then the size limit."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"
LEVELS = (0, 2, 3, 4, 8, 16)


def _store(seed, B, Hkv, T, probs):
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, Hkv, T, 128, generator=g).half()
    v = torch.randn(B, Hkv, T, 128, generator=g).half()
    lv = torch.tensor(LEVELS, dtype=torch.int32)
    bits = lv[torch.multinomial(torch.tensor(probs), B * Hkv * T, replacement=True, generator=g)].reshape(B, Hkv, T)
    bits[..., :4] = 16
    bits[..., -8:] = 16
    st = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=DEV, dtype=torch.float16, key_quantizer="mse",
                                        value_quantizer="mse", seed=seed)
    st.prefill(k.to(DEV), v.to(DEV), bits.to(DEV))
    st._build_items()
    return st


def _call(st, q, static):
    """One decode call through the C ABI; returns (out fp32 [B, Hq, 128], lse [B, Hq])."""
    from kvquant import _lib
    lib = _lib.lib
    B, Hq, _ = q.shape
    n_items = st._items[2]
    out = torch.full((B, Hq, 128), float("nan"), dtype=torch.float32, device=DEV)
    lse = torch.full((B, Hq), float("nan"), dtype=torch.float32, device=DEV)
    common = (q.data_ptr(), _lib.dtype_code(q), B, Hq, 128 ** -0.5, C.byref(st._packed), C.byref(st._worklist),
              st._pi_k_ops.data_ptr(), st.pi_v.data_ptr(), st._decode_cb.data_ptr(), st._decode_cb_host, st._decode_inv, out.data_ptr(), _lib.F32, lse.data_ptr())
    stream = _lib.stream_ptr(torch.device(DEV, torch.cuda.current_device()))
    if static:
        rc = lib.odmkv_decode_attn_static(*common, stream)
    else:
        nbytes = lib.odmkv_decode_workspace_bytes(B, Hq, n_items)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        rc = lib.odmkv_decode_attn(*common, ws.data_ptr(), nbytes, stream)
    _lib.check(rc)
    torch.cuda.synchronize()
    return out.cpu(), lse.cpu()


def test_static_scratch_entry_point_matches_the_workspace_one():
    from kvquant import _lib
    big = _store(71, 2, 2, 3000, (0.2, 0.4, 0.12, 0.1, 0.1, 0.08))
    small = _store(72, 1, 2, 200, (0.1, 0.5, 0.1, 0.1, 0.1, 0.1))
    g = torch.Generator().manual_seed(73)
    q_big = torch.randn(2, 14, 128, generator=g).half().to(DEV)        # G = 7
    q_small = torch.randn(1, 8, 128, generator=g).half().to(DEV)       # G = 4
    for st, q in ((big, q_big), (small, q_small)):                     # the second call is the smaller one
        got, got_lse = _call(st, q, static=True)
        want, want_lse = _call(st, q, static=False)
        assert torch.isfinite(got).all() and torch.isfinite(got_lse).all()
        # the same kernels over the same inputs: the same bits
        assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    # and once more the large one after the small one (the array keeps the last call's contents)
    got, _ = _call(big, q_big, static=True)
    want, _ = _call(big, q_big, static=False)
    assert torch.equal(got, want)
    # a call that does not fit the fixed array is refused, with a message, and launches nothing
    lib = _lib.lib
    n_items = 1 << 16
    assert lib.odmkv_decode_workspace_bytes(2, 14, n_items) > (8 << 20)
    work = _lib.Worklist()
    work.items, work.item_range, work.n_items = big._items[0].data_ptr(), big._items[1].data_ptr(), n_items
    out = torch.zeros(2, 14, 128, device=DEV)
    rc = lib.odmkv_decode_attn_static(q_big.data_ptr(), _lib.F16, 2, 14, 0.1, C.byref(big._packed), C.byref(work),
                                      big._pi_k_ops.data_ptr(), big.pi_v.data_ptr(), big._decode_cb.data_ptr(), big._decode_cb_host, big._decode_inv, out.data_ptr(),
                                      _lib.F32, None, None)
    assert rc == -2 and b"fixed array" in lib.odmkv_last_error()
    torch.cuda.synchronize()
    assert (out == 0).all()


def test_static_call_leaves_device_memory_as_it_is_and_replays_from_a_graph():
    """No allocation: the device's free memory and torch's allocated bytes are the same before and after a
    run of calls (outputs are allocated beforehand); and the call can be captured into a HIP graph, whose
    replays (with eager work and synchronisations between them) give the eager call's bits."""
    from kvquant import _lib
    lib = _lib.lib
    st = _store(81, 1, 4, 2500, (0.15, 0.45, 0.15, 0.1, 0.05, 0.1))
    g = torch.Generator().manual_seed(82)
    qs = [torch.randn(1, 16, 128, generator=g).half().to(DEV) for _ in range(4)]
    q = qs[0].clone()
    out = torch.zeros(1, 16, 128, dtype=torch.float32, device=DEV)
    lse = torch.zeros(1, 16, dtype=torch.float32, device=DEV)

    def call(stream):
        _lib.check(lib.odmkv_decode_attn_static(
            q.data_ptr(), _lib.F16, 1, 16, 128 ** -0.5, C.byref(st._packed), C.byref(st._worklist), st._pi_k_ops.data_ptr(),
            st.pi_v.data_ptr(), st._decode_cb.data_ptr(), st._decode_cb_host, st._decode_inv, out.data_ptr(), _lib.F32,
            lse.data_ptr(), stream))

    dev = torch.device(DEV, torch.cuda.current_device())
    call(_lib.stream_ptr(dev))                                  # the first call on a device looks the array up
    torch.cuda.synchronize()
    free0, allocated0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(20):
        call(_lib.stream_ptr(dev))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.cuda.memory_allocated() == allocated0 and torch.cuda.memory_reserved() == reserved0

    want = []
    for x in qs:                                                # eager results for four queries
        q.copy_(x)
        call(_lib.stream_ptr(dev))
        torch.cuda.synchronize()
        want.append((out.clone(), lse.clone()))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(_lib.stream_ptr(dev))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(_lib.stream_ptr(dev))
    for x, (w_out, w_lse) in zip(qs, want):
        q.copy_(x)
        out.zero_(); lse.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, w_out) and torch.equal(lse, w_lse)
        (out * 2).sum().item()                                  # the program's own eager work between replays
