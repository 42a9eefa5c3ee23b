"""Benchmark of the ODM-KV hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers 32] [--ctx 32768]

Workload (the second benchmark configuration, kernel-only form): 32 independent Llama-3-8B-shaped layers
(Hq 32, Hkv 8, d 128), 32k-token context each, K/V ~ N(0,1) with 8x sink tokens, compressed at a
2.0 average-bit budget (score -> allocate -> window override -> quantise + pack), then decoded one
token at a time over the packed caches.  One "step" = one decode token = the fused LUT attention
over all layers' packed caches, launched layer after layer on one stream.  The packed caches of
32 layers (~0.6 GB) do not fit the 256 MB last-level cache, so every step streams them from HBM.

Prints ONE JSON line:
  value          whole-job GB/s = packed bytes of all layers / mean step time (query preparation + main
                 kernels and launch gaps included; inputs resident in HBM; the step is replayed as
                 one HIP graph unless --no-graph)
  roofline       the main kernel alone (streaming + the merge at its end): packed bytes per launch / its
                 mean duration from HIP events on its own stream, against 8 TB/s
  cpu_baseline   the oracle's restatement of the reference's CPU decode step (SDPA over the
                 re-materialised cache) on this box's host cores, in the same unit
and, as extra fields, the per-layer score+allocate+pack time (the second half of the metric).
"""
from __future__ import annotations

import argparse
import ctypes as C
import gc
import json
import os
import statistics
import sys
import time

# The CPU generator of the synthetic layers runs on all cores right before every timed compression.  Worker threads
# that spin after a parallel region would share the cores with the one thread that launches the kernels; let them
# sleep instead (the thread count is left as it is).  Must be set before the OpenMP runtimes are loaded.
os.environ.setdefault("OMP_WAIT_POLICY", "passive")
os.environ.setdefault("KMP_BLOCKTIME", "0")
os.environ.setdefault("GOMP_SPINCOUNT", "0")

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "odm-kv_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0
TRAFFIC_LAYERS = 6      # layers of the counter runs: the bytes per launch do not depend on how many layers take turns
LEVELS = (0, 2, 3, 4, 8, 16)


def make_layer(li, n_kv, n_q, T, dev):
    """One layer of the workload, drawn from the CPU generator (the same numbers on every machine):
    K, V ~ N(0,1) fp16 with 8x sinks, expected query mu, decode query q."""
    import synthetic
    if (n_kv, n_q) == (8, 32):
        L = synthetic.config("c2", layer=li, T=T)
    elif (n_kv, n_q) == (4, 28):
        L = synthetic.config("c5", layer=li, T=T)
    else:
        L = synthetic.gaussian_layer(2002 + li, n_kv, n_q, T)
    # the decode query in the model's dtype, as a model hands it over (the generator keeps fp16 values in an fp32 tensor)
    return L.keys.to(dev), L.values.to(dev), L.mu.to(dev), L.query[None].to(L.keys.dtype).to(dev)


def load_bench_lib():
    """libodmkv_bench.so: the product library's object files plus the measurement entry points of
    include/odmkv_bench.h (stage selection per call, kernel timing, a plain read)."""
    from kvquant import _lib
    path = os.path.join(ROOT, "odm-kv_amd", "lib", "libodmkv_bench.so")
    lib = C.CDLL(path)
    i32, vp, f32, sz = C.c_int, C.c_void_p, C.c_float, C.c_size_t
    lib.odmkv_last_error.restype = C.c_char_p
    lib.odmkv_bench_timer_create.argtypes = [i32, C.POINTER(vp)]
    lib.odmkv_bench_timer_collect.argtypes = [vp, C.POINTER(C.c_float), i32, C.POINTER(C.c_int)]
    lib.odmkv_bench_timer_destroy.argtypes = [vp]
    lib.odmkv_bench_decode_attn.argtypes = [vp, i32, i32, i32, f32, C.POINTER(_lib.Packed), C.POINTER(_lib.Worklist), vp, vp, vp,
                                            C.POINTER(C.c_float), C.POINTER(C.c_float), vp, i32, vp, vp, sz, vp, i32, vp]
    lib.odmkv_bench_probe_read.argtypes = [vp, sz, i32, vp, vp]
    lib.odmkv_decode_workspace_bytes.restype = sz
    lib.odmkv_decode_workspace_bytes.argtypes = [i32, i32, i32]
    return lib


def bench_decode(blib, st, q, out, ws, stage_mask=7, timer=None):
    """The call of TurboQuantAdaptiveKVCacheState.decode_attention through the measurement library."""
    from kvquant import _lib
    if st._items is None:
        st._build_items()
    B, Hq, _ = q.shape
    rc = blib.odmkv_bench_decode_attn(
        q.data_ptr(), _lib.dtype_code(q), B, Hq, 128 ** -0.5, C.byref(st._packed), C.byref(st._worklist),
        st._pi_k_ops.data_ptr(), st.pi_v.data_ptr(), st._decode_cb.data_ptr(),
        st._decode_cb_host, st._decode_inv, out.data_ptr(), _lib.dtype_code(out), None, ws.data_ptr(), ws.numel(),
        _lib.stream_ptr(q.device), stage_mask, timer)
    if rc != 0:
        raise RuntimeError(blib.odmkv_last_error().decode())


def plain_read_us(blib, dev, pool, nbytes, grid, nbuf, stride, reps=5):
    """Microseconds per launch of a plain streaming read of `nbytes` (odmkv_bench_probe_read), the launches of one sweep
    over `nbuf` buffers of `pool` back to back in one graph between two events: what a launch of that size can reach."""
    import torch
    from kvquant import _lib
    sink = torch.zeros(64, dtype=torch.int32, device=dev)

    def sweep():
        for it in range(nbuf):
            rc = blib.odmkv_bench_probe_read(pool.data_ptr() + it * stride, nbytes, grid, sink.data_ptr(), _lib.stream_ptr(dev))
            assert rc == 0, blib.odmkv_last_error()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sweep()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        sweep()
    g.replay()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (reps * nbuf) * 1e3


def parity_gate(dev):
    """A small instance of the whole path against the CPU oracle, before anything is timed."""
    import numpy as np
    import torch
    import synthetic
    from kvquant.allocator import calibrate_epsilon, optimal_scores_to_bits
    from kvquant.scorer import _launch_score
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    from oracle import allocator as oal, scorer as osc
    from oracle.attention import decode_attention_state
    from oracle.kvstate import KVState
    L = synthetic.gaussian_layer(77, 8, 32, 2048)
    sink = torch.zeros(8, 2048, dtype=torch.bool)
    sink[:, :4] = True
    s = _launch_score(L.keys.to(dev), L.values.to(dev), L.mu.to(dev), None, 32, 4, 1e-2)
    want = osc.risk_score_from_mu(L.keys.float(), L.values.float(), L.mu.unsqueeze(0), 32)
    np.testing.assert_allclose(s.cpu().numpy(), want.numpy(), rtol=1e-3)
    eps = calibrate_epsilon(128, LEVELS, device=dev, value_quantizer="mse")
    bits = optimal_scores_to_bits(s, LEVELS, 2.0, eps, sink.to(dev), eviction_cost=0.5)
    assert torch.equal(bits.cpu(), oal.optimal_scores_to_bits(s.cpu(), LEVELS, 2.0, eps, sink, eviction_cost=0.5))
    bits = bits.clone()
    bits[:, -128:] = 16
    st = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=dev, dtype=torch.float16, key_quantizer="mse",
                                        value_quantizer="mse", seed=42)
    st.prefill(L.keys[None].to(dev), L.values[None].to(dev), bits[None])
    ref = KVState(128, LEVELS, seed=42, order="canonical")
    ref.prefill(L.keys[None], L.values[None], bits[None].cpu())
    got = st.decode_attention(L.query[None].to(dev)).cpu().double()
    exp = decode_attention_state(L.query[None], ref)
    err = ((got - exp).norm(dim=-1) / exp.norm(dim=-1)).max().item()
    assert err < 1e-3, err
    return eps, err


def measure_traffic(args):
    """HBM bytes per launch of the main decode kernel, from the L2 counters, measured by this invocation: two child runs
    of this file's --traffic-probe (the same workload, TRAFFIC_LAYERS layers) under ``rocprofv3 --pmc``, one counter
    each (FETCH_SIZE, WRITE_SIZE; KiB per dispatch), each scaled by what the same counter reads for the probe's plain
    256 MiB device copy.  Runs BEFORE this process touches the GPU (a child must not be started from a process that
    holds the device), one child at a time, each under a hard time limit.  Returns (dict, None) or (None, reason)."""
    import csv
    import shutil
    import subprocess
    import tempfile
    if shutil.which("rocprofv3") is None:
        return None, "rocprofv3 not on PATH"
    if any(k.startswith("ROCPROF") for k in os.environ) or "rocprof" in os.environ.get("LD_PRELOAD", ""):
        return None, "this run is itself under a profiler"
    tmp = tempfile.mkdtemp(prefix="odmkv_pmc_", dir="/tmp")
    env = dict(os.environ, TMPDIR="/tmp")
    res = {}
    try:
        for ctr in ("FETCH_SIZE", "WRITE_SIZE"):
            cmd = ["timeout", "-s", "KILL", "240", "rocprofv3", "--pmc", ctr, "--output-format", "csv", "-d", tmp, "-o", ctr, "--",
                   sys.executable, os.path.abspath(__file__), "--traffic-probe", "--layers", str(TRAFFIC_LAYERS), "--ctx", str(args.ctx),
                   "--target", str(args.target), "--kv-heads", str(args.kv_heads), "--q-heads", str(args.q_heads)]
            print(f"[traffic] {ctr}: counter run of {TRAFFIC_LAYERS} layers", file=sys.stderr, flush=True)
            r = subprocess.run(cmd, cwd=tmp, env=env, stdin=subprocess.DEVNULL, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
            if r.returncode != 0:
                return None, f"counter run for {ctr} ended with status {r.returncode}: {r.stderr[-300:]!r}"
            probe = [json.loads(ln) for ln in r.stdout.splitlines() if ln.startswith("{") and "traffic_probe" in ln]
            found = [os.path.join(d, f) for d, _, fs in os.walk(tmp) for f in fs if f == f"{ctr}_counter_collection.csv"]
            if not probe or not found:
                return None, f"counter run for {ctr} left no output"
            main, copy = [], []
            with open(found[0], newline="") as fh:
                for row in csv.DictReader(fh):
                    if row["Counter_Name"] != ctr:
                        continue
                    if "decode_main_kernel" in row["Kernel_Name"]:
                        main.append(float(row["Counter_Value"]))
                    elif "copyBuffer" in row["Kernel_Name"]:
                        copy.append(float(row["Counter_Value"]))
            if len(main) < 3 or not copy or max(copy) <= 0:
                return None, f"{ctr}: {len(main)} main-kernel dispatches and {len(copy)} copies in the counter file"
            copy_kib = probe[-1]["copy_bytes"] / 1024.0
            factor = copy_kib / max(copy)                 # the largest copy is the probe's 256 MiB one
            res[ctr] = {"kib_per_dispatch_median": round(statistics.median(main), 1), "copy_reads_kib": round(max(copy), 1),
                        "factor": round(factor, 4), "dispatches": len(main)}
            res["packed_bytes_per_layer"] = probe[-1]["packed_bytes_per_layer"]
    except Exception as exc:                                               # noqa: BLE001
        return None, f"{type(exc).__name__}: {exc}"
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    res["bytes"] = int(1024 * sum(res[c]["kib_per_dispatch_median"] * res[c]["factor"] for c in ("FETCH_SIZE", "WRITE_SIZE")))
    return res, None


def press_e2e(dev, T, target, n_new, n_layers=2, vocab=32000):
    """The press end to end on a model of Llama-3-8B's shape (n_layers layers, random weights):
    prefill T tokens under the press, then n_new greedy decode steps: over the packed cache with the
    fused kernel, the same with the model's dense cache copy released, and over the dense
    re-materialised cache with the model's own attention function (what the reference executes).
    Wall time per decode step, device-synchronised; device memory the caches hold after the prefill."""
    import torch
    from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM
    from kvquant import RiskScorer, TurboQuantPerTokenBackendPress, attention_patch
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=4096, num_hidden_layers=n_layers, num_attention_heads=32, num_key_value_heads=8,
                      head_dim=128, intermediate_size=14336, vocab_size=vocab,
                      max_position_embeddings=max(T + n_new + 8, 8192), rope_theta=500000.0, attn_implementation="sdpa")
    # weights are drawn on the device in fp16: a host-side fp32 initialisation of 8 B parameters takes minutes
    default_dtype = torch.get_default_dtype()
    torch.set_default_dtype(torch.float16)
    try:
        with torch.device(dev):
            model = LlamaForCausalLM(cfg).eval()
    finally:
        torch.set_default_dtype(default_dtype)
    print(f"[press-e2e] model of {n_layers} layers built", file=sys.stderr, flush=True)
    ids = torch.randint(0, vocab, (1, T), generator=torch.Generator().manual_seed(1)).to(dev)
    out = {"model": f"{n_layers} x Llama-3-8B-shaped layer, vocabulary {vocab}, random init, fp16", "prefill_tokens": T,
           "decode_tokens": n_new, "target_avg_bits": target}
    tokens = {}
    for mode in ("fused", "fused_released", "dense"):
        os.environ["ODMKV_FUSED_DECODE"] = "0" if mode == "dense" else "1"
        torch.cuda.synchronize()
        base_bytes = torch.cuda.memory_allocated()
        scorer = RiskScorer(n_future_positions=512, n_sink=4, use_vnorm=True, epsilon=1e-2)
        scorer.normalize_grain = "global"
        press = TurboQuantPerTokenBackendPress(
            scorer=scorer, bit_levels=LEVELS, target_avg_bits=target, eviction_cost=0.5, seed=42, decode_quant=True,
            sink_tokens=4, layerwise=True, key_quantizer="mse", value_quantizer="mse", buffer_size=128,
            release_dense_cache=(mode == "fused_released"))
        before = dict(attention_patch.call_counts)
        cache = DynamicCache()
        with torch.inference_mode(), press(model):
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            t0 = time.perf_counter()
            h = model.model(input_ids=ids, past_key_values=cache).last_hidden_state[:, -1:, :]
            tok = model.lm_head(h)[0, -1].argmax().view(1, 1)
            torch.cuda.synchronize()
            t_prefill = time.perf_counter() - t0
            del h
            peak_bytes = torch.cuda.max_memory_allocated() - base_bytes   # activations + caches at the prefill's peak
            cache_bytes = torch.cuda.memory_allocated() - base_bytes      # packed stores + what the HF cache holds
            print(f"[press-e2e] {mode}: prefill of {T} tokens {t_prefill:.2f} s", file=sys.stderr, flush=True)
            steps, emitted = [], [int(tok)]
            for step in range(n_new):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                logits = model(input_ids=tok, past_key_values=cache,
                               position_ids=torch.tensor([[T + step]], device=dev)).logits
                tok = logits[0, -1].argmax().view(1, 1)
                torch.cuda.synchronize()
                steps.append(time.perf_counter() - t0)
                emitted.append(int(tok))
        tokens[mode] = emitted
        print(f"[press-e2e] {mode}: {n_new} decode steps done", file=sys.stderr, flush=True)
        took = {k: attention_patch.call_counts[k] - before[k] for k in before}
        out[mode] = {"prefill_s": round(t_prefill, 3), "decode_step_ms_median": round(statistics.median(steps[4:]) * 1e3, 3),
                     "decode_step_ms_min": round(min(steps[4:]) * 1e3, 3),
                     "decode_step_ms_mean_with_flushes": round(statistics.fmean(steps[4:]) * 1e3, 3),
                     "attention_calls": took, "cache_bytes_after_prefill": int(cache_bytes),
                     "prefill_peak_bytes_over_model": int(peak_bytes)}
        del cache, press
        for layer in model.model.layers:                     # the modules keep their last store attached
            layer.self_attn._odmkv_state = None
            layer.self_attn.masked_key_indices = None
        torch.cuda.empty_cache()
    os.environ.pop("ODMKV_FUSED_DECODE", None)
    cache = DynamicCache()
    with torch.inference_mode():                             # the same prefill with no press attached
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        h = model.model(input_ids=ids, past_key_values=cache).last_hidden_state[:, -1:, :]
        model.lm_head(h)
        torch.cuda.synchronize()
        out["prefill_s_without_press"] = round(time.perf_counter() - t0, 3)
    del cache
    # what the model itself costs per decode step: no press, a 16-token context (attention is negligible)
    cache = DynamicCache()
    with torch.inference_mode():
        tok = model(input_ids=ids[:, :16], past_key_values=cache).logits[0, -1].argmax().view(1, 1)
        steps = []
        for step in range(24):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            tok = model(input_ids=tok, past_key_values=cache,
                        position_ids=torch.tensor([[16 + step]], device=dev)).logits[0, -1].argmax().view(1, 1)
            torch.cuda.synchronize()
            steps.append(time.perf_counter() - t0)
        out["decode_step_ms_model_alone_short_context"] = round(statistics.median(steps[4:]) * 1e3, 3)
    del cache
    same = 0
    for x, y in zip(tokens["fused"], tokens["dense"]):      # greedy tokens agree until the first near-tie
        if x != y:
            break
        same += 1
    out["greedy_tokens_equal_prefix"] = same
    out["dense_over_fused"] = round(out["dense"]["decode_step_ms_median"] / out["fused"]["decode_step_ms_median"], 2)
    out["dense_over_fused_released"] = round(
        out["dense"]["decode_step_ms_median"] / out["fused_released"]["decode_step_ms_median"], 2)
    return out


def cpu_baseline(sample_T, n_kv, n_q, eps, threads):
    """The reference's CPU path, restated by the oracle, on a bounded sample (one layer of
    `sample_T` tokens): compress it, then time what a decode step costs the reference - SDPA over
    the re-materialised dense cache.  Reported as packed bytes per second, the GPU metric's unit."""
    import torch
    import synthetic
    from oracle import allocator as oal, scorer as osc
    from oracle.kvstate import KVState
    torch.set_num_threads(threads)
    L = synthetic.gaussian_layer(2002, n_kv, n_q, sample_T)
    sink = torch.zeros(n_kv, sample_T, dtype=torch.bool)
    sink[:, :4] = True
    t0 = time.perf_counter()
    s = osc.risk_score_from_mu(L.keys.float(), L.values.float(), L.mu.unsqueeze(0), n_q)   # fp32 tensors
    t_score = time.perf_counter() - t0
    t0 = time.perf_counter()
    bits = oal.optimal_scores_to_bits(s.float(), LEVELS, 2.0, eps, sink, eviction_cost=0.5)
    t_alloc = time.perf_counter() - t0
    bits = bits.clone()
    bits[:, -128:] = 16
    ref = KVState(128, LEVELS, seed=42, order="blas")
    t0 = time.perf_counter()
    ref.prefill(L.keys[None], L.values[None], bits[None])
    t_pack = time.perf_counter() - t0
    t0 = time.perf_counter()
    kd, vd = ref.materialize()
    t_mat = time.perf_counter() - t0
    G = n_q // n_kv
    q = L.query[None, :, None, :].float()
    kf = kd.float().repeat_interleave(G, dim=1)
    vf = vd.float().repeat_interleave(G, dim=1)
    mask = ref.visible_mask().repeat_interleave(G, dim=1)[:, :, None, :]
    reps, times = 5, []
    for _ in range(reps + 1):
        t0 = time.perf_counter()
        torch.nn.functional.scaled_dot_product_attention(q, kf, vf, attn_mask=mask)
        times.append(time.perf_counter() - t0)
    t_sdpa = statistics.median(times[1:])
    return {
        "packed_bytes": ref.packed_bytes(), "t_sdpa": t_sdpa, "t_materialize": t_mat,
        "t_score": t_score, "t_alloc": t_alloc, "t_pack": t_pack,
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-graph", action="store_true", help="launch every step from Python instead of replaying a HIP graph")
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--ctx", type=int, default=32768)
    ap.add_argument("--target", type=float, default=2.0)
    ap.add_argument("--kv-heads", type=int, default=8, help="KV heads (default 8: Llama-3-8B; --kv-heads 4 --q-heads 28 --layers 28 "
                                                            "--target 3.0 is configuration c5, Qwen2.5-7B)")
    ap.add_argument("--q-heads", type=int, default=32)
    ap.add_argument("--cpu-sample-ctx", type=int, default=8192)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--read-ceiling", action="store_true",
                    help="time a plain streaming read kernel at the decode kernel's launch sizes (cold buffers) and exit")
    ap.add_argument("--decode-shape", choices=["c3", "c4", "w2", "w3", "w4", "w8", "exact", "b64", "b16"],
                    help="time the fused decode call on six stores of configuration c3's (16 sequences x 8192 tokens, "
                         "cycling budgets) or c4's (131072 tokens, heavy eviction) shape, compressed by the real pipeline, "
                         "or on single-level stores (w2..w8: every token of a 131072-token layer at that width; exact: 32768 "
                         "fp16 tokens), or on batches whose every (sequence, kv-head) holds four quantised levels by fixed shares "
                         "(b64: 64 sequences x 2048 tokens, b16: 16 x 8192), rotating over the stores so that every call reads "
                         "HBM; prints main-kernel and whole-call times and exits")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="for counter runs under rocprofv3 --pmc: a few eager decode steps and one plain 256 MiB "
                         "device copy (the calibration kernel), nothing else timed")
    ap.add_argument("--score-expected", action="store_true",
                    help="time the expected-attention score (mean query + query covariance on the fp32 matrix "
                         "cores) of one --ctx-token layer, rotating over 8 layers' keys and values, and exit")
    ap.add_argument("--score-window", action="store_true",
                    help="time the observation-window attention mass (last 64 queries of every head, per-query causal "
                         "softmax, 16-bit matrix cores) and the risk score built on it for one --ctx-token layer, and exit")
    ap.add_argument("--press-e2e", action="store_true",
                    help="instead of the kernel benchmark: a random-init Llama-3-8B-shaped model (--e2e-layers) under the "
                         "press, prefill of --ctx tokens, then greedy decode with the fused kernel and with the dense "
                         "re-materialised cache (the reference's path); prints per-token times")
    ap.add_argument("--traffic", choices=["live", "none"], default="live",
                    help="live: before the benchmark, two short counter runs of --traffic-probe under rocprofv3 --pmc give "
                         "roofline.traffic (about 25 s each); none: roofline.traffic is null")
    ap.add_argument("--no-e2e", action="store_true",
                    help="leave out the e2e record (a 2-layer Llama-3-8B-shaped model under the press: ms per decode step "
                         "with the fused kernel, with the reference's dense path and of the model alone; about 20 s)")
    ap.add_argument("--e2e-tokens", type=int, default=48)
    ap.add_argument("--e2e-layers", type=int, default=2, help="layers of the --press-e2e model (32 = Llama-3-8B)")
    ap.add_argument("--e2e-vocab", type=int, default=32000, help="vocabulary of the --press-e2e model (Llama-3: 128256)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the path: every box in this build has one GPU and "
              "nothing here shards across devices; run with --gpus 1", file=sys.stderr)
        return 2

    headline = not (args.press_e2e or args.score_expected or args.score_window or args.read_ceiling or args.decode_shape
                    or args.traffic_probe)
    traffic, traffic_note = None, "not measured (--traffic none)"
    if headline and args.traffic == "live":
        traffic, traffic_note = measure_traffic(args)       # child processes: before this one touches the GPU
        if traffic is None:
            print(f"[traffic] not measured: {traffic_note}", file=sys.stderr, flush=True)

    import torch
    from kvquant import _lib
    from kvquant.allocator import optimal_scores_to_bits_batched
    from kvquant.scorer import _launch_score
    from kvquant.tq_adaptive_backend import TurboQuantAdaptiveKVCacheState
    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the ODM-KV kernels have no CPU path", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n_kv, n_q, T, NL = args.kv_heads, args.q_heads, args.ctx, args.layers

    if args.press_e2e:
        print(json.dumps({"press_e2e": press_e2e(dev, T, args.target, args.e2e_tokens, args.e2e_layers,
                                                   args.e2e_vocab)}))
        return 0

    if args.score_expected:
        from kvquant.scorer import _launch_score_expected
        g = torch.Generator().manual_seed(5)
        layers = []
        for _ in range(8):
            k = torch.randn(n_kv, T, 128, generator=g).half().to(dev)
            v = torch.randn(n_kv, T, 128, generator=g).half().to(dev)
            mu = torch.randn(n_q, 128, generator=g).to(dev)
            a = torch.randn(n_q, 128, 32, generator=g) * 0.2
            layers.append((k, v, mu, (a @ a.transpose(-1, -2)).to(dev)))
        out = {}
        for name, with_cov in (("with_covariance", True), ("mean_query_only", False)):
            def sweep():
                for k, v, mu, cov in layers:
                    _launch_score_expected(k, v, mu, cov if with_cov else None, n_q, 4, 1e-2, True)
            for _ in range(3):
                sweep()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(5):
                sweep()
            e1.record()
            torch.cuda.synchronize()
            out[name + "_ms_per_layer"] = round(e0.elapsed_time(e1) / (5 * len(layers)), 4)
        flop = 2.0 * n_q * (T - 4) * 128 * 128
        out["quadratic_form_flop_per_layer"] = flop
        out["quadratic_form_TFLOPs_lower_bound"] = round(flop / ((out["with_covariance_ms_per_layer"]
                                                                   - out["mean_query_only_ms_per_layer"]) * 1e-3) / 1e12, 1)
        out["shape"] = {"Hkv": n_kv, "Hq": n_q, "T": T, "dtype": "fp16"}
        print(json.dumps({"score_expected": out}))
        return 0

    if args.score_window:
        from kvquant.scorer import _launch_window_attention
        g = torch.Generator().manual_seed(6)
        W = 64
        layers = []
        for _ in range(8):
            k = torch.randn(n_kv, T, 128, generator=g).half().to(dev)
            v = torch.randn(n_kv, T, 128, generator=g).half().to(dev)
            q = torch.randn(n_q, W, 128, generator=g).half().to(dev)
            layers.append((k, v, q))
        out = {}
        for name in ("window_attention", "window_risk_score"):
            def sweep():
                for k, v, q in layers:
                    p = _launch_window_attention(k, q, 4, T - W, 128 ** -0.5)
                    if name == "window_risk_score":
                        _launch_score(k[:, 4:], v[:, 4:], None, p, n_kv, 0, 1e-2)
            for _ in range(3):
                sweep()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(5):
                sweep()
            e1.record()
            torch.cuda.synchronize()
            out[name + "_ms_per_layer"] = round(e0.elapsed_time(e1) / (5 * len(layers)), 4)
        out["flop_per_pass"] = 2.0 * n_q * W * (T - 4) * 128
        out["shape"] = {"Hkv": n_kv, "Hq": n_q, "T": T, "window": W, "dtype": "fp16"}
        print(json.dumps({"score_window": out}))
        return 0

    blib = load_bench_lib()
    if args.read_ceiling:
        # what can ONE launch of a given size reach?  buffers rotate through 2 GiB so every launch reads HBM
        pool = torch.ones(2 << 30, dtype=torch.uint8, device=dev)
        rows = []
        for nbytes in (19336677, 80740000, 536870912):
            stride = (nbytes + (2 << 20)) & ~((2 << 20) - 1)
            nbuf = min((2 << 30) // stride, 64)
            for grid in (1024, 2048, 4096):
                # the launches of one sweep over the buffers go back to back (one graph), timed between two
                # events: event pairs around single launches would add about 2 us to each
                avg = plain_read_us(blib, dev, pool, nbytes, grid, nbuf, stride) * 1e-3
                rows.append({"bytes": nbytes, "grid": grid, "buffers": nbuf, "avg_us": round(avg * 1e3, 2),
                             "GBps": round(nbytes / (avg * 1e-3) / 1e9), "pct_of_8TBps": round(100 * nbytes / (avg * 1e-3) / 8e12, 1)})
        print(json.dumps({"read_ceiling": rows}))
        return 0

    eps, gate_err = parity_gate(dev)

    if args.decode_shape:
        import synthetic
        name, n_stores = args.decode_shape, 6
        sts, sqs = [], []
        for li in range(n_stores):
            single = {"w2": 2, "w3": 3, "w4": 4, "w8": 8, "exact": 16}.get(name)
            if name == "c3":
                Ls = [synthetic.gaussian_layer(3003 + 100 * li + s, 8, 32, 8192) for s in range(16)]
                targets = [synthetic.C3_TARGETS[s % 3] for s in range(16)]
            elif name == "c4":
                Ls = [synthetic.lognormal_norm_layer(4004 + li, 8, 32, 131072)]
                targets = [2.0]
            elif name in ("b64", "b16"):
                # batches whose (sequence, kv-head) pairs each hold four quantised levels (fixed shares, drawn per token):
                # 64 sequences x 2048 tokens, 16 x 8192
                nb, nt = (64, 2048) if name == "b64" else (16, 8192)
                g = torch.Generator(device=dev).manual_seed(7007 + li)
                Ls = None
                Bs, Ts = nb, nt
                k = torch.randn(nb, 8, nt, 128, generator=g, device=dev, dtype=torch.float16)
                v = torch.randn(nb, 8, nt, 128, generator=g, device=dev, dtype=torch.float16)
                shares = torch.tensor([0.12, 0.50, 0.18, 0.13, 0.06, 0.01], device=dev)
                idx = torch.multinomial(shares, nb * 8 * nt, replacement=True, generator=g)
                bits = torch.tensor(LEVELS, device=dev, dtype=torch.int32)[idx].reshape(nb, 8, nt)
                bits[..., :4] = 16
                bits[..., -128:] = 16
                st = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=dev, dtype=torch.float16, key_quantizer="mse",
                                                    value_quantizer="mse", seed=42 + li)
                st.prefill(k, v, bits)
                st._build_items()
                sts.append(st)
                sqs.append((torch.randn(nb, 32, 128, generator=g, device=dev, dtype=torch.float16) * 1.5))
                del k, v, bits
                continue
            else:
                Ls = [synthetic.gaussian_layer(6006 + li, 8, 32, 32768 if single == 16 else 131072)]
            Bs, Ts = len(Ls), Ls[0].keys.shape[1]
            k = torch.stack([L.keys for L in Ls]).to(dev)
            v = torch.stack([L.values for L in Ls]).to(dev)
            if single is None:
                sc = torch.stack([_launch_score(k[b], v[b], Ls[b].mu.to(dev), None, 32, 4, 1e-2) for b in range(Bs)])
                bits = optimal_scores_to_bits_batched(sc.reshape(Bs, -1), LEVELS, targets, eps, n_sink=4, period=Ts,
                                                      eviction_cost=0.5).reshape(Bs, 8, Ts)
                bits[..., -128:] = 16
            else:
                sc = None
                bits = torch.full((Bs, 8, Ts), single, dtype=torch.int32, device=dev)
            st = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=dev, dtype=torch.float16, key_quantizer="mse",
                                                value_quantizer="mse", seed=42 + li)
            st.prefill(k, v, bits)
            st._build_items()
            sts.append(st)
            sqs.append(torch.stack([L.query for L in Ls]).half().to(dev))        # the model's dtype
            del k, v, sc, bits
        Bs = sqs[0].shape[0]
        ws_bytes = max(blib.odmkv_decode_workspace_bytes(Bs, 32, st._items[2]) for st in sts)
        wss = [torch.empty(ws_bytes, dtype=torch.uint8, device=dev) for _ in sts]
        outs = [torch.empty(Bs, 32, 128, dtype=torch.float32, device=dev) for _ in sts]

        def sweep(mask):
            for st, q, o, w in zip(sts, sqs, outs, wss):
                bench_decode(blib, st, q, o, w, mask)

        def graph_us(mask, reps=20):
            sweep(7)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                sweep(mask)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            gk = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gk):
                sweep(mask)
            for _ in range(3):
                gk.replay()
            rounds = []
            for _ in range(5):                      # five rounds of `reps` replays: the median, and the extremes beside it
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                e0.record()
                for _ in range(reps):
                    gk.replay()
                e1.record()
                torch.cuda.synchronize()
                rounds.append(e0.elapsed_time(e1) / (reps * n_stores) * 1e3)
            rounds.sort()
            return rounds[2], rounds[0], rounds[-1]

        pb = sum(st.packed_bytes() for st in sts) / n_stores
        (main_us, main_lo, main_hi), (call_us, call_lo, call_hi) = graph_us(2), graph_us(6)
        print(json.dumps({"decode_shape": name, "stores": n_stores, "sequences": Bs, "tokens": int(sts[0].seq_len),
                          "packed_bytes_per_store": int(pb), "work_items": int(sts[0]._items[2]),
                          "level_counts": {str(b): int(sum(st.level_counts()[b] for st in sts) / n_stores) for b in LEVELS},
                          "main_kernel_us": round(main_us, 2), "main_kernel_us_min_max": [round(main_lo, 2), round(main_hi, 2)],
                          "main_kernel_GBps": round(pb / main_us / 1e3, 1),
                          "main_kernel_frac_of_8TBps": round(pb / main_us / 1e3 / 8000.0, 4),
                          "whole_call_us": round(call_us, 2), "whole_call_us_min_max": [round(call_lo, 2), round(call_hi, 2)],
                          "whole_call_GBps": round(pb / call_us / 1e3, 1)}))
        return 0

    # ---- compress every layer: score -> allocate -> window -> pack (timed per layer) ----
    states, qs, t_stage = [], [], {"score": [], "alloc": [], "pack": [], "total": []}
    dense0 = None

    def compress(k, v, mu, seed, ev=None):
        st = TurboQuantAdaptiveKVCacheState(128, LEVELS, device=dev, dtype=torch.float16, key_quantizer="mse",
                                            value_quantizer="mse", seed=seed)
        if ev:
            ev[0].record()
        s = _launch_score(k, v, mu, None, n_q, 4, 1e-2)
        if ev:
            ev[1].record()
        bits = optimal_scores_to_bits_batched(s.reshape(1, -1), LEVELS, [args.target], eps, n_sink=4, period=T,
                                              eviction_cost=0.5).reshape(n_kv, T)
        bits[:, -128:] = 16
        if ev:
            ev[2].record()
        st.prefill(k[None], v[None], bits[None])
        if ev:
            ev[3].record()
        return st, bits

    # what a press does when it is attached to a model: the allocator's small-block pool takes the stores' tables now,
    # not by a device allocation every few layers in the middle of a compression
    from kvquant.tq_adaptive_backend import reserve_state_memory
    reserve_state_memory(dev, 2 * NL)
    warm = None
    for li in range(NL):
        k, v, mu, q = make_layer(li, n_kv, n_q, T, dev)        # about a second of CPU work: the GPU idles meanwhile
        # an untimed pass over OTHER data first (the previous layer's; for the first layer its own, which also warms
        # the allocators): the device is busy and at its clocks again when the timed pass starts, and the timed
        # pass still reads keys and values that no kernel has touched
        compress(*(warm if warm is not None else (k, v, mu)), seed=41)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        torch.cuda.synchronize()
        gc.disable()                     # as timeit does: the interpreter's cyclic collector (0.1-0.3 ms a run) stays out
        st, bits = compress(k, v, mu, 42 + 7 * li, ev)
        torch.cuda.synchronize()
        gc.enable()
        warm = (k, v, mu)
        # device events on the launch stream, no host synchronisation between the stages (the pack
        # stage's own read-back of the level counts is inside its interval)
        t_stage["score"].append(ev[0].elapsed_time(ev[1]) * 1e-3)
        t_stage["alloc"].append(ev[1].elapsed_time(ev[2]) * 1e-3)
        t_stage["pack"].append(ev[2].elapsed_time(ev[3]) * 1e-3)
        t_stage["total"].append(ev[0].elapsed_time(ev[3]) * 1e-3)
        states.append(st)
        qs.append(q)
        if li == 0:
            dense0 = (k, v, bits)
    packed_bytes = sum(s.packed_bytes() for s in states)
    counts = {b: sum(s.level_counts()[b] for s in states) for b in LEVELS}
    print("[stages] ms per layer (score, alloc, pack): " + " ".join(
        f"{a * 1e3:.3f}/{b * 1e3:.3f}/{c * 1e3:.3f}" for a, b, c in zip(t_stage["score"], t_stage["alloc"], t_stage["pack"])),
        file=sys.stderr, flush=True)

    # ---- full-size self-consistency: fused attention == dense attention over the dequantised cache ----
    # (dequantised without rounding to the model dtype and summed in fp64: next to logits of 20 to 100, as the
    # sink tokens of these workloads produce, rounding the dense cache to fp16 alone moves softmax weights by 1e-3)
    kd, vd = states[0].materialize(dtype=torch.float32)
    vis = states[0].visible_mask()
    G = n_q // n_kv
    full_err = 0.0
    for h in range(n_kv):                                   # one KV head at a time: fp64 copies stay small
        qh = qs[0][:, h * G:(h + 1) * G].double()
        logits = torch.einsum("bgd,btd->bgt", qh, kd[:, h].double()) / 128 ** 0.5
        logits = logits.masked_fill(~vis[:, h, None, :], float("-inf"))
        dense_out = torch.einsum("bgt,btd->bgd", torch.softmax(logits, -1), vd[:, h].double())
        if h == 0:
            fused = states[0].decode_attention(qs[0]).double()
        e = (fused[:, h * G:(h + 1) * G] - dense_out).norm(dim=-1) / dense_out.norm(dim=-1)
        full_err = max(full_err, e.max().item())
    assert full_err < 1e-3, f"fused vs dense attention at full size: {full_err}"
    del kd, vd, logits, dense_out, dense0

    # ---- decode steps ----
    def step():
        for st, q in zip(states, qs):
            st.decode_attention(q)

    # the measurement calls go through libodmkv_bench.so with the stores' own buffers; outputs and workspaces
    # are allocated once, outside every timed region
    for st in states:
        if st._items is None:
            st._build_items()
    ws_bytes = max(blib.odmkv_decode_workspace_bytes(1, n_q, st._items[2]) for st in states)
    b_ws = [torch.empty(ws_bytes, dtype=torch.uint8, device=dev) for _ in states]
    b_out = [torch.empty(1, n_q, 128, dtype=torch.float32, device=dev) for _ in states]

    def bench_step(stage_mask=7, timer=None):
        for st, q, o, w in zip(states, qs, b_out, b_ws):
            bench_decode(blib, st, q, o, w, stage_mask, timer)

    def collect_kernel_ms(n_launches, fn):
        """Durations of the main kernel from HIP events attached to its dispatches (launch stream)."""
        timer = C.c_void_p()
        assert blib.odmkv_bench_timer_create(n_launches + 8, C.byref(timer)) == 0, blib.odmkv_last_error()
        fn(timer)
        torch.cuda.synchronize()
        buf = (C.c_float * (n_launches + 8))()
        n = C.c_int(0)
        assert blib.odmkv_bench_timer_collect(timer, buf, len(buf), C.byref(n)) == 0, blib.odmkv_last_error()
        blib.odmkv_bench_timer_destroy(timer)
        return sorted(buf[i] for i in range(n.value))

    if args.traffic_probe:
        for _ in range(3):
            step()
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"traffic_probe": True, "packed_bytes_per_layer": int(packed_bytes / NL), "copy_bytes": 256 << 20}))
        return 0

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # the timed region replays one captured step (64 kernels) so that the host's per-call work does
    # not sit between the kernels; falls back to launching from Python if capture is not possible
    graph, launch_mode = None, "python"
    if not args.no_graph:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                step()
            g.replay()
            torch.cuda.synchronize()
            graph, launch_mode = g, "hip graph"
        except Exception as exc:                                   # noqa: BLE001
            print(f"graph capture not available ({exc}); timing eager launches", file=sys.stderr)
            torch.cuda.synchronize()
    run = graph.replay if graph is not None else step
    for _ in range(3):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    # kernel durations: an eager pass over the same rotating 32 buffers, then one buffer alone (cache-resident)
    prof_steps = min(args.steps, 20)
    kernel_ms = collect_kernel_ms(prof_steps * NL, lambda t: [bench_step(7, t) for _ in range(prof_steps)])
    hot_ms = collect_kernel_ms(200, lambda t: [bench_decode(blib, states[0], qs[0], b_out[0], b_ws[0], 7, t) for _ in range(200)])

    def graph_ms_per_launch(stage_mask, reps):
        """The step's 32 decode calls with the given stages, captured as one graph and replayed between two
        HIP events on the launch stream; elapsed / launches.  Per-launch event pairs (above) add about 2 us
        to every launch; this does not."""
        bench_step(7)                                    # a full call fills the workspaces the partial stages reuse
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            bench_step(stage_mask)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        gk = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gk):
            bench_step(stage_mask)
        for _ in range(3):
            gk.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            gk.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (reps * NL)

    kern_alone_ms = with_merge_ms = None
    if graph is not None:
        try:
            kern_alone_ms = graph_ms_per_launch(2, min(args.steps, 50))      # the main kernel alone, back to back
            with_merge_ms = graph_ms_per_launch(6, min(args.steps, 50))      # with its merge: the whole call
        except Exception as exc:                                   # noqa: BLE001
            print(f"main-kernel-only graph not available ({exc}); using per-launch events", file=sys.stderr)
            torch.cuda.synchronize()

    def pct(v, p):
        return v[min(len(v) - 1, int(p / 100.0 * len(v)))]

    ms_per_step = elapsed / args.steps * 1e3
    value = packed_bytes / (elapsed / args.steps) / 1e9
    bytes_per_launch = packed_bytes / NL
    events_avg_ms = sum(kernel_ms) / max(len(kernel_ms), 1)
    kern_avg_ms = kern_alone_ms if kern_alone_ms is not None else events_avg_ms
    achieved = bytes_per_launch / (kern_avg_ms * 1e-3) / 1e9
    # what a launch of this size can reach: a plain streaming read of the same number of bytes per launch, timed the same
    # way (one graph of launches over NL buffers, so that every launch reads memory), outside the timed region
    plain = None
    try:
        nb = int(bytes_per_launch)
        stride = (nb + (2 << 20)) & ~((2 << 20) - 1)
        pool = torch.ones(stride * NL, dtype=torch.uint8, device=dev)
        us = plain_read_us(blib, dev, pool, nb, 4096, NL, stride)
        plain = {"bytes_per_launch": nb, "us_per_launch": round(us, 2), "GBps": round(nb / us / 1e3, 1),
                 "frac_of_peak": round(nb / us / 1e3 / HBM_PEAK_GBS, 4), "kernel_over_plain_read": round(us / (kern_avg_ms * 1e3), 3)}
        del pool
    except Exception as exc:                                       # noqa: BLE001
        print(f"plain-read figure not available ({exc})", file=sys.stderr)

    out = {
        "metric": "LUT decode-attn achieved GB/s (% HBM peak); ms to score+pack a 32k-token layer",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 products, f32 accumulate (2/3/4/8-bit codes)", "data": "synthetic",
        "config": {"workload": f"{'c2' if (n_kv, n_q, NL) == (8, 32, 32) else 'custom'} kernel-only: {NL} layers x [Hkv {n_kv}, T {T}, d 128] fp16, Hq {n_q}, {args.target} avg bits, "
                               "1 decode token per step over all layers' packed caches",
                   "levels": list(LEVELS), "n_sink": 4, "window": 128, "launch": launch_mode},
        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "packed_bytes_per_layer": int(bytes_per_launch),
        "level_counts": counts,
        "score_alloc_pack_ms_per_layer": round(statistics.median(t_stage["total"]) * 1e3, 3),
        "stage_ms": {k: round(statistics.median(v) * 1e3, 3) for k, v in t_stage.items()},
        "stage_ms_min_max": {k: [round(min(v) * 1e3, 3), round(max(v) * 1e3, 3)] for k, v in t_stage.items()},
        "parity": {"gate_attn_rel_err": gate_err, "full_size_fused_vs_dense_rel_err": full_err},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": None if traffic is None else traffic["bytes"],
                     "traffic_source": (traffic_note if traffic is None else
                                        {"how": f"this invocation: rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, over bench.py --traffic-probe "
                                                f"--layers {TRAFFIC_LAYERS} (child runs before the timed part), KiB per dispatch (median) x the "
                                                "factor the same counter gives for a plain 256 MiB copy",
                                         "FETCH_SIZE": traffic["FETCH_SIZE"], "WRITE_SIZE": traffic["WRITE_SIZE"],
                                         "over_algorithmic": round(traffic["bytes"] / traffic["packed_bytes_per_layer"], 4)}),
                     "plain_read_of_the_same_size": plain,
                     "kernel": "decode_main_kernel", "kernel_avg_us": round(kern_avg_ms * 1e3, 2),
                     "kernel_avg_method": ("the step's main-kernel launches alone (no merge) as one graph, replayed between two "
                                           "HIP events on the launch stream: elapsed / launches, launch gaps included"
                                           if kern_alone_ms is not None else "per-launch HIP event pairs"),
                     "with_merge_kernel_us": None if with_merge_ms is None else round(with_merge_ms * 1e3, 2),
                     "per_launch_events_avg_us": round(events_avg_ms * 1e3, 2),
                     "per_launch_events_median_us": round(pct(kernel_ms, 50) * 1e3, 2),
                     "per_launch_events_p10_us": round(pct(kernel_ms, 10) * 1e3, 2),
                     "per_launch_events_p90_us": round(pct(kernel_ms, 90) * 1e3, 2), "launches": len(kernel_ms),
                     "single_buffer_cache_resident_median_us": round(pct(hot_ms, 50) * 1e3, 2)},
    }
    if not args.no_cpu:
        # the GPU box hands one job a 16-thread share of its host, whatever os.cpu_count() shows
        threads = min(os.cpu_count() or 1, 16)
        cb = cpu_baseline(args.cpu_sample_ctx, n_kv, n_q, eps, threads)
        out["cpu_baseline"] = {
            "value": round(cb["packed_bytes"] / cb["t_sdpa"] / 1e9, 3), "unit": "GB/s", "cores": threads,
            "host_cpu_count": os.cpu_count(), "kind": "port",
            "sample": f"one layer, T={args.cpu_sample_ctx}: oracle compress, then median of 5 torch-CPU fp32 SDPA calls over "
                      "the re-materialised dense cache (what a reference decode step costs), packed bytes / time",
            "sdpa_ms": round(cb["t_sdpa"] * 1e3, 2), "materialize_ms": round(cb["t_materialize"] * 1e3, 1),
            "score_ms": round(cb["t_score"] * 1e3, 1), "alloc_ms": round(cb["t_alloc"] * 1e3, 1),
            "pack_ms": round(cb["t_pack"] * 1e3, 1), "cpu_model": _cpu_model(),
        }
    if not args.no_e2e and (n_kv, n_q) == (8, 32):
        # outside every timed region above: what the kernels buy a whole decode step (host side of the press included)
        torch.cuda.empty_cache()
        try:
            e = press_e2e(dev, T, args.target, 24, n_layers=2, vocab=32000)
            out["e2e"] = {
                "model": e["model"], "prefill_tokens": T, "decode_tokens": 24, "note": "wall ms per decode step, device-synchronised, median",
                "fused_ms_per_step": e["fused"]["decode_step_ms_median"],
                "fused_dense_cache_released_ms_per_step": e["fused_released"]["decode_step_ms_median"],
                "dense_reference_path_ms_per_step": e["dense"]["decode_step_ms_median"],
                "model_alone_short_context_ms_per_step": e["decode_step_ms_model_alone_short_context"],
                "dense_over_fused": e["dense_over_fused"],
                "cache_bytes_after_prefill": {m: e[m]["cache_bytes_after_prefill"] for m in ("fused", "fused_released", "dense")},
                "attention_calls": {m: e[m]["attention_calls"] for m in ("fused", "fused_released", "dense")},
            }
        except Exception as exc:                                           # noqa: BLE001
            out["e2e"] = {"error": f"{type(exc).__name__}: {exc}"}
    print(json.dumps(out))
    return 0


def _cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


if __name__ == "__main__":
    sys.exit(main())
