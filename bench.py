#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

A "step" is one greedy decode token of BASELINE config 4: a random-init 9B-class Q4_K decoder
(36 layers, hidden 4096, FFN 12288, 32 query / 8 KV heads of 128, tied f16 LM head over a
151,936-token vocabulary), KV cache prefilled to 2048 positions, every op on the HIP path
through the C ABI, one 4-byte token readback per step.  Prints ONE JSON line with
  value     decode tokens/s over exactly --steps steps (weights, KV and activations resident
            in HBM; the only host traffic is the token id),
  roofline  the dominant kernel (the fused gate/up Q4_K GEMV, 56.7 MB of weights per launch)
            timed with HIP events on the op stream, against the 8 TB/s HBM peak,
  cpu_baseline  the CPU oracle's decode step timed on this host's cores on a bounded sample.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per fused gate/up launch from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs, scaled
# by the same counters' readings for a cast kernel of known traffic (x2.000 and x1.000):
# 55,683 KiB fetched + 48 KiB written.
GATE_UP_TRAFFIC_BYTES = 57088000


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gate_up_kernel_bandwidth(dec, reps):
    """Average duration of the fused gate/up GEMV launch, measured with HIP events on the
    stream the kernel runs on.  Launches cycle through the layers' weights (36 x 56.6 MB,
    far beyond the 256 MB infinity cache) so every launch streams from HBM; the launches of
    one sweep are enqueued back to back between two events, so the figure is the kernel's
    duration plus the dispatch gap between consecutive kernels."""
    from doppler_amd import capi
    L, c = dec.L, dec.cfg
    Hd, I = c["hidden"], c["inter"]
    ev = [ctypes.c_void_p() for _ in range(2)]
    for e in ev:
        capi.check(L.dh_event_create(ctypes.byref(e)))

    def sweep():
        for d in dec.layers:
            # the launch the decode step makes: RMSNorm prologue + gate/up + SiLU gating
            capi.check(L.dh_q4k_ffn_gate_up_rmsnorm(dec.x2.data_ptr(), d["post_attn_norm"].data_ptr(), c["eps"], 0,
                                                    d["wgate"].data_ptr(), d["wup"].data_ptr(), dec.act.data_ptr(),
                                                    1, Hd, I, capi.ACT_SILU, 1.0, 0.0))
    sweep()                                # warms code and TLBs
    capi.check(L.dh_sync())
    total_ms, n = 0.0, 0
    for r in range(reps):
        capi.check(L.dh_event_record(ev[0]))
        sweep()
        capi.check(L.dh_event_record(ev[1]))
        ms = ctypes.c_float()
        capi.check(L.dh_event_elapsed_ms(ev[0], ev[1], ctypes.byref(ms)))
        total_ms += ms.value
        n += len(dec.layers)
    for e in ev:
        capi.check(L.dh_event_destroy(e))
    return total_ms / max(n, 1)


def layer_chain_bandwidth(dec, reps):
    """Average duration of the chained launch of a layer (o + residual, RMSNorm + gate/up + SiLU, down +
    residual, next layer's RMSNorm + q/k/v: dh_q4k_gemv_chain), measured like the gate/up launch above,
    cycling through the layers' weights; (ms per launch, algorithmic bytes per launch)."""
    from doppler_amd import capi, synth
    L, c = dec.L, dec.cfg
    Hd, I = c["hidden"], c["inter"]
    chains = [dec._chain_phases(li) for li in range(len(dec.layers) - 1)]      # the last layer's has three products
    if not chains:
        return None
    qkv_n = dec.qs + 2 * dec.ks
    nbytes = (synth.q4k_nbytes(Hd, dec.qs) + 2 * synth.q4k_nbytes(I, Hd) + synth.q4k_nbytes(Hd, I) + synth.q4k_nbytes(qkv_n, Hd)
              + 4 * (dec.qs + 2 * Hd + Hd + Hd + I + I + Hd + Hd + Hd + Hd + qkv_n))   # inputs, residuals, norm weights, outputs
    ev = [ctypes.c_void_p() for _ in range(2)]
    for e in ev:
        capi.check(L.dh_event_create(ctypes.byref(e)))

    def sweep():
        for arr, n in chains:
            capi.check(L.dh_q4k_gemv_chain(dec.attn.data_ptr(), arr, n))
    sweep()
    capi.check(L.dh_sync())
    total_ms, n = 0.0, 0
    for r in range(reps):
        capi.check(L.dh_event_record(ev[0]))
        sweep()
        capi.check(L.dh_event_record(ev[1]))
        ms = ctypes.c_float()
        capi.check(L.dh_event_elapsed_ms(ev[0], ev[1], ctypes.byref(ms)))
        total_ms += ms.value
        n += len(chains)
    for e in ev:
        capi.check(L.dh_event_destroy(e))
    return total_ms / max(n, 1), nbytes


def js_reference_timings():
    """Runs oracle/js/reference_port.mjs (one thread, as the reference's JS is) and returns its
    timings in milliseconds, or None when node is missing."""
    import shutil
    import subprocess
    node = shutil.which("node")
    if not node:
        return None
    try:
        r = subprocess.run([node, os.path.join(ROOT, "oracle", "js", "reference_port.mjs"), "time"],
                           capture_output=True, text=True, timeout=300, check=True)
        return json.loads(r.stdout.strip().splitlines()[-1])
    except Exception as e:      # a baseline, never a reason to lose the GPU result
        log("[bench] JS port timing failed: %r" % (e,))
        return None


def js_host_decode(cfg, layers, embed, final_norm, prefill, warmup, steps):
    """Decode tokens/s of the JavaScript host on the same model: node subprocess over
    doppler_amd/js/bench/decode_bench.mjs (loader -> prefill -> decodeStep loop with a blocking readback per
    step, the same positions through decodeGreedy's staged readback, then the captured-graph loop).  Returns its JSON, or None when node or the addon is missing."""
    import shutil
    import subprocess
    import tempfile
    from doppler_amd import rdrr
    node = shutil.which("node")
    addon = os.path.join(ROOT, "doppler_amd", "js", "doppler_hip.node")
    if not node or not os.path.exists(addon):
        log("[bench] JS host skipped (node or the addon missing)")
        return None
    base = "/dev/shm" if os.path.isdir("/dev/shm") and os.access("/dev/shm", os.W_OK) else None
    d = tempfile.mkdtemp(prefix="doppler_amd_bench_", dir=base)
    try:
        t0 = time.time()
        rdrr.write_artifact(d, cfg, layers, embed, final_norm, shard_bytes=256 << 20)
        log("[bench] artifact for the JS host written in %.1f s" % (time.time() - t0))
        r = subprocess.run([node, os.path.join(ROOT, "doppler_amd", "js", "bench", "decode_bench.mjs"), d, str(prefill),
                            str(warmup), str(steps), "graph"], capture_output=True, text=True, timeout=600)
        if r.returncode != 0:
            log("[bench] JS host failed: %s" % r.stderr[-2000:])
            return None
        res = json.loads(r.stdout.strip().splitlines()[-1])
        for k in ("tokens_per_s", "ms_per_step", "graph_tokens_per_s", "graph_ms_per_step", "greedy_tokens_per_s",
                  "greedy_ms_per_step"):
            if k in res:
                res[k] = round(res[k], 3)
        return res
    except Exception as e:      # a side measurement, never a reason to lose the GPU result
        log("[bench] JS host failed: %r" % (e,))
        return None
    finally:
        shutil.rmtree(d, ignore_errors=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="debug only: fewer layers (result is not the metric)")
    ap.add_argument("--prefill", type=int, default=None, help="debug only: shorter prefill")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-js-host", action="store_true", help="skip the JavaScript-host side measurement")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three f32->f16 casts of 16 Mi elements (64 MiB read, 32 MiB written): a "
                         "streaming kernel of known traffic to scale rocprofv3 FETCH_SIZE / WRITE_SIZE with")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (single-stream decode has nothing to shard in this tier); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from doppler_amd import decoder, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(1)

    c = dict(synth.CFG4)
    prefill, _ = c.pop("prefill"), c.pop("steps")
    if args.layers:
        c["layers"] = args.layers
    if args.prefill is not None:
        prefill = args.prefill
    BATCH = 16                       # extra positions for the batched-decode side measurement
    max_seq = prefill + args.warmup + args.steps + 2 * BATCH + 40
    cfg = dict(c, max_seq=max_seq)

    t0 = time.time()
    layers, embed, final_norm, cos, sin = decoder.random_model(cfg, seed=4, max_seq=max_seq)
    log("[bench] synthetic weights generated in %.1f s" % (time.time() - t0))
    t0 = time.time()
    dec = decoder.HipDecoder(cfg, layers, embed, final_norm, cos, sin, max_seq)
    log("[bench] uploaded in %.1f s" % (time.time() - t0))

    # ---- KV prefill (outside the timed region): the prompt goes through the batched path, Q4_K
    #      prefill GEMMs and matrix-core prefill attention, up to 2048 tokens at a time
    ids = synth.rng(40).integers(0, cfg["vocab"], max(prefill, 1))
    dec.prefill(ids[:prefill], chunk=2048)                   # warms code and buffers; rows are rewritten below
    dec.L.dh_sync()
    t0 = time.perf_counter()
    tok = dec.prefill(ids[:prefill], chunk=2048)
    dec.L.dh_sync()
    prefill_s = time.perf_counter() - t0
    log("[bench] prefill of %d positions in %.3f s (%.0f tokens/s)" % (prefill, prefill_s, prefill / prefill_s))

    pos = prefill
    for _ in range(args.warmup):
        tok = dec.step(tok, pos)
        pos += 1
    torch.cuda.synchronize()
    capi_sync = dec.L.dh_sync
    capi_sync()
    # the timed region: K greedy steps through the generation loop (every token read back, one step late:
    # HipDecoder.decode_greedy), then the same K positions again one blocking step at a time for comparison
    dec.decode_greedy(tok, pos, 2)                # pinned staging memory and events are made here, outside the timing
    capi_sync()
    t0 = time.perf_counter()
    tokens = dec.decode_greedy(tok, pos, args.steps)
    capi_sync()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    tok_s = args.steps / elapsed
    t0 = time.perf_counter()
    tokens_blocking = []
    t_ = tok
    for i in range(args.steps):
        t_ = dec.step(t_, pos + i)
        tokens_blocking.append(t_)
    capi_sync()
    blocking_tok_s = args.steps / (time.perf_counter() - t0)
    if tokens_blocking != tokens:
        log("[bench] FAILED: the generation loop and the blocking steps disagree: %r vs %r" % (tokens[:8], tokens_blocking[:8]))
        sys.exit(1)
    tok = tokens[-1]
    pos += args.steps
    log("[bench] the same %d steps, one blocking step at a time: %.1f tok/s" % (args.steps, blocking_tok_s))
    ctx_mid = prefill + args.warmup + args.steps // 2
    step_bytes = dec.weight_bytes_per_token(ctx_mid)
    log("[bench] %d steps in %.3f s -> %.1f tok/s (%.0f GB/s of algorithmic traffic)" %
        (args.steps, elapsed, tok_s, step_bytes * tok_s / 1e9))

    # ---- side measurement: the same steps submitted 16 at a time with the token fed back on the
    #      device (the reference's batched decode); not the headline value, which keeps the
    #      reference's default of one token readback per step
    dec.decode_batch(tok, pos, BATCH)
    capi_sync()
    t0 = time.perf_counter()
    dec.decode_batch(tok, pos + BATCH, BATCH)
    capi_sync()
    batched_tok_s = BATCH / (time.perf_counter() - t0)
    log("[bench] batched decode, %d tokens per submit: %.1f tok/s" % (BATCH, batched_tok_s))

    # ---- side measurement: the step captured once into a HIP graph and replayed (one launch per
    #      token instead of ~220); same kernels, same readback
    pos_g = pos + 2 * BATCH
    gtok = dec.step_graph(tok, pos_g)                 # eager run + capture + first replay
    for i in range(1, 4):
        gtok = dec.step_graph(gtok, pos_g + i)
    capi_sync()
    n_graph = min(32, max_seq - (pos_g + 4))
    t0 = time.perf_counter()
    for i in range(n_graph):
        gtok = dec.step_graph(gtok, pos_g + 4 + i)
    capi_sync()
    graph_tok_s = n_graph / (time.perf_counter() - t0)
    dec.release_graph()
    log("[bench] graph replay: %.1f tok/s" % graph_tok_s)

    # ---- side measurements (A/B, same positions rewritten): the captured step with its attention
    #      nodes moved by the host before every replay instead of reading the key count on the device
    def timed_steps(fn, first_tok, n=24):
        t = first_tok
        for i in range(4):
            t = fn(t, pos_g + i)
        capi_sync()
        t0_ = time.perf_counter()
        for i in range(n):
            t = fn(t, pos_g + 4 + i)
        capi_sync()
        return n / (time.perf_counter() - t0_)
    dec.capture_step(pos_g, device_kv_len=False)
    graph_patched_tok_s = timed_steps(dec.step_graph, tok)
    dec.release_graph()
    log("[bench] graph replay with host-patched attention nodes: %.1f tok/s" % graph_patched_tok_s)
    # ... and the eager step with every product its own launch (six per layer)
    unchained_tok_s = None
    if dec.chain_gemvs:
        try:
            dec.set_chain_gemvs(False)
            unchained_tok_s = timed_steps(dec.step, tok)
            log("[bench] eager steps with one launch per product (no chained GEMVs): %.1f tok/s" % unchained_tok_s)
        except Exception as e:      # a side measurement, never a reason to lose the result
            log("[bench] unchained measurement failed: %r" % (e,))
        finally:
            dec.set_chain_gemvs(True)

    # ---- roofline of the dominant kernel
    Hd, I = cfg["hidden"], cfg["inter"]
    launch_bytes = 2 * synth.q4k_nbytes(I, Hd) + 2 * Hd * 4 + I * 4      # weights, x + norm weight, output
    avg_ms = gate_up_kernel_bandwidth(dec, reps=4)
    achieved = launch_bytes / (avg_ms * 1e-3) / 1e9
    # the same product runs inside the decode step as the second phase of the layer's chained launch; that
    # launch as a whole (four products, 108.5 MB) is measured beside it
    chain_roof = None
    if dec.chain_gemvs:
        try:
            m = layer_chain_bandwidth(dec, reps=4)
            if m:
                chain_roof = {"kernel": "chained layer launch: o + residual, RMSNorm + gate/up + SiLU, down + residual, RMSNorm + next q/k/v",
                              "bytes_per_launch": int(m[1]), "avg_launch_us": round(m[0] * 1e3, 2),
                              "achieved": round(m[1] / (m[0] * 1e-3) / 1e9, 1), "frac": round(m[1] / (m[0] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
                log("[bench] chained layer launch: %.2f us, %.0f GB/s" % (chain_roof["avg_launch_us"], chain_roof["achieved"]))
        except Exception as e:      # a side measurement
            log("[bench] chained-launch measurement failed: %r" % (e,))
    roofline = {"bound": "hbm", "kernel": "q4k fused RMSNorm + gate/up GEMV + SiLU [2x12288x4096]", "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "bytes_per_launch": launch_bytes, "avg_launch_us": round(avg_ms * 1e3, 2),
                "traffic": GATE_UP_TRAFFIC_BYTES if (Hd, I) == (4096, 12288) else None,
                "traffic_source": "stored figure from the rocprofv3 FETCH_SIZE / WRITE_SIZE runs summarised under "
                                  "profiles/ (not measured in this run)",
                "in_step": chain_roof}

    if args.copy_calibration:
        # a streaming kernel of known traffic: reads 64 MiB of f32, writes 32 MiB of f16
        from doppler_amd import capi as _capi
        src = torch.ones(16 << 20, dtype=torch.float32, device="cuda")
        dst = torch.empty(16 << 20, dtype=torch.float16, device="cuda")
        for _ in range(3):
            _capi.check(dec.L.dh_cast_f32_to_f16(src.data_ptr(), dst.data_ptr(), src.numel()))
        capi_sync()

    # ---- CPU baseline: the oracle's decode step (a restatement of the reference's JS per-op
    #      references) on this host, same weights, same KV
    cpu = None
    if not args.no_cpu_baseline:
        import oracle
        ol = []
        for i, l in enumerate(layers):
            d = dict(l)
            k, v = dec.read_kv(i, prefill)
            d["cache_k"] = np.zeros((max_seq, cfg["kv_heads"], cfg["head_dim"]), np.uint16)
            d["cache_v"] = np.zeros_like(d["cache_k"])
            d["cache_k"].reshape(-1)[:k.size] = k
            d["cache_v"].reshape(-1)[:v.size] = v
            ol.append(d)
        ocl = oracle.DecoderOracle(cfg, ol, embed, final_norm, cos, sin)
        n_cpu, t_cpu, ctok = 0, 0.0, int(ids[-1])
        t0 = time.perf_counter()
        while n_cpu < 3 or (t_cpu < 12.0 and n_cpu < 64):
            ctok = ocl.step(ctok, prefill + n_cpu)
            n_cpu += 1
            t_cpu = time.perf_counter() - t0
        threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        js = js_reference_timings()
        cpu = {"value": round(n_cpu / t_cpu, 4), "unit": "tokens/s", "cores": threads, "host_cpus": os.cpu_count(),
               "kind": "port",
               "sample": "%d full decode steps of the same model from the same prefilled KV cache "
                         "(C restatement of the reference's JS per-op references, f64 accumulate, OpenMP)" % n_cpu,
               # the reference's CPU path is single-threaded JavaScript: the same per-op references
               # restated in JS and timed under this host's node, per-op, on the small configs
               "js_port_single_thread_ms": js}

    # ---- the same model through the JavaScript host (the reference's host language): RDRR artifact
    #      written to memory-backed storage, read by the JS loader, decoded through the N-API addon
    js_host = None
    if not args.no_js_host:
        js_host = js_host_decode(cfg, layers, embed, final_norm, prefill, args.warmup, min(args.steps, 48))

    out = {
        "metric": "decode tokens/sec at 9B-class Q4_K, 1 GPU (Q4_K GEMV HBM GB/s in roofline)",
        "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32 activations and sums; Q4_K products on the int8 matrix cores with activations as 21-bit block fixed point (one exponent per 32-element sub-block, exact int32 sums); f16 KV cache and LM head", "data": "synthetic",
        "config": {"workload": "BASELINE configs[4]: 36-layer 9B-class Q4_K decoder, hidden 4096, FFN 12288, "
                               "32/8 heads x128, vocab 151936, KV prefilled to %d, greedy, batch 1" % prefill,
                   "layers": cfg["layers"], "context": prefill, "algorithmic_bytes_per_step": step_bytes,
                   "hbm_frac_whole_step": round(step_bytes * tok_s / 1e9 / HBM_PEAK_GBPS, 4),
                   "batched_decode_16_per_submit_tokens_per_s": round(batched_tok_s, 2),
                   "graph_replay_tokens_per_s": round(graph_tok_s, 2),
                   "graph_replay_host_patched_tokens_per_s": round(graph_patched_tok_s, 2),
                   "blocking_step_tokens_per_s": round(blocking_tok_s, 2),
                   "launches_per_layer": 2 if dec.chain_merges_attention else (3 if dec.chain_gemvs else 6),
                   "unchained_tokens_per_s": round(unchained_tok_s, 2) if unchained_tok_s else None,
                   "js_host": js_host,
                   "prefill_tokens_per_s": round(prefill / prefill_s, 1)},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "tokens_head": tokens[:4],
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
