"""Benchmark of the wave-index decode attention step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c1|c4|c5] [--layers L]

A step is one layer's decode attention (retroinfer_cache.compute) for the whole batch: centroid
scoring, zone selection, estimation zone and attention over steady zone + retrieved clusters,
with the index and all K/V resident in HBM before the timed region.  Step i runs layer
i mod L; every layer has its own seeded synthetic K/V and index, built by the library's own
prefill k-means.  Prints one JSON line (see the keys at the bottom).
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # bytes/s, MI355X
# 16-bit element type of queries, keys, values and the index (--dtype): bfloat16 is the benchmark's, IEEE half
# the default of the reference's harnesses (simple_test.py:29, throughput_eval/test.py:28)
DT, DT_NAME = torch.bfloat16, "bf16"

# HBM bytes per attend_kernel launch come from rocprofv3 counter runs of this script (FETCH_SIZE and
# WRITE_SIZE, each scaled by what the counter reads for the known-size copy of --copy-probe): the figures
# sit in a small data file next to the summary they were taken from, with a hash of the kernel source
# they were measured on; a figure measured on another version of the kernel is not reported.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "attend_kernel_traffic.json")
ATTEND_SOURCES = [os.path.join(ROOT, "retrievalattention_amd", "csrc", f) for f in ("attend.hip", "attend_common.h")]


def kernel_source_hash():
    import hashlib
    h = hashlib.sha256()
    for f in ATTEND_SOURCES:
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def measured_traffic(config):
    """(bytes per attend_kernel launch or None, where the figure comes from)."""
    try:
        with open(TRAFFIC_FILE) as fh:
            rec = json.load(fh).get(config)
    except (OSError, ValueError):
        return None, f"{os.path.relpath(TRAFFIC_FILE, ROOT)} missing"
    if not rec:
        return None, f"no counter run recorded for {config}"
    if rec.get("kernel_source_sha256_16") != kernel_source_hash():
        return None, f"{rec['source']}: measured on another version of the kernel (stale, not reported)"
    nbytes = int((rec["fetch_kib"] * rec["fetch_scale"] + rec["write_kib"] * rec["write_scale"]) * 1024)
    return nbytes, rec["source"]

CONFIGS = {
    # name: batch, kv heads, group size, clustered tokens, mixture centres, centroids, segments, outliers, layers
    "c1": dict(B=1, Hkv=8, gs=4, N=8192, K=512, nc=512, S=1, outliers=False, L=1,
               desc="Llama-3-8B shape, batch 1, 8192 tokens, 512 centroids"),
    "c2": dict(B=4, Hkv=8, gs=4, N=131072, K=8192, nc=8192, S=16, outliers=True, L=32,
               desc="Llama-3-8B shape (32 q / 8 kv heads, dim 128), batch 4, 131072 tokens, 8192 centroids"),
    "c4": dict(B=16, Hkv=4, gs=7, N=61440, K=3840, nc=3840, S=8, outliers=False, L=28,
               desc="Qwen2.5-7B shape, batch 16, 61440 tokens, 3840 centroids (device-resident variant)"),
    "c5": dict(B=8, Hkv=8, gs=8, N=262144, K=16384, nc=16384, S=32, outliers=True, L=1,
               desc="Qwen2.5-72B single layer, batch 8, 262144 tokens, 16384 centroids"),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_cache(cfg, L, dev, residency="device", block_cache="device", estimate_next=False, new=2,
                device_positions=False, overlap_miss_staging=False):
    from retrievalattention_amd import synth
    from retrievalattention_amd.cache_hub import retroinfer_cache
    B, Hkv, gs, N = cfg["B"], cfg["Hkv"], cfg["gs"], cfg["N"]
    nprobe = max(1, int(cfg["nc"] * 0.018))
    es = int(cfg["nc"] * 0.232)
    ctx = N + synth.STEADY_START + synth.STEADY_END
    cache = retroinfer_cache(
        valid_start=[0] * B, layer_num=L, batch_size=B, max_length=ctx + new, num_key_value_heads=Hkv,
        num_heads=Hkv * gs, head_dim=128, dtype=DT, layer_mapping={str(l): "cuda:0" for l in range(L)},
        max_new_length=new, static_pattern_start=synth.STEADY_START, static_pattern_end=synth.STEADY_END, core=8,
        n_centroids=cfg["nc"], n_segment=cfg["S"], nprobe=nprobe, max_compute_cluster_num=nprobe + es,
        cache_unit_size=8, cache_cluster_num=max(int(cfg["nc"] * 0.05), nprobe), num_gpus=1, model_size=0,
        kv_residency=residency,
        block_cache=block_cache, use_cluster_estimation=estimate_next, device_positions=device_positions,
        overlap_miss_staging=overlap_miss_staging)
    queries = []
    t0 = time.time()
    for l in range(L):
        qs = []
        for b in range(B):
            ks, vs = [], []
            for h in range(Hkv):
                k, v, q = synth.make_group(l, b, h, N, cfg["K"], gs, outliers=cfg["outliers"],
                                           n_extra=synth.STEADY_START + synth.STEADY_END, device=dev)
                # steady zone = the extra tokens: 4 first, 64 last
                k = torch.cat([k[N:N + 4], k[:N], k[N + 4:]]).to(DT)
                v = torch.cat([v[N:N + 4], v[:N], v[N + 4:]]).to(DT)
                ks.append(k); vs.append(v); qs.append(q.to(DT))
            K = torch.stack(ks, 1)[None].contiguous()   # [1, ctx, Hkv, D]
            V = torch.stack(vs, 1)[None].contiguous()
            cache.prefill_update_kv_cache(None, K, V, l, b)
            cache.sync(l, b)
            del K, V, ks, vs
        queries.append(torch.cat(qs).view(B, 1, Hkv * gs, 128).contiguous())
        if l == 0 or (l + 1) % 8 == 0:
            torch.cuda.synchronize()
            log(f"[bench] built layer {l + 1}/{L} ({time.time() - t0:.1f}s)")
    cache.prepare_cache()
    cache.temp_keys = cache.temp_values = None
    torch.cuda.empty_cache()
    # one generated token per layer so that the steady zone has its 69th entry
    g = torch.Generator(device=dev).manual_seed(12345)
    for l in range(L):
        kn = torch.randn(B, 1, Hkv, 128, generator=g, device=dev).to(DT)
        vn = torch.randn(B, 1, Hkv, 128, generator=g, device=dev).to(DT)
        cache.decode_update_kv_cache(kn, vn, l)
    return cache, queries, nprobe, es


def algorithmic_bytes(cache, cfg, nprobe, es, layer, static_len):
    """HBM bytes one decode layer-step has to touch: centroids once, queries, mask, value-sum rows
    and sizes of the estimation zone, K and V of retrieved + steady tokens once, output."""
    BG, gs, nc, D, e = cfg["B"] * cfg["Hkv"], cfg["gs"], cfg["nc"], 128, 2
    if getattr(cache, "meta", None) is not None:
        t_ret = cache.meta[:, 1].sum().item()
    else:   # worker-thread block cache manager: no device-side layout record, the valid lengths hold the same count
        t_ret = int((cache.valid_lengths[layer % 2] - static_len).sum().item())
    parts = {
        "centroids": BG * nc * D * e + BG * gs * D * e + BG * nc,
        "estimation": BG * es * (D * e + e),
        "kv": 2 * e * D * (t_ret + BG * static_len),
        "out": BG * gs * D * e,
    }
    return parts, t_ret


def read_probe(dev, mib=64, nbuf=24):
    """What a read-only kernel reaches: ri_probe_stream_read over `nbuf` buffers of `mib` MiB in turn
    (1.5 GiB in all, far more than the 256 MB last-level cache holds), one launch per buffer inside a
    HIP graph, for several workgroup counts and loads in flight; best of five replays each."""
    from retrievalattention_amd import _lib
    lib = _lib.lib()
    nbytes = mib << 20
    bufs = [torch.ones(nbytes, dtype=torch.uint8, device=dev) for _ in range(nbuf)]
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    out = {}
    for wgs in (256, 512, 1024, 2048, 4096):
        for u in (4, 8, 16):
            def launches():
                st = torch.cuda.current_stream().cuda_stream
                for b in bufs:
                    _lib.check(lib.ri_probe_stream_read(b.data_ptr(), nbytes, wgs, u, sink.data_ptr(), st), "probe")
            launches()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                launches()
            best = float("inf")
            for _ in range(5):
                best = min(best, time_region(g.replay, 2))
            out[f"{wgs}x256_threads_{u}_loads"] = round(nbytes * nbuf / best / 1e9, 1)
    top = max(out, key=out.get)
    return {"unit": "GB/s", "bytes_per_launch": nbytes, "buffers_cycled": nbuf, "best": top, "best_GBps": out[top],
            "frac_of_peak": out[top] * 1e9 / HBM_PEAK, "all": out}


def time_region(fn, iters):
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) * 1e-3 / iters


MFMA_BF16_PEAK = 2.5e15  # FLOP/s, MI355X dense bf16


def bench_kmeans(cfg, dev, iters=10, reps=3):
    """Prefill clustering of one sequence (all kv heads) with the library's own driver:
    9 segmented spherical Lloyd iterations + 1 global one + value sums + inverted lists."""
    from retrievalattention_amd import synth, kernels
    from retrievalattention_amd.cache_hub.kmeans import segment_k_means_csr
    Hkv, N, nc, S = cfg["Hkv"], cfg["N"], cfg["nc"], cfg["S"]
    ks, vs = [], []
    for h in range(Hkv):
        k, v, _ = synth.make_group(0, 0, h, N, cfg["K"], cfg["gs"], outliers=cfg["outliers"], n_extra=0, device=dev)
        ks.append(k.to(DT)); vs.append(v.to(DT))
    K, V = torch.stack(ks).contiguous(), torch.stack(vs).contiguous()
    K = (K - K.mean(dim=1, keepdim=True)).contiguous()          # keys are centred before clustering
    r = segment_k_means_csr(K, V, nc, iters, S, reuse_graph=False)   # warm-up; its result is kept below
    # the library replays a clustering as one captured graph from the third call with keys at the same
    # address on (as every layer and sequence of a prefill after the first two does): two untimed calls
    for _ in range(2):
        segment_k_means_csr(K, V, nc, iters, S, reuse_graph=True)
    t = time_region(lambda: segment_k_means_csr(K, V, nc, iters, S, reuse_graph=True), reps)
    # the global assignment alone: the one launch that holds most of the FLOPs
    assign = torch.empty((Hkv, N), dtype=torch.int32, device=dev)
    t_as = time_region(lambda: kernels.kmeans_assign(K, r.centroids, assign, Hkv, N, nc, 1, N), reps)
    flops = 2.0 * 128 * Hkv * N * ((iters - 1) * nc / S + nc)
    flops_as = 2.0 * 128 * Hkv * N * nc
    # the same clustering without segments (every iteration scores all centroids), from a seeded
    # random choice of initial tokens
    g = torch.Generator(device=dev).manual_seed(0)
    init = torch.sort(torch.randperm(N, generator=g, device=dev)[:nc]).values
    for _ in range(2):
        segment_k_means_csr(K, V, nc, iters, 1, init_indices=init, reuse_graph=True)
    t_un = time_region(lambda: segment_k_means_csr(K, V, nc, iters, 1, init_indices=init, reuse_graph=True), reps)
    flops_un = 2.0 * 128 * Hkv * N * iters * nc
    unseg = {"ms_per_sequence": t_un * 1e3, "algorithmic_flops": flops_un, "achieved": flops_un / t_un / 1e12,
             "frac": flops_un / t_un / MFMA_BF16_PEAK, "init": "seeded random tokens"}
    return {"unsegmented": unseg, "ms_per_sequence": t * 1e3, "tokens": N, "kv_heads": Hkv, "centroids": nc, "segments": S,
            "iterations": iters, "algorithmic_flops": flops, "bound": "mfma", "achieved": flops / t / 1e12,
            "peak": MFMA_BF16_PEAK / 1e12, "unit": "TFLOP/s", "frac": flops / t / MFMA_BF16_PEAK,
            "global_assign": {"us": t_as * 1e6, "achieved": flops_as / t_as / 1e12,
                              "frac": flops_as / t_as / MFMA_BF16_PEAK}}


def kmeans_cpu_baseline(cfg, iters=10):
    """The CPU restatement of the clustering (oracle/kmeans.py) on a bounded sample of the same keys: the nine
    segmented iterations of ONE 8192-token segment of one head, and the final assignment + update of 8192 of
    the head's tokens against all its centroids; scaled linearly to one sequence (all heads, all segments, all
    tokens).  The arithmetic per token and centroid is the same for every segment and head, so the scaling is
    by counts only."""
    from oracle import kmeans as okm
    from retrievalattention_amd import synth
    torch.set_num_threads(os.cpu_count() or 1)
    Hkv, N, nc, S = cfg["Hkv"], cfg["N"], cfg["nc"], cfg["S"]
    nseg, ncs = N // S, nc // S
    k, _, _ = synth.make_group(0, 0, 0, N, cfg["K"], cfg["gs"], outliers=cfg["outliers"], n_extra=0)
    k = k.to(DT)
    k = (k - k.mean(dim=0, keepdim=True)).contiguous()
    cent = k[okm.init_indices(N, nc)].clone()
    d, c = k[:nseg], cent[:ncs]
    t0 = time.time()
    for _ in range(iters - 1):
        c, _, _ = okm.train_step(d, c, True)
    t_seg = time.time() - t0
    sample = min(N, 8192)
    t0 = time.time()
    okm.train_step(k[:sample], cent, False)
    t_glob = time.time() - t0
    per_seq = Hkv * (S * t_seg + (N / sample) * t_glob)
    return {"ms_per_sequence": per_seq * 1e3, "unit": "ms", "cores": torch.get_num_threads(), "kind": "port",
            "measured_s": {"segment_sweep_9_iterations": t_seg, "final_pass_on_sample_tokens": t_glob},
            "sample": f"oracle/kmeans.py on head 0 of the same keys: {iters - 1} segmented iterations of one {nseg}-token "
                      f"segment ({ncs} centroids) and the final pass over {sample} tokens against {nc} centroids, "
                      f"{t_seg + t_glob:.1f} s of CPU work",
            "extrapolation": f"{Hkv} heads x ({S} segments x segment sweep + {N // sample} x final-pass sample): linear "
                             f"in tokens, segments and heads",
            "note": "the checker's restatement (float64 scores, numpy), not a tuned CPU implementation"}


def cpu_baseline(cache, cfg, queries, nprobe, es, static_len, max_seconds=10.0, max_samples=100, min_samples=3):
    """The CPU restatement (oracle/) of the same decode step, layer 0, on the host cores."""
    from oracle import pipeline
    BG, gs = cfg["B"] * cfg["Hkv"], cfg["gs"]
    torch.set_num_threads(os.cpu_count() or 1)
    l = 0
    rows = cache.store_rows[l]
    sk = [cache.list_keys[l].view(BG, -1, 128)[g, :rows[g]].cpu().clone() for g in range(BG)]
    sv = [cache.list_values[l].view(BG, -1, 128)[g, :rows[g]].cpu().clone() for g in range(BG)]
    args = (queries[l].view(BG, gs, 128).cpu(), cache.steady_zone_keys[l].view(BG, -1, 128).cpu(),
            cache.steady_zone_values[l].view(BG, -1, 128).cpu(), static_len, cache.centroids[l].cpu(),
            cache.value_sum[l].cpu(), cache.centroids_mask[l].cpu(), cache.cluster_size_i32[l].cpu(),
            cache.cluster_size[l].cpu(), sk, sv, cache.cluster_start[l].cpu().long(), nprobe, es, 8,
            cache.buffer_size)
    if min_samples > 1:
        pipeline.decode_step(*args)  # warm-up
    times = []
    t_all = time.time()
    while len(times) < max_samples and (len(times) < min_samples or time.time() - t_all < max_seconds):
        t0 = time.time()
        ref, _ = pipeline.decode_step(*args)
        times.append(time.time() - t0)
    times.sort()
    return times[len(times) // 2], len(times), ref


def bench_estimate_next(args, cache, queries, outs, L, static_len):
    """The reference's use_cluster_estimation mode over the device-resident store: layers 0 and 1 choose
    their zones from their own query; every later layer's zones are chosen at the end of the layer before
    it, from a predicted query.  The bench predicts perfectly (the next layer's true query), so
    the outputs must agree with those of the plain step; one pass over the L layers is one decoded token."""
    def step(l):
        return cache._compute(queries[l], l, queries[l + 1] if l + 1 < L else None, static_len)

    for l in range(L):
        o = step(l)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for l in range(L):
            step(l)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    cycle = torch.cuda.CUDAGraph()
    with torch.cuda.graph(cycle):
        cyc_outs = [step(l) for l in range(L)]
    cycle.replay()
    torch.cuda.synchronize()
    # same zones as the plain step; the estimation zone's scores come from another accumulation order
    for l in range(L):
        d = (cyc_outs[l].float() - outs[l].float()).abs()
        if float(d.max()) > 2e-2 or float(d.mean()) > 2e-3:
            sys.exit(f"next-layer estimation: layer {l} differs from the plain step (max-abs {float(d.max())})")
    n_cyc = max(1, args.steps // L)
    for _ in range(max(1, args.warmup // L)):
        cycle.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_cyc):
        cycle.replay()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / (n_cyc * L)
    return {"us_per_layer_step": t * 1e6, "layers_per_token": L,
            "note": "zones of layer l+1 chosen at the end of layer l from the (here exact) "
                    "predicted query; layers 0 and 1 select for themselves; outputs checked against the plain step"}


def bench_end_to_end(args, cfg, dev):
    """A whole decoded token of a Llama-shaped model (random weights, the config's attention shape)
    around the wave-index cache built from the synthetic K/V: every layer's norm, QKV projection,
    rotary embedding, cache append, wave-index attention, output projection and MLP, captured once as
    one HIP graph and replayed token after token (the steady zone grows by one row per token)."""
    from retrievalattention_amd.model_hub import LlamaModel, LlamaShape
    L, B, tokens = cfg["L"], cfg["B"], args.steps
    heads = cfg["Hkv"] * cfg["gs"]
    shape = LlamaShape(hidden_size=heads * 128, intermediate_size=cfg.get("ffn", 14336), num_layers=L, num_heads=heads,
                       num_key_value_heads=cfg["Hkv"], head_dim=128, vocab_size=128256)
    cache, queries, nprobe, es = build_cache(cfg, L, dev, new=tokens + args.warmup + 8, device_positions=True)
    del queries
    ctx = cache.context
    model = LlamaModel(shape, ctx + tokens + args.warmup + 16, device=dev, seed=0)
    model.kv_cache, model.attention_type = cache, "RetroInfer"
    model.position.fill_(ctx)
    tok = torch.zeros(B, 1, dtype=torch.int64, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        logits = model.decode_forward(tok)          # first token eagerly (warm-up for the capture)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        logits = model.decode_forward(tok)
    def one():
        graph.replay()
        cache.token_replayed()
        tok.copy_(logits.argmax(-1))
    for _ in range(args.warmup):
        one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(tokens):
        one()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / tokens
    weights = sum(w.numel() * 2 for l in model.layers for w in (l.wqkv, l.wo, l.gate_up_proj, l.down_proj)) + model.lm_head.numel() * 2
    print(json.dumps({
        "metric": "decode tokens/s end to end (random-weight model of the config's shape around the wave-index cache)",
        "value": B / t, "unit": "tokens/s", "n_gpus": 1, "steps": tokens, "warmup": args.warmup, "ms_per_step": t * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": DT_NAME, "data": "synthetic",
        "config": {"workload": f"{args.config}: {cfg['desc']}; {L} layers, hidden {shape.hidden_size}, MLP "
                               f"{shape.intermediate_size}, vocabulary {shape.vocab_size}; one HIP graph per token",
                   "batch": B, "context_tokens": ctx, "weight_bytes": weights,
                   "weights_at_hbm_peak_ms": weights / HBM_PEAK * 1e3},
        "roofline": None, "cpu_baseline": None}))


def bench_host(args, cfg, cache, queries, L, nprobe, es, static_len, config_name=None, cpu_seconds=10.0):
    """Host-resident clustered K/V: the reference's operator sequence (score+select, id copy to the
    host, block-cache look-up on the worker pool, gather of misses over the host link and hits
    from the device cache, attention, cache admission).  The first pass over the layers runs
    with an empty block cache (every retrieved block is a miss); repeating the same queries then
    hits for every block that was admitted."""
    B = cfg["B"]

    def step(l):
        return cache._compute(queries[l], l, None, static_len)

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for l in range(L):
        step(l)
    torch.cuda.synchronize()
    t_cold = (time.perf_counter() - t0) / L
    use_graph = cache.block_cache == "device" and not args.no_graph
    if use_graph:
        # the device-side manager has no host round trip: the steps replay as HIP graphs.  A graph
        # launch has a fixed cost of its own, so one graph holds a cycle of the layers, and the warm
        # measurement (same queries every time) one graph of several cycles
        cycle = torch.cuda.CUDAGraph()
        with torch.cuda.graph(cycle):
            for l in range(L):
                step(l)
        reps = max(1, 32 // L)
        multi = torch.cuda.CUDAGraph()
        with torch.cuda.graph(multi):
            for _ in range(reps):
                for l in range(L):
                    step(l)
        run_cycle = cycle.replay
        run_many, many = multi.replay, reps * L
    else:
        def run_cycle():
            for l in range(L):
                step(l)
        run_many, many = run_cycle, L
    for _ in range(max(1, args.warmup // many)):
        run_many()
    torch.cuda.synchronize()
    n_warm = max(1, args.steps // many)
    t0 = time.perf_counter()
    for _ in range(n_warm):
        run_many()
    torch.cuda.synchronize()
    t_warm = (time.perf_counter() - t0) / (n_warm * many)
    stats = [cache.block_cache_stats(l) for l in range(L)]
    hit, miss = sum(s_[0] for s_ in stats), sum(s_[1] for s_ in stats)
    # drifting queries: each step's query is the layer's query plus noise drawn from a small pool, so
    # part of every probe list is new and its blocks come over the host link
    drift = {}
    for sigma in [float(x) for x in args.drift.split(",") if x]:
        g = torch.Generator(device=queries[0].device).manual_seed(7)
        base = [q.clone() for q in queries]
        pool = [[(b.float() + sigma * b.float().std() * torch.randn(b.shape, generator=g, device=b.device))
                 .to(b.dtype) for _ in range(8)] for b in base]

        def drift_cycle(c):
            for l in range(L):
                queries[l].copy_(pool[l][c % 8])
            run_cycle()

        n_cyc = max(1, args.steps // L)
        for c in range(max(1, args.warmup // L)):
            drift_cycle(c)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for c in range(n_cyc):
            drift_cycle(c)
        torch.cuda.synchronize()
        t_d = (time.perf_counter() - t0) / (n_cyc * L)
        # hit and miss blocks of 8 more (untimed) cycles
        dh = dm = 0
        for c in range(n_cyc, n_cyc + 8):
            drift_cycle(c)
            torch.cuda.synchronize()
            for l in range(L):
                h_, m_ = cache.block_cache_stats(l)
                dh += h_
                dm += m_
        per_step_miss = dm / (8 * L)
        drift[f"noise_{sigma}"] = {"us_per_layer_step": t_d * 1e6, "hit_blocks_sampled": dh, "miss_blocks_sampled": dm,
                                   "hit_fraction": dh / max(dh + dm, 1),
                                   "host_link_GBps": per_step_miss * 8 * 128 * 2 * 2 / t_d / 1e9}
        for q, b in zip(queries, base):
            q.copy_(b)
    # warm steady state, stage by stage: the same layer cycle launched eagerly with an event pair around
    # each stage (every retrieved block hits: the stream of cache blocks, estimation rows and steady zone
    # through attend_kernel is what moves the bytes)
    BG, gs = cfg["B"] * cfg["Hkv"], cfg["gs"]
    stage_us = None
    if cache.block_cache == "device":
        from retrievalattention_amd import kernels
        names = ["score_select", "lru_access_update", "concat_gather (miss staging)", "attention", "admission scatter"]
        n_k = max(L, min(args.steps, 128) // L * L)
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(6)] for _ in range(n_k)]
        D, rows, stage0 = 128, cache.cache_blocks * cache.page_size, cache.cache_size * cache.page_size
        out_tmp = torch.empty((BG, gs, D), dtype=DT, device=queries[0].device)
        for i in range(n_k):
            l, e = i % L, ev[i]
            q = queries[l].view(BG, gs, D)
            ck, cv = cache.cache_keys[l].view(BG, rows, D), cache.cache_values[l].view(BG, rows, D)
            e[0].record()
            cache._select(queries[l], l, 0, False)
            e[1].record()
            cache._access_in_place(l, 0)
            e[2].record()
            cache._stage_misses(l, 0)
            e[3].record()
            kernels.wave_attention(q, cache.steady_zone_keys[l], cache.steady_zone_values[l], static_len, ck, cv,
                                   cache.row_src, cache.meta, cache.est_ids[0] if es > 0 else None,
                                   cache.logits if es > 0 else None, cache.value_sum[l], cache.cluster_size[l], out_tmp,
                                   cache.valid_lengths[0], es, cache.RSQRT_DIM)
            e[4].record()
            kernels.gather_copy_and_scatter(
                ck[:, stage0:], cache.cache_keys[l], cv[:, stage0:], cache.cache_values[l],
                cache.update_buffer_indices[l], cache.update_unit_sizes[l], cache.update_cache_indices[l],
                cache.update_num_units[l], BG, rows, cache.cache_stride, cache.buffer_size, 0)
            e[5].record()
            if i % 16 == 15:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        stage_us = {nm: sum(e[k].elapsed_time(e[k + 1]) for e in ev) * 1e3 / n_k for k, nm in enumerate(names)}
    elif es > 0:
        # worker-thread manager: the attention launch over the execution buffer as the last warm step left it
        # (hits and staged misses assembled behind the steady zone), an event pair around each eager launch
        from retrievalattention_amd import kernels
        l, n_k = L - 1, 32
        buf = l % 2
        out_tmp = torch.empty((BG, gs, 128), dtype=DT, device=queries[0].device)
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(n_k)]
        for e in ev:
            e[0].record()
            kernels.buffer_attention(queries[l].view(BG, gs, 128), cache.execution_buffer_keys[buf],
                                     cache.execution_buffer_values[buf], cache.valid_lengths[buf], cache.est_ids[buf],
                                     cache.logits, cache.value_sum[l], cache.cluster_size[l], out_tmp, es,
                                     cache.RSQRT_DIM)
            e[1].record()
        torch.cuda.synchronize()
        stage_us = {"attention": sum(e[0].elapsed_time(e[1]) for e in ev) * 1e3 / n_k}
    parts, t_ret = algorithmic_bytes(cache, cfg, nprobe, es, (L - 1), static_len)
    attn_bytes = parts["estimation"] + parts["kv"] + parts["out"]
    total_bytes = sum(parts.values())
    roofline = None
    if stage_us is not None:
        t_attn = stage_us["attention"] * 1e-6
        where = ("ri_wave_attention over the block cache, every block a hit" if cache.block_cache == "device"
                 else "ri_buffer_attention over the assembled execution buffer")
        traffic, traffic_source = measured_traffic(f"{config_name or args.config}_host")
        roofline = {"bound": "hbm", "kernel": f"attend_kernel ({where})",
                    "achieved": attn_bytes / t_attn / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                    "frac": attn_bytes / t_attn / HBM_PEAK, "traffic": traffic,
                    "traffic_source": traffic_source,
                    "launch_us": stage_us["attention"], "algorithmic_bytes": attn_bytes,
                    "note": "event pair around one eager launch (includes its dispatch)"}
    cpu = None
    if not args.no_cpu_baseline:
        t_cpu, n, ref = cpu_baseline(cache, cfg, queries, nprobe, es, static_len, max_seconds=cpu_seconds,
                                     min_samples=3 if cpu_seconds > 0 else 1)
        out0 = step(0)
        torch.cuda.synchronize()
        d = (out0.view(BG, gs, 128).cpu().float() - ref.float()).abs()
        cpu = {"value": B / (cfg["L"] * t_cpu), "unit": "tokens/s", "us_per_layer_step": t_cpu * 1e6,
               "cores": torch.get_num_threads(), "kind": "port",
               "sample": f"median of {n} full-shape decode layer-steps of layer 0 (oracle/pipeline.py)",
               "note": "the checker's restatement, not a tuned CPU implementation: float64 matrix products and a "
                       "Python loop over the groups",
               "max_abs_vs_gpu": float(d.max()), "mean_abs_vs_gpu": float(d.mean())}
    link = max((v["host_link_GBps"] for v in drift.values()), default=0.0)
    # what the link gives a plain copy: 256 MiB from pinned host memory to the device, best of 5
    pin = torch.empty(256 << 20, dtype=torch.uint8, pin_memory=True)
    dst = torch.empty(256 << 20, dtype=torch.uint8, device=queries[0].device)
    t_copy = float("inf")
    for _ in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dst.copy_(pin, non_blocking=True)
        torch.cuda.synchronize()
        t_copy = min(t_copy, time.perf_counter() - t0)
    link_peak = pin.numel() / t_copy / 1e9
    del pin, dst
    return ({
        "metric": "decode tokens/s at 128K ctx (attention only, B / (L * t_layer_step)); us/layer-step and % HBM roofline alongside",
        "value": B / (cfg["L"] * t_warm), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": t_warm * 1e3, "us_per_layer_step": t_warm * 1e6, "cold_us_per_layer_step": t_cold * 1e6,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": DT_NAME, "data": "synthetic",
        "config": {"workload": f"{args.config}: {cfg['desc']}; clustered K/V in pinned host memory, block cache of "
                               f"{cache.cache_size if hasattr(cache, 'cache_size') else '?'} blocks per group, "
                               f"block cache manager on the {cache.block_cache}, miss staging "
                               f"{'beside' if cache.overlap_miss_staging else 'before'} the attention, nprobe {nprobe}, "
                               f"estimation zone {es}, {L} layers, "
                               f"{'HIP graph replay (a cycle of the layers per graph)' if use_graph else 'eager launches'}, warm = same "
                               f"queries repeated", "batch": B, "context_tokens": cfg["N"],
                   "layers_for_tokens_per_s": cfg["L"], "warm_hit_blocks": hit, "warm_miss_blocks": miss},
        "step_roofline": {"bound": "hbm", "algorithmic_bytes": total_bytes, "achieved": total_bytes / t_warm / 1e9,
                          "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": total_bytes / t_warm / HBM_PEAK},
        "stages_us": stage_us,
        "drifting_queries": drift,
        "host_link": {"bound": "host link (pinned host memory read in place by concat_gather_kernel)",
                      "achieved": link, "peak": link_peak, "unit": "GB/s", "frac": link / link_peak if link else None,
                      "note": "achieved = missed K and V bytes per step over the whole step time, best drift level; "
                              "peak = a 256 MiB copy from pinned host memory measured in this run"},
        "roofline": roofline, "cpu_baseline": cpu})


def compact(rec):
    """What an entry of other_configs carries: the step time, both rooflines and the check against the oracle."""
    out = {k: rec[k] for k in ("us_per_layer_step", "cold_us_per_layer_step", "value", "unit", "step_roofline", "roofline",
                               "stages_us", "host_link", "drifting_queries") if k in rec}
    out["workload"] = rec["config"]["workload"]
    cpu = rec.get("cpu_baseline")
    if cpu:
        out["max_abs_vs_oracle"] = cpu["max_abs_vs_gpu"]
        out["mean_abs_vs_oracle"] = cpu["mean_abs_vs_gpu"]
        out["cpu_us_per_layer_step"] = cpu["us_per_layer_step"]
        out["cpu_sample"] = cpu["sample"]
    if "stages" in rec:
        out["stages_us"] = {k: v.get("us_in_step", v["us"]) for k, v in rec["stages"].items()}
    return out


def bench_device(args, cfg, config_name, L, dev, extras=True):
    """The layer-step over a device-resident store for one configuration; returns the record.  extras: the
    read probe, the prefill clustering, next-layer estimation and the full CPU baseline (the headline
    configuration); without them only one CPU layer-step is run, for the check against the oracle."""
    B, Hkv, gs = cfg["B"], cfg["Hkv"], cfg["gs"]
    BG = B * Hkv
    est_next = extras and args.estimate_next and not args.no_graph and L >= 4
    cache, queries, nprobe, es = build_cache(cfg, L, dev, "device", "device", est_next, overlap_miss_staging=False)
    static_len = cache.static_pattern_total  # 4 + 64 + the token being decoded (already counted)

    # every layer-step is "not the last layer" for timing purposes: same static_len everywhere
    def step(l):
        return cache._compute_device(queries[l], l, static_len, l % 2)

    outs = [step(l) for l in range(L)]
    torch.cuda.synchronize()

    graphs = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for l in range(L):
                step(l)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graphs = []
        for l in range(L):
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                o = step(l)
            graphs.append((gr, o))
        torch.cuda.synchronize()
        # replays must reproduce the eager result
        for l in range(L):
            graphs[l][0].replay()
        torch.cuda.synchronize()
        for l in range(L):
            if not torch.equal(graphs[l][1], outs[l]):
                sys.exit(f"graph replay of layer {l} differs from the eager result")

    # one graph for a whole cycle of the L layers (what a decoded token replays): a graph launch has a
    # fixed cost of its own, which a per-layer graph would pay L times per token
    # (a config with few layers repeats its cycle inside the graph, up to 32 steps per graph)
    cycle, CL = None, L * max(1, 32 // L)
    if graphs is not None:
        cycle = torch.cuda.CUDAGraph()
        with torch.cuda.graph(cycle):
            cycle_outs = [step(i % L) for i in range(CL)]
        cycle.replay()
        torch.cuda.synchronize()
        for i in range(CL):
            if not torch.equal(cycle_outs[i], outs[i % L]):
                sys.exit(f"cycle graph: step {i} differs from the eager result")

    # the timed region is exactly args.steps layer-steps: whole graphs of CL steps, then one graph that
    # holds the remaining steps % CL steps
    tail, n_tail = None, args.steps % CL
    if graphs is not None and n_tail:
        tail = torch.cuda.CUDAGraph()
        with torch.cuda.graph(tail):
            for i in range(n_tail):
                step(i % L)

    def run_steps(i0, n):
        """Steps i0 .. i0+n-1 of the layer cycle."""
        i = i0
        while i < i0 + n:
            if cycle is not None and i % CL == 0 and i + CL <= i0 + n:
                cycle.replay()
                i += CL
            elif tail is not None and i % CL == 0 and i + n_tail == i0 + n:
                tail.replay()
                i += n_tail
            else:
                run(i)
                i += 1

    def run(i):
        l = i % L
        if graphs is not None:
            graphs[l][0].replay()
        else:
            step(l)

    run_steps(0, max(args.warmup, CL))
    torch.cuda.synchronize()
    # the timed region (args.steps layer-steps between two synchronisations) is repeated and the median
    # repetition reported.  A region shorter than one graph of CL steps is a single graph replay of about a
    # millisecond, of which the launch from the host and the synchronisation are a visible part (about 1 us per
    # layer-step at 20 steps): such a region replays its graph `inner` times back to back, and the time is
    # divided by all the layer-steps it ran
    inner = max(1, 320 // args.steps) if (graphs is not None and args.steps < CL) else 1
    reps_t = []
    for _ in range(max(args.repeats, 1)):
        t0 = time.perf_counter()
        for _ in range(inner):
            run_steps(0, args.steps)
        torch.cuda.synchronize()
        reps_t.append((time.perf_counter() - t0) / (args.steps * inner))
    reps_t.sort()
    t_step = reps_t[len(reps_t) // 2]

    # the dominant kernel's duration inside the replayed step: the same layer cycle without its launch
    # (score_kernel + dist_kernel + select_kernel only), both cycles timed by one event pair each on the
    # launch stream; the difference is attend_kernel plus the gap in front of it
    t_attn_in_step = None
    if graphs is not None:
        sel_cycle = torch.cuda.CUDAGraph()
        with torch.cuda.graph(sel_cycle):
            for i in range(CL):
                cache._select(queries[i % L], i % L, i % 2, True)
        torch.cuda.synchronize()
        e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        best = [float("inf"), float("inf")]
        n_cyc = max(1, args.steps // CL)
        for _ in range(3):
            for _ in range(2):
                cycle.replay()
            e0.record()
            for _ in range(n_cyc):
                cycle.replay()
            e1.record()
            for _ in range(n_cyc):
                sel_cycle.replay()
            e2.record()
            torch.cuda.synchronize()
            best = [min(best[0], e0.elapsed_time(e1)), min(best[1], e1.elapsed_time(e2))]
        t_attn_in_step = (best[0] - best[1]) * 1e-3 / (n_cyc * CL)
        t_select_in_step = best[1] * 1e-3 / (n_cyc * CL)

    # per-kernel pass: the same layer cycle launched eagerly, one event pair around each entry point's
    # launches on the launch stream (cold caches as in the timed region: every step is another layer)
    from retrievalattention_amd import kernels, _lib
    stream = torch.cuda.current_stream().cuda_stream
    n_k = min(args.steps, 256)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(n_k)]
    out_tmp = torch.empty((BG, gs, 128), dtype=DT, device=dev)

    def attend(l, slot):
        kernels.wave_attention(
            queries[l].view(BG, gs, 128), cache.steady_zone_keys[l], cache.steady_zone_values[l], static_len,
            cache.list_keys[l], cache.list_values[l], None, cache.meta, cache.est_ids[slot], cache.logits,
            cache.value_sum[l], cache.cluster_size[l], out_tmp, cache.valid_lengths[slot], es, cache.RSQRT_DIM,
            ret_tok_off=cache.ret_tok_off, ret_start=cache.ret_start)

    for i in range(n_k + 8):
        l, slot = i % L, i % 2
        e = ev[max(i - 8, 0)]
        e[0].record()
        cache._select(queries[l], l, slot, True)      # score_kernel + dist_kernel + select_kernel
        e[1].record()
        attend(l, slot)                                # attend_kernel (merge fused in)
        e[2].record()
        _lib.check(_lib.lib().ri_null_launch(stream), "ri_null_launch")
        e[3].record()
        if i % 32 == 31:
            torch.cuda.synchronize()                   # keep the launch queue short: events stay adjacent
    torch.cuda.synchronize()
    t_select = sum(e[0].elapsed_time(e[1]) for e in ev) * 1e-3 / n_k
    t_attn = sum(e[1].elapsed_time(e[2]) for e in ev) * 1e-3 / n_k
    t_null = sum(e[2].elapsed_time(e[3]) for e in ev) * 1e-3 / n_k
    parts, t_ret = algorithmic_bytes(cache, cfg, nprobe, es, (n_k + 7) % L, static_len)
    total_bytes = sum(parts.values())
    score_bytes = parts["centroids"]
    attn_bytes = parts["estimation"] + parts["kv"] + parts["out"]

    Lmodel = cfg["L"]
    tokens_per_s = B / (Lmodel * t_step)
    result = {
        "metric": "decode tokens/s at 128K ctx (attention only, B / (L * t_layer_step)); us/layer-step and % HBM roofline alongside",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": t_step * 1e3, "us_per_layer_step": t_step * 1e6, "higher_is_better": True,
        "timed_region": {"repeats": len(reps_t), "statistic": "median", "min_us_per_layer_step": reps_t[0] * 1e6,
                         "max_us_per_layer_step": reps_t[-1] * 1e6, "layer_steps_per_region": args.steps * inner,
                         "replays_of_the_steps_per_region": inner},
        "scaling": "weak", "vs_baseline": None, "dtype": DT_NAME, "data": "synthetic",
        "config": {"workload": f"{config_name}: {cfg['desc']}; nprobe {nprobe}, estimation zone {es}, "
                               f"steady zone {static_len}, {L} layers with independent seeds (seeded Gaussian-mixture "
                               f"K/V drawn by torch's generator on the device), "
                               f"{'HIP graph replay (32 layer-steps per graph)' if graphs is not None else 'eager launches'}",
                   "batch": B, "context_tokens": cfg["N"], "layers_for_tokens_per_s": Lmodel,
                   "retrieved_tokens_per_group": t_ret / BG},
        "step_roofline": {"bound": "hbm", "algorithmic_bytes": total_bytes, "achieved": total_bytes / t_step / 1e9,
                          "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": total_bytes / t_step / HBM_PEAK},
        "stages": {
            "score_select": {"us": t_select * 1e6, "algorithmic_bytes": score_bytes,
                             "GBps": score_bytes / t_select / 1e9},
            "wave_attention": {"us": t_attn * 1e6, "algorithmic_bytes": attn_bytes,
                               "GBps": attn_bytes / t_attn / 1e9},
        },
    }
    # dominant kernel: attend_kernel, the one launch of ri_wave_attention (longest kernel, and the one that
    # moves the K/V bytes).  Its duration is taken inside the replayed step (step cycle minus the cycle
    # without it); an event pair around one eager launch also counts the dispatch of the launch
    # (eager_event_us; null_launch_us is what the same pair reads around an empty kernel).
    t_dom = t_attn_in_step if t_attn_in_step else t_attn
    traffic, traffic_source = measured_traffic(config_name)
    result["roofline"] = {"bound": "hbm", "kernel": "attend_kernel (ri_wave_attention)",
                          "achieved": attn_bytes / t_dom / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                          "frac": attn_bytes / t_dom / HBM_PEAK, "traffic": traffic, "traffic_source": traffic_source,
                          "launch_us": t_dom * 1e6, "eager_event_us": t_attn * 1e6, "null_launch_us": t_null * 1e6,
                          "algorithmic_bytes": attn_bytes,
                          "launches_timed": max(1, args.steps // CL) * CL if t_attn_in_step else n_k}
    if t_attn_in_step:
        result["stages"]["score_select"]["us_in_step"] = t_select_in_step * 1e6
        result["stages"]["wave_attention"]["us_in_step"] = t_attn_in_step * 1e6
    if est_next:
        result["next_layer_estimation"] = bench_estimate_next(args, cache, queries, outs, L, static_len)
    if extras and not args.no_read_probe:
        result["read_probe"] = read_probe(dev)
    if not args.no_cpu_baseline:
        t_cpu, n, ref = cpu_baseline(cache, cfg, queries, nprobe, es, static_len, max_seconds=10.0 if extras else 0.0,
                                     min_samples=3 if extras else 1)
        d = (outs[0].view(BG, gs, 128).cpu().float() - ref.float()).abs()
        result["cpu_baseline"] = {"value": B / (Lmodel * t_cpu), "unit": "tokens/s", "us_per_layer_step": t_cpu * 1e6,
                                  "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"median of {n} full-shape decode layer-steps of layer 0 (oracle/pipeline.py)" +
                                            (", about 10 s of CPU work" if extras else ""),
                                  "note": "the checker's restatement, not a tuned CPU implementation: float64 matrix "
                                          "products and a Python loop over the groups",
                                  "max_abs_vs_gpu": float(d.max()), "mean_abs_vs_gpu": float(d.mean())}
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=640)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--layers", type=int, default=0, help="distinct layers (default: the config's)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16"],
                    help="16-bit element type of the tensors (bf16: the benchmark's; fp16: the reference harnesses' default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of HIP graph replays")
    ap.add_argument("--residency", default="device", choices=["device", "host"],
                    help="host: clustered K/V in pinned host memory behind the block cache (staged operator path, "
                         "eager launches; reports the cold first pass and the warm steady state)")
    ap.add_argument("--block-cache", default="device", choices=["device", "host"],
                    help="with --residency host: block cache manager as a kernel (HIP graph replays) or the "
                         "reference's worker threads (eager launches)")
    ap.add_argument("--overlap", action="store_true",
                    help="with --residency host: attend the cached rows while the missed blocks are staged")
    ap.add_argument("--drift", default="0.5,0.75,1.0",
                    help="with --residency host: noise levels of the drifting-query measurements (empty: none)")
    ap.add_argument("--no-kmeans", action="store_true", help="skip the prefill clustering measurement")
    ap.add_argument("--estimate-next", action="store_true",
                    help="also measure the step with next-layer cluster estimation (zones of layer l+1 chosen "
                         "at the end of layer l from a predicted query)")
    ap.add_argument("--end-to-end", action="store_true",
                    help="a whole decoded token of a random-weight model of the config's shape (all layers, one "
                         "HIP graph per token) instead of the attention-only layer-step")
    ap.add_argument("--repeats", type=int, default=21,
                    help="repetitions of the timed region of --steps layer-steps; the median is reported")
    ap.add_argument("--no-read-probe", action="store_true",
                    help="skip the read-only streaming probe (the measured read ceiling of the part, reported as read_probe)")
    ap.add_argument("--read-probe", action="store_true", help="kept for older command lines: the probe runs by default")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="with the default configuration: skip the short runs of c1, c5 and c4 (host-resident) that are "
                         "reported as other_configs")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run 8 device copies of 256 MiB (a known-size kernel to scale rocprofv3 byte counters by)")
    args = ap.parse_args()
    global DT, DT_NAME
    if args.dtype == "fp16":
        DT, DT_NAME = torch.float16, "f16"
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the wave-index path has no cross-GPU exchange (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = CONFIGS[args.config]
    L = args.layers or cfg["L"]
    B, Hkv, gs = cfg["B"], cfg["Hkv"], cfg["gs"]
    BG = B * Hkv
    if args.copy_probe:
        a = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        b = torch.empty_like(a)
        for _ in range(8):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b
    if args.end_to_end:
        return bench_end_to_end(args, cfg, dev)
    if args.residency == "host":
        cache, queries, nprobe, es = build_cache(cfg, L, dev, "host", args.block_cache, False,
                                                 overlap_miss_staging=args.overlap)
        print(json.dumps(bench_host(args, cfg, cache, queries, L, nprobe, es, cache.static_pattern_total)))
        return
    result = bench_device(args, cfg, args.config, L, dev, extras=True)
    torch.cuda.empty_cache()      # the cache and its graphs went with the function's locals
    if not args.no_kmeans:
        km = bench_kmeans(cfg, dev)
        if not args.no_cpu_baseline:
            km["cpu_baseline"] = kmeans_cpu_baseline(cfg)
            km["cpu_baseline"]["cpu_over_gpu"] = km["cpu_baseline"]["ms_per_sequence"] / km["ms_per_sequence"]
        result["prefill_kmeans"] = km
        from retrievalattention_amd import kernels
        kernels.release_cached_graphs(retired_workspaces=False)
        torch.cuda.empty_cache()
    if args.config == "c2" and not args.no_other_configs:
        # the other named configurations, each on a short run of its own (the c2 cache is gone by now)
        import copy
        others = {}
        sub = copy.copy(args)
        sub.steps, sub.warmup, sub.repeats, sub.estimate_next = min(args.steps, 128), min(args.warmup, 32), 7, False
        sub.drift, sub.no_graph = "0.75", False
        for name, cname, Ls in (("c1", "c1", 8), ("c5", "c5", 2)):
            log(f"[bench] other config {name}")
            others[name] = compact(bench_device(sub, CONFIGS[cname], cname, Ls, dev, extras=False))
            torch.cuda.empty_cache()
        log("[bench] other config c4_host")
        c4 = CONFIGS["c4"]
        cache, queries, nprobe, es = build_cache(c4, 2, dev, "host", "device", False, overlap_miss_staging=False)
        others["c4_host"] = compact(bench_host(sub, c4, cache, queries, 2, nprobe, es, cache.static_pattern_total,
                                               config_name="c4", cpu_seconds=0.0))
        del cache, queries
        torch.cuda.empty_cache()
        result["other_configs"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
