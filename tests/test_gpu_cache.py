"""retroinfer_cache end to end on the GPU: prefill clustering, decode steps, both residencies."""
import math

import numpy as np
import pytest
import torch

from oracle import pipeline, scoring, attention
from tests.parity import check_zone_sets

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def _close(got, ref):
    d = (got.float() - ref.float()).abs()
    assert float(d.max()) <= MAX_ABS and float(d.mean()) <= MEAN_ABS, (float(d.max()), float(d.mean()))


def _make_cache(dev, residency, layers, B, Hkv, gs, ctx, n_centroids, n_segment, nprobe, es, new=8,
                cache_cluster_num=None, use_cluster_estimation=False, device_positions=False, valid_start=None,
                dt=torch.bfloat16):
    from retrievalattention_amd.cache_hub import retroinfer_cache
    # "host-cpu": host-resident store with the reference's worker-thread block cache manager;
    # "host": the same store with the device-side manager
    block_cache = "host" if residency == "host-cpu" else "device"
    overlap = residency == "host-overlap"   # device-side manager, cached rows attended beside the miss staging
    residency = "host" if overlap else residency
    if residency == "device-pos":       # device-resident store with the steady length kept on the device
        residency, device_positions = "device", True
    residency = "host" if residency == "host-cpu" else residency
    return retroinfer_cache(
        valid_start=valid_start or [0] * B, layer_num=layers, batch_size=B, max_length=ctx + new, num_key_value_heads=Hkv,
        num_heads=Hkv * gs, head_dim=128, dtype=dt, layer_mapping={str(l): "cuda:0" for l in range(layers)},
        max_new_length=new, static_pattern_start=4, static_pattern_end=64, core=4, n_centroids=n_centroids,
        n_segment=n_segment, nprobe=nprobe, max_compute_cluster_num=nprobe + es, cache_unit_size=8,
        cache_cluster_num=cache_cluster_num if cache_cluster_num is not None else 3 * nprobe, num_gpus=1,
        model_size=8, use_cluster_estimation=use_cluster_estimation, kv_residency=residency,
        block_cache=block_cache, device_positions=device_positions, overlap_miss_staging=overlap,
        # the options that change no result ride along on two of the modes
        pin_workers=block_cache == "host", profiler_ranges=overlap)


def _prefill(cache, K, V, layers, B):
    """K, V [layers][B] tensors [1, ctx, Hkv, 128] on the device."""
    for b in range(B):
        for l in range(layers):
            cache.prefill_update_kv_cache(None, K[l][b], V[l][b], l, b)
            cache.sync(l, b)
    cache.prepare_cache()


def _gen(layers, B, Hkv, gs, ctx, nmix, dev, seed, dt=torch.bfloat16):
    from retrievalattention_amd import synth
    K, V = [], []
    for l in range(layers):
        k, v, _ = synth.make_batch(seed + l, B, Hkv, ctx, nmix, gs, outliers=True, dtype=dt)
        K.append([k[b].transpose(0, 1)[None].contiguous().to(dev) for b in range(B)])
        V.append([v[b].transpose(0, 1)[None].contiguous().to(dev) for b in range(B)])
    return K, V


@pytest.mark.parametrize("residency", ["device", "host", "host-overlap", "host-cpu"])
def test_decode_matches_oracle(dev, residency, dt=torch.bfloat16):
    """Prefill + three decode steps; every compute() is compared with the oracle's decode step
    run on the index the cache actually holds."""
    layers, B, Hkv, gs, ctx = 2, 2, 2, 4, 4096 + 68
    nc, S, nprobe, es = 256, 1, 8, 60
    cache = _make_cache(dev, residency, layers, B, Hkv, gs, ctx, nc, S, nprobe, es, dt=dt)
    K, V = _gen(layers, B, Hkv, gs, ctx, 256, dev, 0, dt=dt)
    _prefill(cache, K, V, layers, B)
    assert cache.context == ctx
    BG = B * Hkv
    g = torch.Generator().manual_seed(9)
    # the oracle needs the cluster-contiguous store: rebuild it on the CPU from the cache's assignment
    stores = []
    for l in range(layers):
        sk, sv, st = [], [], []
        for b in range(B):
            for h in range(Hkv):
                # use the sizes the cache reports; order inside a cluster = ascending token id
                size = cache.cluster_size[l][b * Hkv + h].cpu().float().to(torch.int64)
                if residency == "device":
                    gi = b * Hkv + h
                    rows = int(cache.store_rows[l][gi])
                    sk.append(cache.list_keys[l].view(BG, -1, 128)[gi, :rows].cpu())
                    sv.append(cache.list_values[l].view(BG, -1, 128)[gi, :rows].cpu())
                else:
                    gi = b * Hkv + h
                    rows = int(size.sum())
                    sk.append(cache.list_keys[l].view(BG, -1, 128)[gi, :rows].clone())
                    sv.append(cache.list_values[l].view(BG, -1, 128)[gi, :rows].clone())
                st.append(torch.cumsum(size, 0) - size)
        stores.append((sk, sv, torch.stack(st)))
    for step in range(3):
        for l in range(layers):
            k_new = torch.randn(B, 1, Hkv, 128, generator=g).to(dt)
            v_new = torch.randn(B, 1, Hkv, 128, generator=g).to(dt)
            q = torch.randn(B, 1, Hkv * gs, 128, generator=g).to(dt)
            cache.decode_update_kv_cache(k_new.to(dev), v_new.to(dev), l)
            out = cache.compute(q.to(dev), l)
            torch.cuda.synchronize()
            static_len = cache.static_pattern_total if l == layers - 1 else cache.static_pattern_total + 1
            if l == layers - 1:
                static_len = cache.static_pattern_total  # already advanced by decode_update_kv_cache
            size_bf = cache.cluster_size[l].cpu()
            size_i = size_bf.float().to(torch.int32)
            ref, aux = pipeline.decode_step(
                q.view(BG, gs, 128), cache.steady_zone_keys[l].view(BG, -1, 128).cpu(),
                cache.steady_zone_values[l].view(BG, -1, 128).cpu(), static_len, cache.centroids[l].cpu(),
                cache.value_sum[l].cpu(), cache.centroids_mask[l].cpu(), size_i, size_bf, stores[l][0], stores[l][1],
                stores[l][2], nprobe, es, 8, cache.buffer_size, logits=cache.logits.cpu())
            _close(out.cpu().view(BG, gs, 128), ref)
            buf = l % 2
            assert torch.equal(cache.cI[buf][:, :nprobe].cpu(), aux["ret"])
            assert torch.equal(cache.cI[buf][:, nprobe:].cpu(), aux["est"])
            assert torch.equal(cache.valid_lengths[buf].cpu().long(), static_len + aux["offs"][:, -1])
    assert cache.context == ctx + 3 and out.dtype == dt


@pytest.mark.parametrize("residency", ["device", "host", "host-overlap", "host-cpu"])
def test_decode_matches_oracle_float16(dev, residency):
    """The same with IEEE half elements, the default of the reference's harnesses (simple_test.py:29,
    throughput_eval/test.py:28): index, stores, scores, probabilities and outputs all in fp16."""
    test_decode_matches_oracle(dev, residency, dt=torch.float16)


def test_full_retrieval_equals_dense_attention(dev):
    """Property (v): probing every cluster with no estimation zone is dense attention over
    steady zone + all clustered tokens, whatever the partition."""
    layers, B, Hkv, gs, ctx = 1, 1, 2, 4, 2048 + 68
    nc = 128
    cache = _make_cache(dev, "device", layers, B, Hkv, gs, ctx, nc, 1, nc, 0)
    cache.buffer_size = 10 ** 6 // 8   # no page cut-off
    cache.allocate_computation_buffer()
    K, V = _gen(layers, B, Hkv, gs, ctx, 100, dev, 3)
    _prefill(cache, K, V, layers, B)
    g = torch.Generator().manual_seed(1)
    q = torch.randn(B, 1, Hkv * gs, 128, generator=g).to(torch.bfloat16)
    kn = torch.randn(B, 1, Hkv, 128, generator=g).to(torch.bfloat16)
    vn = torch.randn(B, 1, Hkv, 128, generator=g).to(torch.bfloat16)
    cache.decode_update_kv_cache(kn.to(dev), vn.to(dev), 0)
    out = cache.compute(q.to(dev), 0).cpu()
    kk = torch.cat([K[0][0][0].cpu(), kn[0]], 0).transpose(0, 1)   # [Hkv, ctx+1, D]
    vv = torch.cat([V[0][0][0].cpu(), vn[0]], 0).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.view(Hkv, gs, 128).float(), kk.float(), vv.float())
    _close(out.view(Hkv, gs, 128), ref)


@pytest.mark.parametrize("host_kind", ["host", "host-overlap", "host-cpu"])
def test_host_and_device_residency_agree_and_cache_warms(dev, host_kind):
    """Same inputs through both residencies: identical selections, outputs within tolerance;
    repeated queries turn misses into hits in the LRU block cache."""
    layers, B, Hkv, gs, ctx = 1, 2, 2, 7, 3072 + 68
    nc, nprobe, es = 192, 6, 40
    K, V = _gen(layers, B, Hkv, gs, ctx, 192, dev, 5)
    cd = _make_cache(dev, "device", layers, B, Hkv, gs, ctx, nc, 1, nprobe, es)
    ch = _make_cache(dev, host_kind, layers, B, Hkv, gs, ctx, nc, 1, nprobe, es)
    _prefill(cd, K, V, layers, B)
    _prefill(ch, K, V, layers, B)
    assert torch.equal(cd.centroids[0], ch.centroids[0])
    g = torch.Generator().manual_seed(2)
    q = torch.randn(B, 1, Hkv * gs, 128, generator=g).to(torch.bfloat16).to(dev)
    kn = torch.randn(B, 1, Hkv, 128, generator=g).to(torch.bfloat16).to(dev)
    vn = torch.randn(B, 1, Hkv, 128, generator=g).to(torch.bfloat16).to(dev)
    hits = []
    for step in range(3):
        for c in (cd, ch):
            c.decode_update_kv_cache(kn, vn, 0)
        od, oh = cd.compute(q, 0), ch.compute(q, 0)
        torch.cuda.synchronize()
        _close(oh.cpu(), od.cpu())
        assert torch.equal(cd.cI[0].cpu(), ch.cI[0].cpu())
        assert torch.equal(cd.valid_lengths[0].cpu(), ch.valid_lengths[0].cpu())
        hits.append(ch.block_cache_stats(0)[0])
    assert hits[0] == 0 and hits[1] > 0 and hits[2] >= hits[1]
    if host_kind in ("host", "host-overlap"):
        # device-side manager: what sits in the block cache is what the store holds for those clusters
        lru, BG = ch.device_lru[0], B * Hkv
        size = ch.cluster_size_i32[0].cpu()
        start = ch.cluster_start[0].cpu()
        stamp, boff, bids = lru.stamp.cpu(), lru.blk_off.cpu(), lru.blk_ids.cpu()
        ck = ch.cache_keys[0].view(BG, -1, 8, 128).cpu()
        cv = ch.cache_values[0].view(BG, -1, 8, 128).cpu()
        lk, lv = ch.list_keys[0].view(BG, -1, 128), ch.list_values[0].view(BG, -1, 128)
        checked = 0
        for gi in range(BG):
            used = []
            for c in torch.nonzero(stamp[gi, :nc]).flatten().tolist():
                n = int(size[gi, c])
                ids = bids[gi, int(boff[gi, c]):int(boff[gi, c + 1])].tolist()
                used += ids
                got_k = ck[gi, ids].reshape(-1, 128)[:n]
                got_v = cv[gi, ids].reshape(-1, 128)[:n]
                r0 = int(start[gi, c])
                assert torch.equal(got_k, lk[gi, r0:r0 + n]) and torch.equal(got_v, lv[gi, r0:r0 + n])
                checked += 1
            free = lru.free_list[gi, :int(lru.free_count[gi])].tolist()
            assert len(set(used)) == len(used) and not set(used) & set(free)
            assert len(used) + len(free) == ch.cache_size
        assert checked > 0


@pytest.mark.parametrize("host_kind", ["host", "host-overlap", "host-cpu"])
def test_no_block_cache(dev, host_kind):
    """cache_cluster_num = 0, as the reference's throughput harness sets it (throughput_eval/test.py:77: no GPU
    block cache): every retrieved cluster is read from the host store at every step and nothing is admitted
    (wave_buffer_cpu.cpp:119-130 with a capacity of 0); selections equal those of the device-resident cache and
    outputs agree within tolerance, step after step."""
    layers, B, Hkv, gs, ctx = 1, 2, 2, 4, 3072 + 68
    nc, nprobe, es = 192, 6, 40
    K, V = _gen(layers, B, Hkv, gs, ctx, 192, dev, 6)
    cd = _make_cache(dev, "device", layers, B, Hkv, gs, ctx, nc, 1, nprobe, es)
    ch = _make_cache(dev, host_kind, layers, B, Hkv, gs, ctx, nc, 1, nprobe, es, cache_cluster_num=0)
    assert ch.cache_size == 0
    _prefill(cd, K, V, layers, B)
    _prefill(ch, K, V, layers, B)
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, 1, Hkv * gs, 128, generator=g).to(torch.bfloat16).to(dev)
    kn = torch.randn(B, 1, Hkv, 128, generator=g).to(torch.bfloat16).to(dev)
    vn = torch.randn(B, 1, Hkv, 128, generator=g).to(torch.bfloat16).to(dev)
    for step in range(3):
        for c in (cd, ch):
            c.decode_update_kv_cache(kn, vn, 0)
        od, oh = cd.compute(q, 0), ch.compute(q, 0)
        torch.cuda.synchronize()
        _close(oh.cpu(), od.cpu())
        assert torch.equal(cd.cI[0].cpu(), ch.cI[0].cpu())
        assert torch.equal(cd.valid_lengths[0].cpu(), ch.valid_lengths[0].cpu())
        hit, miss = ch.block_cache_stats(0)
        assert hit == 0 and miss > 0
        assert int(ch.update_num_units[0].sum()) == 0


def test_limits_are_checked_at_construction(dev):
    """The kernels' limits surface when the cache is built, with a message that names the limit."""
    with pytest.raises(ValueError, match="nprobe must be in 1..4096"):
        _make_cache(dev, "device", 1, 1, 1, 4, 70000 + 68, 65536, 1, 5000, 100)
    with pytest.raises(ValueError, match="at most 65536"):
        _make_cache(dev, "device", 1, 1, 1, 4, 70000 + 68, 65544, 1, 8, 100)
    with pytest.raises(ValueError, match="at most 16 query heads"):
        _make_cache(dev, "device", 1, 1, 1, 32, 4096 + 68, 256, 1, 8, 60)
    with pytest.raises(ValueError, match="must not be negative"):
        _make_cache(dev, "host", 1, 1, 1, 4, 4096 + 68, 256, 1, 8, 60, cache_cluster_num=-1)
    with pytest.raises(ValueError, match="at most 4096 groups"):
        _make_cache(dev, "device", 1, 1025, 4, 1, 4096 + 68, 256, 1, 8, 60)


def test_residencies_agree_random_shapes(dev):
    """The four ways to hold the clustered K/V (device store; host store with the device-side block cache, with and
    without the cached rows attended beside the miss staging; host store with the worker-thread block cache) on 16
    shapes drawn from a fixed seed: 1-2 layers, batch 1-3, 1-4 kv heads, group sizes 1-8, 1-4 k-means segments,
    block caches from exactly one probe list (every step evicts) to ten, repeated and fresh queries.  Selections
    and valid lengths identical, outputs within tolerance of the device store's."""
    import random
    rnd = random.Random(4711)
    kinds = ["device", "host", "host-overlap", "host-cpu"]
    for it in range(16):
        layers, B, Hkv, gs = rnd.choice([1, 2]), rnd.choice([1, 2, 3]), rnd.choice([1, 2, 4]), rnd.choice([1, 2, 4, 7, 8])
        S = rnd.choice([1, 1, 2, 4])
        nc = 32 * S * rnd.randint(1, 6)
        ctx = 68 + S * rnd.randint(max(nc // S, 64), 1200)
        nprobe = rnd.randint(1, max(1, nc // 6))
        es = rnd.choice([0, rnd.randint(0, nc - nprobe)])
        ccn = rnd.choice([nprobe, nprobe + 1, 2 * nprobe, 3 * nprobe, 10 * nprobe])
        label = (layers, B, Hkv, gs, ctx, nc, S, nprobe, es, ccn)
        K, V = _gen(layers, B, Hkv, gs, ctx, max(nc // 2, 8), dev, 40 + it)
        caches = [_make_cache(dev, k, layers, B, Hkv, gs, ctx, nc, S, nprobe, es, cache_cluster_num=ccn) for k in kinds]
        for c in caches:
            _prefill(c, K, V, layers, B)
        g = torch.Generator().manual_seed(it)
        draw = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16).to(dev)
        qs = [draw(B, 1, Hkv * gs, 128) for _ in range(3)]
        for step in range(rnd.randint(2, 6)):
            for l in range(layers):
                q = qs[rnd.randrange(3)] if rnd.random() < 0.6 else draw(B, 1, Hkv * gs, 128)
                kn, vn = draw(B, 1, Hkv, 128), draw(B, 1, Hkv, 128)
                outs = []
                for c in caches:
                    c.decode_update_kv_cache(kn, vn, l)
                    outs.append(c.compute(q, l).clone())
                torch.cuda.synchronize()
                for k, c, o in zip(kinds[1:], caches[1:], outs[1:]):
                    assert bool(torch.isfinite(o.float()).all()), (label, k, step, l)
                    _close(o.cpu(), outs[0].cpu())
                    assert torch.equal(caches[0].cI[l % 2].cpu(), c.cI[l % 2].cpu()), (label, k, step, l)
                    assert torch.equal(caches[0].valid_lengths[l % 2].cpu(), c.valid_lengths[l % 2].cpu()), (label, k, step, l)
        del caches


def test_residencies_agree_with_cluster_estimation_random_shapes(dev):
    """use_cluster_estimation through the four residencies on 12 shapes drawn from a fixed seed (3-5 layers, 1-3
    tokens, short contexts, so that the one new token of a layer carries weight): zones from a predicted query
    from the third layer on.  Selections and valid lengths identical, outputs within tolerance of the device
    store's.  (The worker-thread mode assembles a layer's buffer during the previous layer, before the layer's
    new token exists; the token's row is brought in before the attention.)"""
    import random
    rnd = random.Random(77)
    kinds = ["device", "host", "host-overlap", "host-cpu"]
    for it in range(12):
        layers, B, Hkv, gs = rnd.choice([3, 4, 5]), rnd.choice([1, 2, 3]), rnd.choice([1, 2, 4]), rnd.choice([1, 2, 4, 7, 8])
        S = rnd.choice([1, 1, 2, 4])
        nc = 32 * S * rnd.randint(1, 6)
        ctx = 68 + S * rnd.randint(max(nc // S, 64), 1200)
        nprobe = rnd.randint(1, max(1, nc // 6))
        es = rnd.choice([0, rnd.randint(0, nc - nprobe)])
        ccn = rnd.choice([nprobe, 2 * nprobe, 3 * nprobe, 10 * nprobe])
        tokens = rnd.randint(1, 3)
        label = (layers, B, Hkv, gs, ctx, nc, S, nprobe, es, ccn, tokens)
        K, V = _gen(layers, B, Hkv, gs, ctx, max(nc // 2, 8), dev, 140 + it)
        caches = [_make_cache(dev, k, layers, B, Hkv, gs, ctx, nc, S, nprobe, es, cache_cluster_num=ccn,
                              use_cluster_estimation=True) for k in kinds]
        for c in caches:
            _prefill(c, K, V, layers, B)
        g = torch.Generator().manual_seed(it)
        draw = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16).to(dev)
        for tok in range(tokens):
            qs = [draw(B, 1, Hkv * gs, 128) for _ in range(layers)]
            qp = [(q.float() + 0.5 * torch.randn(q.shape, generator=g).to(dev)).to(torch.bfloat16) for q in qs]
            for l in range(layers):
                kn, vn = draw(B, 1, Hkv, 128), draw(B, 1, Hkv, 128)
                outs = []
                for c in caches:
                    c.decode_update_kv_cache(kn, vn, l)
                    outs.append(c.compute(qs[l], l, qp[l + 1] if l + 1 < layers else None).clone())
                torch.cuda.synchronize()
                for k, c, o in zip(kinds[1:], caches[1:], outs[1:]):
                    assert bool(torch.isfinite(o.float()).all()), (label, k, tok, l)
                    _close(o.cpu(), outs[0].cpu())
                    assert torch.equal(caches[0].cI[l % 2].cpu(), c.cI[l % 2].cpu()), (label, k, tok, l)
                    assert torch.equal(caches[0].valid_lengths[l % 2].cpu(), c.valid_lengths[l % 2].cpu()), (label, k, tok, l)
        del caches


@pytest.mark.parametrize("residency", ["device", "host", "host-overlap", "host-cpu"])
def test_next_layer_cluster_estimation(dev, residency, dt=torch.bfloat16):
    """use_cluster_estimation (reference: retroinfer_cache.py:565, 582-595): layers 0 and 1 choose their
    zones from their own query; every later layer uses the zones the previous layer chose from a
    predicted query, scores its estimation zone with the true query and attends the retrieval zone
    exactly.  Checked against the oracle with the same split between zone query and true query."""
    layers, B, Hkv, gs, ctx = 4, 2, 2, 4, 4096 + 68
    nc, nprobe, es = 256, 8, 60
    cache = _make_cache(dev, residency, layers, B, Hkv, gs, ctx, nc, 1, nprobe, es, use_cluster_estimation=True, dt=dt)
    K, V = _gen(layers, B, Hkv, gs, ctx, 256, dev, 11, dt=dt)
    _prefill(cache, K, V, layers, B)
    BG = B * Hkv
    g = torch.Generator().manual_seed(12)
    q_true = [torch.randn(B, 1, Hkv * gs, 128, generator=g).to(dt) for _ in range(layers)]
    # the prediction for layer l (made at layer l-1) is off by a fair amount: zones differ from the true ones
    q_pred = [(q.float() + 0.5 * torch.randn(q.shape, generator=g)).to(dt) for q in q_true]
    differs = 0
    for l in range(layers):
        kn = torch.randn(B, 1, Hkv, 128, generator=g).to(dt)
        vn = torch.randn(B, 1, Hkv, 128, generator=g).to(dt)
        cache.decode_update_kv_cache(kn.to(dev), vn.to(dev), l)
        nxt = q_pred[l + 1].to(dev) if l + 1 < layers else None
        out = cache.compute(q_true[l].to(dev), l, nxt)
        torch.cuda.synchronize()
        static_len = cache.static_pattern_total if l == layers - 1 else cache.static_pattern_total + 1
        if l == layers - 1:
            static_len = cache.static_pattern_total
        size_bf = cache.cluster_size[l].cpu()
        size_i = size_bf.float().to(torch.int32)
        rows = size_i.sum(1)
        lk, lv = cache.list_keys[l].view(BG, -1, 128), cache.list_values[l].view(BG, -1, 128)
        sk = [lk[gi, :int(rows[gi])].cpu() for gi in range(BG)]
        sv = [lv[gi, :int(rows[gi])].cpu() for gi in range(BG)]
        start = torch.cumsum(size_i.long(), 1) - size_i.long()
        zone = None
        if l >= 2:   # zones were chosen at layer l-1 from the predicted query
            zone = scoring.logits_fp32(q_pred[l].view(BG, gs, 128), cache.centroids[l].cpu(), 1.0 / math.sqrt(128))
        ref, aux = pipeline.decode_step(
            q_true[l].view(BG, gs, 128), cache.steady_zone_keys[l].view(BG, -1, 128).cpu(),
            cache.steady_zone_values[l].view(BG, -1, 128).cpu(), static_len, cache.centroids[l].cpu(),
            cache.value_sum[l].cpu(), cache.centroids_mask[l].cpu(), size_i, size_bf, sk, sv, start, nprobe, es, 8,
            cache.buffer_size, zone_logits=zone)
        _close(out.cpu().view(BG, gs, 128), ref)
        buf = l % 2
        cI = cache.cI[buf].cpu()
        check_zone_sets(aux["dist"], cI[:, :nprobe], cI[:, nprobe:], aux["ret"], aux["est"], nprobe, es, band=1.0)
        if l >= 2:   # the predicted zones are not the true query's zones (otherwise the test shows nothing)
            _, aux_true = pipeline.decode_step(
                q_true[l].view(BG, gs, 128), cache.steady_zone_keys[l].view(BG, -1, 128).cpu(),
                cache.steady_zone_values[l].view(BG, -1, 128).cpu(), static_len, cache.centroids[l].cpu(),
                cache.value_sum[l].cpu(), cache.centroids_mask[l].cpu(), size_i, size_bf, sk, sv, start, nprobe, es, 8,
                cache.buffer_size)
            differs += int((aux_true["ret"] != aux["ret"]).any())
    assert differs > 0


@pytest.mark.parametrize("residency", ["device", "host", "host-cpu"])
def test_next_layer_cluster_estimation_float16(dev, residency):
    test_next_layer_cluster_estimation(dev, residency, dt=torch.float16)


def test_reference_stale_row_switch(dev):
    """reference_stale_row=True (worker-thread manager with next-layer estimation) reproduces the reference's
    arithmetic: from the third layer on the execution buffer was assembled during the previous layer, before the
    layer's new token was appended (retroinfer_cache.py:644-652 against :541-542), so the attention reads the
    row as it was then (zeros for the first generated token) instead of the token's K/V.  Checked against the
    oracle fed that stale row; without the switch the same layers match the oracle fed the real row."""
    from retrievalattention_amd.cache_hub import retroinfer_cache
    layers, B, Hkv, gs, ctx = 4, 1, 2, 4, 2048 + 68
    nc, nprobe, es = 128, 6, 30
    K, V = _gen(layers, B, Hkv, gs, ctx, 128, dev, 21)
    BG = B * Hkv
    outs = {}
    for stale in (False, True):
        cache = retroinfer_cache(
            valid_start=[0] * B, layer_num=layers, batch_size=B, max_length=ctx + 8, num_key_value_heads=Hkv,
            num_heads=Hkv * gs, head_dim=128, dtype=torch.bfloat16, layer_mapping={str(l): "cuda:0" for l in range(layers)},
            max_new_length=8, static_pattern_start=4, static_pattern_end=64, core=4, n_centroids=nc, n_segment=1,
            nprobe=nprobe, max_compute_cluster_num=nprobe + es, cache_unit_size=8, cache_cluster_num=3 * nprobe,
            num_gpus=1, model_size=8, use_cluster_estimation=True, kv_residency="host", block_cache="host",
            reference_stale_row=stale)
        _prefill(cache, K, V, layers, B)
        g = torch.Generator().manual_seed(22)
        q = [torch.randn(B, 1, Hkv * gs, 128, generator=g).to(torch.bfloat16) for _ in range(layers)]
        for l in range(layers):
            kn = (4 * torch.randn(B, 1, Hkv, 128, generator=g)).to(torch.bfloat16)   # a key that matters
            vn = (4 * torch.randn(B, 1, Hkv, 128, generator=g)).to(torch.bfloat16)
            cache.decode_update_kv_cache(kn.to(dev), vn.to(dev), l)
            out = cache.compute(q[l].to(dev), l, q[l + 1].to(dev) if l + 1 < layers else None)
            torch.cuda.synchronize()
            static_len = cache.static_pattern_total if l == layers - 1 else cache.static_pattern_total + 1
            size_bf = cache.cluster_size[l].cpu()
            size_i = size_bf.float().to(torch.int32)
            rows = size_i.sum(1)
            lk, lv = cache.list_keys[l].view(BG, -1, 128), cache.list_values[l].view(BG, -1, 128)
            sk = [lk[gi, :int(rows[gi])].clone() for gi in range(BG)]
            sv = [lv[gi, :int(rows[gi])].clone() for gi in range(BG)]
            stk = cache.steady_zone_keys[l].view(BG, -1, 128).cpu().clone()
            stv = cache.steady_zone_values[l].view(BG, -1, 128).cpu().clone()
            if stale and l >= 2:
                stk[:, static_len - 1] = 0
                stv[:, static_len - 1] = 0
            ref, _ = pipeline.decode_step(
                q[l].view(BG, gs, 128), stk, stv, static_len, cache.centroids[l].cpu(), cache.value_sum[l].cpu(),
                cache.centroids_mask[l].cpu(), size_i, size_bf, sk, sv, torch.cumsum(size_i.long(), 1) - size_i.long(),
                nprobe, es, 8, cache.buffer_size)
            _close(out.cpu().view(BG, gs, 128), ref)
            outs[(stale, l)] = out.cpu().float()
        del cache
    # the switch changes something from the third layer on, and nothing before
    assert torch.equal(outs[(False, 0)], outs[(True, 0)]) and torch.equal(outs[(False, 1)], outs[(True, 1)])
    assert float((outs[(False, 2)] - outs[(True, 2)]).abs().max()) > 1e-2


@pytest.mark.parametrize("residency", ["device", "host", "host-cpu", "device-pos"])
def test_index_growth_after_1024_generated_tokens(dev, residency, dt=torch.bfloat16):
    """Decode-time index update (reference: retroinfer_cache.py:462-546): once the steady zone holds
    1024 tokens beyond its 4 + 64, they are clustered into 64 new centroids and appended to the index
    and the store; the last 64 stay as the local window.  Checked: the appended store rows are exactly
    the folded tokens, and decoding afterwards matches the oracle on the grown index."""
    layers, B, Hkv, gs, ctx = 1, 2, 2, 4, 2048 + 68
    nc, nprobe, es, new = 128, 8, 40, 1100
    # the first sequence is left-padded: it holds fewer clustered tokens than the second, so the groups
    # append their folded tokens at different store rows (reference: wave_buffer_cpu.cpp:658)
    vstart = [64, 0]
    cache = _make_cache(dev, residency, layers, B, Hkv, gs, ctx, nc, 1, nprobe, es, new=new, valid_start=vstart, dt=dt)
    K, V = _gen(layers, B, Hkv, gs, ctx, 128, dev, 21, dt=dt)
    _prefill(cache, K, V, layers, B)
    BG = B * Hkv
    Ng = [ctx - 68 - vstart[gi // Hkv] for gi in range(BG)]     # clustered prompt tokens per group
    g = torch.Generator().manual_seed(22)
    gk = torch.randn(B, 1030, Hkv, 128, generator=g).to(dt)
    gv = torch.randn(B, 1030, Hkv, 128, generator=g).to(dt)
    q = torch.randn(B, 1, Hkv * gs, 128, generator=g).to(dt).to(dev)
    lk, lv = cache.list_keys[0].view(BG, -1, 128), cache.list_values[0].view(BG, -1, 128)
    before_k = [lk[gi, :Ng[gi]].cpu().clone() for gi in range(BG)]
    before_v = [lv[gi, :Ng[gi]].cpu().clone() for gi in range(BG)]
    for t in range(1030):
        cache.decode_update_kv_cache(gk[:, t:t + 1].to(dev), gv[:, t:t + 1].to(dev), 0)
        # keep the block cache busy before the index grows; with the steady length on the device
        # every token's attention runs (it is what moves the device-side position on)
        if t in (0, 700) or residency == "device-pos":
            cache.compute(q, 0)
    torch.cuda.synchronize()
    if residency == "device-pos":
        assert int(cache.steady_len_dev) == cache.static_pattern_total + 1
        assert int(cache.steady_pos_dev) == cache.static_pattern_total
    assert cache.n_centroids == nc + 64 and cache.centroids[0].shape[1] == nc + 64
    assert cache.static_pattern_total == 4 + 64 + (1030 - 1024)   # the fold happened on the 1025th call
    lk, lv = cache.list_keys[0].view(BG, -1, 128), cache.list_values[0].view(BG, -1, 128)
    size_i = cache.cluster_size_i32[0].cpu()
    start_new = cache.cluster_start[0].cpu()[:, nc:]
    for b in range(B):
        for h in range(Hkv):
            gi = b * Hkv + h
            N = Ng[gi]
            folded_k = torch.cat([K[0][b][0, ctx - 64:, h].cpu(), gk[b, :960, h]])      # prompt tail + first 960 generated
            folded_v = torch.cat([V[0][b][0, ctx - 64:, h].cpu(), gv[b, :960, h]])
            # the prompt's clusters were not touched, the folded tokens sit right behind them
            assert torch.equal(lk[gi, :N].cpu(), before_k[gi]) and torch.equal(lv[gi, :N].cpu(), before_v[gi])
            got_k, got_v = lk[gi, N:N + 1024].cpu(), lv[gi, N:N + 1024].cpu()
            # cluster by cluster: rows [start, start + size) hold tokens of the folded set in ascending
            # token order, and every folded token sits in exactly one cluster
            fk = {bytes(r.view(torch.int16).numpy().tobytes()): i for i, r in enumerate(folded_k)}
            seen = []
            for c in range(64):
                s0, n = int(start_new[gi, c]) - N, int(size_i[gi, nc + c])
                ids = [fk[bytes(r.view(torch.int16).numpy().tobytes())] for r in got_k[s0:s0 + n]]
                assert ids == sorted(ids), "tokens inside a cluster must be ascending"
                assert torch.equal(got_v[s0:s0 + n], folded_v[ids])
                seen += ids
            assert sorted(seen) == list(range(1024))
    assert bool((size_i[:, nc:].sum(1) == 1024).all())
    assert size_i.sum(1).tolist() == [n + 1024 for n in Ng]
    out = cache.compute(q, 0)
    torch.cuda.synchronize()
    sk = [lk[gi, :Ng[gi] + 1024].cpu() for gi in range(BG)]
    sv = [lv[gi, :Ng[gi] + 1024].cpu() for gi in range(BG)]
    start = torch.cumsum(size_i.long(), 1) - size_i.long()
    assert torch.equal(start.int(), cache.cluster_start[0].cpu())
    static_len = cache.static_pattern_total
    ref, aux = pipeline.decode_step(
        q.cpu().view(BG, gs, 128), cache.steady_zone_keys[0].view(BG, -1, 128).cpu(),
        cache.steady_zone_values[0].view(BG, -1, 128).cpu(), static_len, cache.centroids[0].cpu(),
        cache.value_sum[0].cpu(), cache.centroids_mask[0].cpu(), size_i, cache.cluster_size[0].cpu(), sk, sv, start,
        nprobe, es, 8, cache.buffer_size)
    _close(out.cpu().view(BG, gs, 128), ref)
    cI = cache.cI[0].cpu()
    check_zone_sets(aux["dist"], cI[:, :nprobe], cI[:, nprobe:], aux["ret"], aux["est"], nprobe, es, band=1.0)


@pytest.mark.parametrize("residency", ["device", "host"])
def test_index_growth_after_1024_generated_tokens_float16(dev, residency):
    test_index_growth_after_1024_generated_tokens(dev, residency, dt=torch.float16)


def test_captured_steps_replay_token_after_token(dev):
    """device_positions: the steady zone's length lives on the device, so one captured decode step per
    layer (append the token's K/V, attend) is replayed for token after token while the zone grows.
    Every replayed token must match a twin cache that is stepped eagerly with the reference's calls."""
    layers, B, Hkv, gs, ctx = 2, 2, 2, 4, 2048 + 68
    nc, nprobe, es, tokens = 128, 8, 40, 6
    K, V = _gen(layers, B, Hkv, gs, ctx, 128, dev, 31)
    eager = _make_cache(dev, "device", layers, B, Hkv, gs, ctx, nc, 1, nprobe, es, new=64)
    replay = _make_cache(dev, "device", layers, B, Hkv, gs, ctx, nc, 1, nprobe, es, new=64, device_positions=True)
    _prefill(eager, K, V, layers, B)
    _prefill(replay, K, V, layers, B)
    g = torch.Generator().manual_seed(32)
    draw = lambda: ([torch.randn(B, 1, Hkv * gs, 128, generator=g).to(torch.bfloat16).to(dev) for _ in range(layers)],
                    [torch.randn(B, 1, Hkv, 128, generator=g).to(torch.bfloat16).to(dev) for _ in range(layers)],
                    [torch.randn(B, 1, Hkv, 128, generator=g).to(torch.bfloat16).to(dev) for _ in range(layers)])
    q_in = [torch.empty(B, 1, Hkv * gs, 128, dtype=torch.bfloat16, device=dev) for _ in range(layers)]
    k_in = [torch.empty(B, 1, Hkv, 128, dtype=torch.bfloat16, device=dev) for _ in range(layers)]
    v_in = [torch.empty(B, 1, Hkv, 128, dtype=torch.bfloat16, device=dev) for _ in range(layers)]

    def step(cache, l, q, k, v):
        cache.decode_update_kv_cache(k, v, l)
        return cache.compute(q, l)

    def load(qs, ks, vs):
        for l in range(layers):
            q_in[l].copy_(qs[l]); k_in[l].copy_(ks[l]); v_in[l].copy_(vs[l])

    # first token eagerly on both (also the warm-up that capture needs), on a side stream
    qs, ks, vs = draw()
    load(qs, ks, vs)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        first = [step(replay, l, q_in[l], k_in[l], v_in[l]) for l in range(layers)]
    torch.cuda.current_stream().wait_stream(side)
    ref = [step(eager, l, qs[l], ks[l], vs[l]) for l in range(layers)]
    torch.cuda.synchronize()
    for l in range(layers):
        assert torch.equal(first[l], ref[l])
    assert replay.static_pattern_total == eager.static_pattern_total == 69
    # capture one step per layer
    graphs = []
    for l in range(layers):
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            o = step(replay, l, q_in[l], k_in[l], v_in[l])
        graphs.append((gr, o))
    assert replay.static_pattern_total == 69          # capturing moved nothing on the host
    for t in range(tokens):
        qs, ks, vs = draw()
        load(qs, ks, vs)
        assert not replay.fold_due()
        for l in range(layers):
            graphs[l][0].replay()
        replay.token_replayed()
        ref = [step(eager, l, qs[l], ks[l], vs[l]) for l in range(layers)]
        torch.cuda.synchronize()
        for l in range(layers):
            d = (graphs[l][1].float() - ref[l].float()).abs()
            assert float(d.max()) <= 2e-3, (t, l, float(d.max()))
        assert replay.static_pattern_total == eager.static_pattern_total == 70 + t
        assert int(replay.steady_len_dev) == replay.static_pattern_total + 1
        for l in range(layers):   # the replays appended the same rows as the eager calls
            n = eager.static_pattern_total
            assert torch.equal(replay.steady_zone_keys[l][:, :, :n], eager.steady_zone_keys[l][:, :, :n])
    assert int(replay.valid_lengths[(layers - 1) % 2].min()) > 69 + tokens - 1   # the grown zone was attended
