"""Full-size cases: the benchmark shapes end to end on the GPU.

At these sizes the CPU oracle is still affordable for one decode layer-step (tens to hundreds
of milliseconds), so outputs and selections are compared with it directly; on top of that the
tests use properties that hold at any size: exact linearity in the values (scaling every value
by two, exact in bf16, must double the output bit for bit and leave the selections alone),
partition invariants of the clustering, and run-to-run reproducibility.
"""
import numpy as np
import pytest
import torch

from oracle import pipeline
from tests.parity import check_zone_sets

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_ABS = 2e-2, 2e-3

SHAPES = {
    # batch, kv heads, group size, clustered tokens, centroids, segments, outlier channels, seed, residency
    "c1": dict(B=1, Hkv=8, gs=4, N=8192, nc=512, S=1, outliers=False, seed=0, residency="device"),
    "c2": dict(B=4, Hkv=8, gs=4, N=131072, nc=8192, S=16, outliers=True, seed=0, residency="device"),
    "c4": dict(B=16, Hkv=4, gs=7, N=61440, nc=3840, S=8, outliers=False, seed=1, residency="host"),
    "c5": dict(B=8, Hkv=8, gs=8, N=262144, nc=16384, S=32, outliers=True, seed=0, residency="device"),
}


def _build(dev, cfg, dt=torch.bfloat16):
    """One layer of the cache at a benchmark shape, K/V from the seeded generator on the device."""
    from retrievalattention_amd import synth
    from retrievalattention_amd.cache_hub import retroinfer_cache
    B, Hkv, gs, N, nc = cfg["B"], cfg["Hkv"], cfg["gs"], cfg["N"], cfg["nc"]
    nprobe, es = max(1, int(nc * 0.018)), int(nc * 0.232)
    ctx = N + synth.STEADY_START + synth.STEADY_END
    cache = retroinfer_cache(
        valid_start=[0] * B, layer_num=1, batch_size=B, max_length=ctx + 4, num_key_value_heads=Hkv,
        num_heads=Hkv * gs, head_dim=128, dtype=dt, layer_mapping={"0": "cuda:0"}, max_new_length=4,
        static_pattern_start=synth.STEADY_START, static_pattern_end=synth.STEADY_END, core=8, n_centroids=nc,
        n_segment=cfg["S"], nprobe=nprobe, max_compute_cluster_num=nprobe + es, cache_unit_size=8,
        cache_cluster_num=max(int(nc * 0.05), nprobe), num_gpus=1, model_size=0, kv_residency=cfg["residency"])
    qs = []
    for b in range(B):
        ks, vs = [], []
        for h in range(Hkv):
            k, v, q = synth.make_group(cfg["seed"], b, h, N, nc, gs, outliers=cfg["outliers"],
                                       n_extra=synth.STEADY_START + synth.STEADY_END, device=dev)
            ks.append(torch.cat([k[N:N + 4], k[:N], k[N + 4:]]).to(dt))
            vs.append(torch.cat([v[N:N + 4], v[:N], v[N + 4:]]).to(dt))
            qs.append(q.to(dt))
        K = torch.stack(ks, 1)[None].contiguous()
        V = torch.stack(vs, 1)[None].contiguous()
        cache.prefill_update_kv_cache(None, K, V, 0, b)
        cache.sync(0, b)
        del K, V, ks, vs
    cache.prepare_cache()
    q = torch.cat(qs).view(B, 1, Hkv * gs, 128).contiguous()
    return cache, q, nprobe, es


def _oracle_step(cache, q, static_len, nprobe, es):
    BG, gs = cache.batch_groups, cache.group_size
    size_i = cache.cluster_size_i32[0].cpu() if cache.kv_residency == "device" else \
        cache.cluster_size[0].cpu().float().to(torch.int32)
    rows = size_i.sum(1)
    lk, lv = cache.list_keys[0].view(BG, -1, 128), cache.list_values[0].view(BG, -1, 128)
    sk = [lk[g, :int(rows[g])].cpu() for g in range(BG)]
    sv = [lv[g, :int(rows[g])].cpu() for g in range(BG)]
    start = torch.cumsum(size_i.long(), 1) - size_i.long()
    torch.set_num_threads(16)
    return pipeline.decode_step(
        q.view(BG, gs, 128).cpu(), cache.steady_zone_keys[0].view(BG, -1, 128).cpu(),
        cache.steady_zone_values[0].view(BG, -1, 128).cpu(), static_len, cache.centroids[0].cpu(),
        cache.value_sum[0].cpu(), cache.centroids_mask[0].cpu(), size_i, cache.cluster_size[0].cpu(), sk, sv, start,
        nprobe, es, 8, cache.buffer_size)


def _step(cache, q, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    kn = torch.randn(cache.batch_size, 1, cache.kv_head, 128, generator=g, device=dev).to(q.dtype)
    vn = torch.randn(cache.batch_size, 1, cache.kv_head, 128, generator=g, device=dev).to(q.dtype)
    cache.decode_update_kv_cache(kn, vn, 0)
    out = cache.compute(q, 0)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("name", ["c1", "c2", "c5", "c4"])
def test_benchmark_shape_decode(dev, name, dt=torch.bfloat16):
    cfg = SHAPES[name]
    cache, q, nprobe, es = _build(dev, cfg, dt)
    BG, gs = cache.batch_groups, cache.group_size
    # clustering invariants at full size
    if cache.kv_residency == "device":
        size = cache.cluster_size_i32[0]
        assert bool((size.sum(1) == cfg["N"]).all())
        assert torch.equal(cache.cluster_start[0].long(), torch.cumsum(size.long(), 1) - size.long())
    else:
        assert bool((cache.cluster_size[0].float().sum(1) == cfg["N"]).all())
    assert torch.equal(cache.centroids_mask[0], cache.cluster_size[0] == 0)

    out = _step(cache, q, dev, 77)
    static_len = cache.static_pattern_total
    ref, aux = _oracle_step(cache, q, static_len, nprobe, es)
    d = (out.view(BG, gs, 128).cpu().float() - ref.float()).abs()
    assert float(d.max()) <= MAX_ABS and float(d.mean()) <= MEAN_ABS, (float(d.max()), float(d.mean()))
    # selections against the oracle's scores: equal except ties within one bf16 ulp of a zone boundary
    cI = cache.cI[0].cpu()
    swaps = check_zone_sets(aux["dist"], cI[:, :nprobe], cI[:, nprobe:], aux["ret"], aux["est"], nprobe, es, band=1.0,
                            label=f"full size {name}" + (" f16" if dt == torch.float16 else ""))
    assert swaps <= BG * 8
    if cache.kv_residency == "host":
        # second step with the same query: blocks admitted by the first step now hit
        hit, miss = cache.block_cache_stats(0)
        assert hit == 0 and miss > 0
        out_b = _step(cache, q, dev, 78)
        assert cache.block_cache_stats(0)[0] > 0
        ref_b, _ = _oracle_step(cache, q, cache.static_pattern_total, nprobe, es)
        d = (out_b.view(BG, gs, 128).cpu().float() - ref_b.float()).abs()
        assert float(d.max()) <= MAX_ABS and float(d.mean()) <= MEAN_ABS
        return

    # exact linearity in the values: doubling every value doubles the output bit for bit
    sel_before = cache.cI[0].clone()
    out1 = cache.compute(q, 0).clone()
    for t in (cache.list_values[0], cache.steady_zone_values[0], cache.value_sum[0]):
        t.mul_(2)
    out2 = cache.compute(q, 0)
    torch.cuda.synchronize()
    assert torch.equal(cache.cI[0], sel_before)
    if dt == torch.float16:
        # an output below the smallest normal half (2^-14) was rounded on the coarser subnormal grid (2^-24)
        normal = out1.abs() >= 2.0 ** -14
        assert torch.equal(out2[normal], (out1 * 2)[normal])
        assert float((out2.float() - 2 * out1.float()).abs().max()) <= 2.0 ** -24
    else:
        assert torch.equal(out2.view(torch.int16), (out1 * 2).view(torch.int16))
    # and the step is reproducible run to run
    out3 = cache.compute(q, 0)
    torch.cuda.synchronize()
    assert torch.equal(out3, out2)


@pytest.mark.parametrize("name", ["c1", "c2", "c4"])
def test_benchmark_shape_decode_float16(dev, name):
    """The benchmark shapes with IEEE half elements (the default of the reference's harnesses, simple_test.py:29):
    the same checks, scores and probabilities rounded to fp16."""
    test_benchmark_shape_decode(dev, name, dt=torch.float16)


@pytest.mark.parametrize("S", [16, 1])
def test_kmeans_full_size_properties(dev, S):
    """Prefill clustering at the k-means benchmark shape: 8 heads x 131072 tokens, 8192 centroids,
    10 iterations, seeded random-token initialisation; with the 16 segments the cache uses, and
    unsegmented (every iteration scores all 8192 centroids)."""
    from retrievalattention_amd import synth, kernels
    from retrievalattention_amd.cache_hub.kmeans import segment_k_means_csr
    G, N, nc = 8, 131072, 8192
    ks, vs = [], []
    for h in range(G):
        k, v, _ = synth.make_group(0, 0, h, N, nc, 4, outliers=False, device=dev)
        ks.append(k.to(torch.bfloat16)); vs.append(v.to(torch.bfloat16))
    K, V = torch.stack(ks).contiguous(), torch.stack(vs).contiguous()
    g = torch.Generator(device=dev).manual_seed(123)
    init = torch.sort(torch.randperm(N, generator=g, device=dev)[:nc]).values
    r = segment_k_means_csr(K, V, nc, 10, S, init_indices=init)
    r2 = segment_k_means_csr(K, V, nc, 10, S, init_indices=init)
    torch.cuda.synchronize()
    # reproducible bit for bit
    for a, b in ((r.centroids, r2.centroids), (r.value_sum, r2.value_sum), (r.members, r2.members),
                 (r.counts, r2.counts)):
        assert torch.equal(a, b)
    counts, offsets, members, assign = r.counts.long(), r.offsets.long(), r.members.long(), r.assign.long()
    assert bool((counts.sum(1) == N).all())
    assert torch.equal(offsets[:, 1:], torch.cumsum(counts, 1)) and bool((offsets[:, 0] == 0).all())
    for h in range(G):
        # every token in exactly one list, lists grouped by cluster and ascending inside
        assert torch.equal(torch.sort(members[h]).values, torch.arange(N, device=dev))
        cl = assign[h][members[h]]
        assert bool((cl[1:] >= cl[:-1]).all())
        same = cl[1:] == cl[:-1]
        assert bool((members[h][1:][same] > members[h][:-1][same]).all())
        assert torch.equal(torch.bincount(assign[h], minlength=nc), counts[h])
        # centroid = mean of member keys, value sum = sum of member values (fp32 order differs: tolerance)
        ksum = torch.zeros(nc, 128, device=dev, dtype=torch.float32).index_add_(0, assign[h], K[h].float())
        vsum = torch.zeros(nc, 128, device=dev, dtype=torch.float32).index_add_(0, assign[h], V[h].float())
        nz = counts[h] > 0
        mean = ksum[nz] / counts[h][nz, None].float()
        assert torch.allclose(r.centroids[h][nz].float(), mean, rtol=2 ** -7, atol=1e-3)
        assert torch.allclose(r.value_sum[h][nz].float(), vsum[nz], rtol=2 ** -7, atol=2e-2)
    # assignment optimality on a sample: the chosen centroid's score is the maximum (fp64 check)
    a2 = torch.empty(G, N, dtype=torch.int32, device=dev)
    kernels.kmeans_assign(K, r.centroids, a2, G, N, nc, 1, N)
    torch.cuda.synchronize()
    gs_ = torch.Generator(device=dev).manual_seed(5)
    for h in (0, G - 1):
        idx = torch.randint(N, (2048,), generator=gs_, device=dev)
        s = K[h][idx].double() @ r.centroids[h].double().T
        best = s.max(1).values
        got = s.gather(1, a2[h][idx].long()[:, None])[:, 0]
        assert bool((got >= best - 1e-5 * best.abs().clamp(min=1.0)).all())
