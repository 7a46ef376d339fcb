"""The index that prefill_update_kv_cache writes, against the oracle (GPU).

Reference: cache_hub/retroinfer_cache.py:384-436 (steady zone slices, bf16 mean, centred keys into
segment_k_means, centroids = clustering centroids + mean, mask = size == 0, bf16 sizes) and
wave_buffer_cpu.cpp:545-567 (K/V rows re-organised cluster by cluster).

The clustering trajectory itself is chaotic under near-ties of the assignment (checked step by step in
test_gpu_kmeans.py), so the index is checked given the final assignment the kernels produced: everything
the wrapper derives from it must equal the oracle's result bit for bit.  When the oracle's own end-to-end
run lands on the same assignment (the usual case) the whole index, empty clusters included, must equal
oracle.pipeline.prefill_index.
"""
import numpy as np
import pytest
import torch

from oracle import kmeans as okm
from oracle import pipeline
from tests.parity import ulp_distance_bf16

pytestmark = pytest.mark.gpu


def _cache(dev, residency, B, Hkv, gs, ctx, nc, S, valid_start):
    from retrievalattention_amd.cache_hub import retroinfer_cache
    block_cache = "host" if residency == "host-cpu" else "device"
    return retroinfer_cache(
        valid_start=valid_start, layer_num=1, batch_size=B, max_length=ctx + 8, num_key_value_heads=Hkv,
        num_heads=Hkv * gs, head_dim=128, dtype=torch.bfloat16, layer_mapping={"0": "cuda:0"}, max_new_length=8,
        static_pattern_start=4, static_pattern_end=64, core=4, n_centroids=nc, n_segment=S, nprobe=8,
        max_compute_cluster_num=48, cache_unit_size=8, cache_cluster_num=24, num_gpus=1, model_size=8,
        kv_residency="host" if residency.startswith("host") else "device", block_cache=block_cache)


@pytest.mark.parametrize("residency", ["device", "host", "host-cpu"])
def test_prefill_index_matches_oracle(dev, residency, monkeypatch):
    import importlib
    from retrievalattention_amd import synth
    rc_mod = importlib.import_module("retrievalattention_amd.cache_hub.retroinfer_cache")   # the module, not the class
    B, Hkv, gs, ctx, nc, S = 2, 2, 4, 2048 + 68, 128, 2
    vstart = [0, 40]                       # the second sequence is left-padded
    cache = _cache(dev, residency, B, Hkv, gs, ctx, nc, S, vstart)
    k, v, _ = synth.make_batch(7, B, Hkv, ctx, 100, gs, outliers=True)      # [B, Hkv, ctx, 128] bf16 on the CPU
    # a few clusters stay empty: 100 mixture centres for 128 centroids, and a block of identical tokens
    k[:, :, 300:340] = k[:, :, 300:301]

    recorded = []
    real = rc_mod.segment_k_means_csr

    def spy(key, value, num_centroids, **kw):
        r = real(key, value, num_centroids, **kw)
        recorded.append(dict(key=key.cpu().clone(), value=value.cpu().clone(), centroids=r.centroids.cpu().clone(),
                             assign=r.assign.cpu().clone(), counts=r.counts.cpu().clone(), kw=kw, nc=num_centroids))
        return r

    monkeypatch.setattr(rc_mod, "segment_k_means_csr", spy)
    for b in range(B):
        K = k[b].transpose(0, 1)[None].contiguous().to(dev)
        V = v[b].transpose(0, 1)[None].contiguous().to(dev)
        rk, rv = cache.prefill_update_kv_cache(None, K, V, 0, b)
        cache.sync(0, b)
        assert torch.equal(rk, K[:, vstart[b]:]) and torch.equal(rv, V[:, vstart[b]:])
    cache.prepare_cache()
    torch.cuda.synchronize()
    assert len(recorded) == B and cache.context == ctx

    BG = B * Hkv
    lk, lv = cache.list_keys[0].view(BG, -1, 128), cache.list_values[0].view(BG, -1, 128)
    whole_index_checked = 0
    for b in range(B):
        vs = vstart[b]
        N = ctx - 68 - vs
        keys, vals = k[b, :, vs + 4:ctx - 64], v[b, :, vs + 4:ctx - 64]          # [Hkv, N, 128]
        rec = recorded[b]
        assert rec["nc"] == nc and rec["kw"].get("num_segments") == S
        # steady zone: first 4 valid tokens, then the last 64 (retroinfer_cache.py:406-413)
        for zone, src in ((cache.steady_zone_keys[0], k), (cache.steady_zone_values[0], v)):
            assert torch.equal(zone[b, :, :4].cpu(), src[b, :, vs:vs + 4])
            assert torch.equal(zone[b, :, 4:68].cpu(), src[b, :, ctx - 64:])
        # bf16 mean over the clustered tokens (:416): the reference takes torch.mean of the bf16 tensor on
        # the device; it must sit within one bf16 ulp of the exact mean, and is then the value used
        mean = torch.mean(keys.contiguous().to(dev), dim=1, keepdim=True).cpu()
        exact = keys.double().mean(dim=1, keepdim=True).to(torch.bfloat16)
        assert int(ulp_distance_bf16(mean, exact).max()) <= 1
        centred = keys - mean                                                      # bf16 arithmetic, as :419
        assert torch.equal(rec["key"], centred), "segment_k_means must receive bf16(keys - bf16 mean)"
        assert torch.equal(rec["value"], vals)
        # independent end-to-end run of the oracle on the same tensors
        ref = pipeline.prefill_index(keys, vals, nc, S)
        for h in range(Hkv):
            gi = b * Hkv + h
            a = rec["assign"][h].numpy().astype(np.int64)
            lists, cnt = okm.reverse_index(a, nc)
            s, cnt2 = okm.cluster_sums(centred[h], a, nc)
            assert np.array_equal(cnt, cnt2) and int(cnt.sum()) == N
            filled = torch.from_numpy(cnt > 0)
            assert int((~filled).sum()) > 0, "the case should contain empty clusters"
            # centroids = bf16(bf16(sum / count) + mean) for filled clusters (:429); empty ones keep the
            # clustering's centroid, plus the mean
            c_km = okm.update(rec["centroids"][h], s, cnt, False)
            assert torch.equal(c_km, rec["centroids"][h])
            assert torch.equal(cache.centroids[0][gi].cpu(), c_km + mean[h])
            assert torch.equal(cache.value_sum[0][gi].cpu(), okm.value_sum(vals[h], a, nc))
            assert torch.equal(cache.centroids_mask[0][gi].cpu(), ~filled)
            size = torch.from_numpy(cnt)
            assert torch.equal(cache.cluster_size[0][gi].cpu(), size.to(torch.bfloat16))
            assert torch.equal(cache.cluster_size_i32[0][gi].cpu(), size)
            start = torch.cumsum(size.long(), 0) - size.long()
            assert torch.equal(cache.cluster_start[0][gi].cpu().long(), start)
            assert cache.store_rows[0][gi] == N
            # store: rows [start[c], start[c] + size[c]) are cluster c's tokens in ascending order
            sk, sv, st = pipeline.cluster_store(keys[h], vals[h], lists, size)
            assert torch.equal(st, start)
            assert torch.equal(lk[gi, :N].cpu(), sk), "key store rows are misplaced"
            assert torch.equal(lv[gi, :N].cpu(), sv), "value store rows are misplaced"
            for c in (0, 1, nc // 2, nc - 1):
                s0, n = int(start[c]), int(size[c])
                assert torch.equal(lk[gi, s0:s0 + n].cpu(), keys[h][torch.from_numpy(lists[c, :n].astype(np.int64))])
            # when the oracle's own trajectory ends on the same assignment, the whole index agrees
            if np.array_equal(ref["assign"][h], a):
                whole_index_checked += 1
                assert torch.equal(cache.centroids[0][gi].cpu(), ref["centroids"][h])
                assert torch.equal(cache.value_sum[0][gi].cpu(), ref["value_sum"][h])
                assert torch.equal(cache.centroids_mask[0][gi].cpu(), ref["mask"][h])
                assert torch.equal(cache.cluster_size[0][gi].cpu(), ref["size_bf16"][h])
    print(f"[prefill index] {whole_index_checked} of {BG} heads reproduced the oracle's end-to-end run exactly")


def test_permute_rows_bit_exact(dev):
    """ri_permute_rows: out[p, i] = in[p, members[p, i]] with row strides larger than the row count on
    both sides; rows of the output beyond the count stay untouched (wave_buffer_cpu.cpp:545-567)."""
    from retrievalattention_amd import kernels
    g = torch.Generator().manual_seed(3)
    for P, N, si, so in ((3, 1000, 1100, 1300), (1, 17, 17, 40), (5, 4096, 4096, 4096), (2, 1, 8, 8)):
        src = torch.randn(P, si, 128, generator=g).to(torch.bfloat16)
        members = torch.stack([torch.randperm(N, generator=g) for _ in range(P)]).to(torch.int32)
        if N > 2:
            members[0, 1] = members[0, 0]          # a gather, not necessarily a permutation
        dst = torch.full((P, so, 128), 7.0, dtype=torch.bfloat16)
        sd, md, dd = src.to(dev), members.to(dev), dst.to(dev)
        kernels.permute_rows(sd, md, dd, P, N, si, so)
        torch.cuda.synchronize()
        ref = dst.clone()
        for p in range(P):
            ref[p, :N] = src[p, members[p].long()]
        assert torch.equal(dd.cpu(), ref)
    # a view as destination: rows land behind an offset inside a larger store (how the index fold appends)
    P, N, stride, base = 2, 64, 256, 100
    src = torch.randn(P, N, 128, generator=g).to(torch.bfloat16)
    members = torch.stack([torch.randperm(N, generator=g) for _ in range(P)]).to(torch.int32)
    store = torch.zeros(P, stride, 128, dtype=torch.bfloat16, device=dev)
    kernels.permute_rows(src.to(dev), members.to(dev), store[:, base:], P, N, N, stride)
    torch.cuda.synchronize()
    ref = torch.zeros(P, stride, 128, dtype=torch.bfloat16)
    for p in range(P):
        ref[p, base:base + N] = src[p, members[p].long()]
    assert torch.equal(store.cpu(), ref)
