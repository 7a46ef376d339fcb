"""Host wave buffer (LRU block cache manager, K/V re-organisation, worker pool) against the
list model in oracle/wavebuf.py and the invariants of the reference's BufferManager
(wave_buffer_cpu.cpp:102-257).  Runs without a GPU: this part of the library is host code."""
import numpy as np
import pytest
import torch

from oracle.wavebuf import LruModel


def _wb(B, H, nprobe, nc, final_nc, buffer_size, capacity, threads=3, list_len=4096, in_len=4096, mod=None):
    """A wave buffer with its index and K/V tensors; `mod` = module providing ThreadPool and WaveBufferCPU
    (the library's by default)."""
    if mod is None:
        from retrievalattention_amd import kernels as mod
    pool = mod.ThreadPool(threads)
    wb = mod.WaveBufferCPU(B, H, 128, nprobe, 8, nc, final_nc, buffer_size, capacity, threads, pool.get())
    BG = B * H
    z = lambda *s: torch.zeros(s, dtype=torch.int32)
    idx = dict(hit_ids=z(BG, buffer_size), hit_sizes=z(BG, buffer_size), hit_cum=z(BG, buffer_size), hit_n=z(BG),
               miss_ids=z(BG, buffer_size), miss_sizes=z(BG, buffer_size), miss_cum=z(BG, buffer_size), miss_n=z(BG),
               upd_buf=z(BG, buffer_size), upd_sizes=z(BG, buffer_size), upd_cache=z(BG, buffer_size), upd_n=z(BG),
               searched=torch.zeros(BG, nprobe, dtype=torch.int64))
    wb.set_indices(*idx.values())
    kv = dict(ivf_k=torch.zeros(B, H, list_len, 128, dtype=torch.bfloat16), ivf_v=torch.zeros(B, H, list_len, 128, dtype=torch.bfloat16),
              in_k=torch.zeros(H, in_len, 128, dtype=torch.bfloat16), in_v=torch.zeros(H, in_len, 128, dtype=torch.bfloat16))
    wb.set_kv(*kv.values())
    return wb, idx, kv, pool


def _construct(wb, kv, B, H, nc, n_tokens, rng):
    """Random clustering per batch; returns sizes [B*H, nc] and the expected organised K rows."""
    sizes_all, expect = [], []
    for b in range(B):
        kv["in_k"].copy_(torch.randn(kv["in_k"].shape).to(torch.bfloat16))
        kv["in_v"].copy_(torch.randn(kv["in_v"].shape).to(torch.bfloat16))
        a = rng.integers(0, nc, (H, n_tokens))
        a[:, :3] = 0
        sizes = np.stack([np.bincount(a[h], minlength=nc) for h in range(H)]).astype(np.int32)
        mx = int(sizes.max())
        lists = np.zeros((H, nc, mx), dtype=np.int32)
        for h in range(H):
            order = np.argsort(a[h], kind="stable")
            off = np.concatenate([[0], np.cumsum(sizes[h])])
            for c in range(nc):
                lists[h, c, :sizes[h, c]] = order[off[c]:off[c + 1]]
            expect.append((kv["in_k"][h][torch.from_numpy(order)].clone(), kv["in_v"][h][torch.from_numpy(order)].clone()))
        wb.async_construction(torch.from_numpy(lists), torch.from_numpy(sizes), b)
        wb.construction_sync()
        sizes_all.append(sizes)
    return np.concatenate(sizes_all), expect


def test_construction_organises_kv_by_cluster():
    rng = np.random.default_rng(0)
    B, H, nc, n = 2, 3, 40, 700
    wb, idx, kv, pool = _wb(B, H, 5, nc, nc, 64, 32)
    sizes, expect = _construct(wb, kv, B, H, nc, n, rng)
    for g in range(B * H):
        assert torch.equal(kv["ivf_k"].view(B * H, -1, 128)[g, :n], expect[g][0])
        assert torch.equal(kv["ivf_v"].view(B * H, -1, 128)[g, :n], expect[g][1])


@pytest.mark.parametrize("capacity,buffer_size,seed", [(40, 64, 0), (12, 64, 1), (200, 10, 2), (0, 64, 3)])
def test_lru_matches_model(capacity, buffer_size, seed):
    """Random probe sequences with locality; every access/update list must equal the model's,
    with the invariants of the block cache holding at each step."""
    rng = np.random.default_rng(seed)
    B, H, nc, n, nprobe = 1, 4, 48, 900, 6
    wb, idx, kv, pool = _wb(B, H, nprobe, nc, nc, buffer_size, capacity)
    sizes, _ = _construct(wb, kv, B, H, nc, n, rng)
    BG = B * H
    models = [LruModel(sizes[g], 8, capacity, buffer_size) for g in range(BG)]
    hot = [rng.choice(nc, 12, replace=False) for _ in range(BG)]
    for step in range(40):
        for g in range(BG):
            pick = rng.choice(hot[g], nprobe, replace=False) if rng.random() < 0.7 else rng.choice(nc, nprobe, replace=False)
            idx["searched"][g] = torch.from_numpy(pick.astype(np.int64))
        wb.batch_access()
        wb.sync()
        for g in range(BG):
            hit, miss = models[g].access(idx["searched"][g].tolist())
            nh, nm = int(idx["hit_n"][g]), int(idx["miss_n"][g])
            assert nh == len(hit) and nm == len(miss)
            got_hit = list(zip(idx["hit_ids"][g, :nh].tolist(), idx["hit_sizes"][g, :nh].tolist(), idx["hit_cum"][g, :nh].tolist()))
            got_miss = list(zip(idx["miss_ids"][g, :nm].tolist(), idx["miss_sizes"][g, :nm].tolist(), idx["miss_cum"][g, :nm].tolist()))
            assert got_hit == hit and got_miss == miss
            upd = models[g].update()
            nu = int(idx["upd_n"][g])
            got_upd = list(zip(idx["upd_cache"][g, :nu].tolist(), idx["upd_sizes"][g, :nu].tolist(), idx["upd_buf"][g, :nu].tolist()))
            assert got_upd == upd
            # invariants: resident blocks within capacity, block ids unique and in range
            blocks = [b for ids in models[g].resident.values() for b in ids]
            assert len(blocks) == len(set(blocks)) and len(blocks) + len(models[g].free) == capacity
            assert all(0 <= b < capacity for b in blocks)
            # every probed cluster that fits appears exactly once, in hits or misses
            assert sum(s for _, s, _ in hit) + sum(s for _, s, _ in miss) <= buffer_size * 8
    if buffer_size == 10:
        assert wb.overflow_events() > 0           # the buffer cut-off was exercised
    if capacity == 0:
        assert all(int(idx["hit_n"][g]) == 0 for g in range(BG))   # nothing is ever admitted


def test_eviction_is_least_recently_used():
    """Capacity for exactly three 1-block clusters: touching A keeps it, the untouched one goes."""
    B, H, nc, nprobe = 1, 1, 8, 1
    wb, idx, kv, pool = _wb(B, H, nprobe, nc, nc, 8, 3)
    sizes = np.full((1, nc), 5, dtype=np.int32)
    lists = np.arange(nc * 5, dtype=np.int32).reshape(1, nc, 5)
    wb.async_construction(torch.from_numpy(lists), torch.from_numpy(sizes), 0)
    wb.construction_sync()

    def probe(c):
        idx["searched"][0, 0] = c
        wb.batch_access(); wb.sync()
        return int(idx["hit_n"][0]), int(idx["miss_n"][0])

    assert probe(0) == (0, 1) and probe(1) == (0, 1) and probe(2) == (0, 1)
    assert probe(0) == (1, 0)          # A is resident and becomes most recent
    assert probe(3) == (0, 1)          # admits D, evicts B (least recently used)
    assert probe(1) == (0, 1)          # B is gone (this evicts C)
    assert probe(0) == (1, 0)          # A survived both evictions


def test_empty_clusters_are_skipped_and_update_kv_appends():
    """A probed cluster of size 0 yields no block (the reference would emit a bogus 8-vector
    block, wave_buffer_cpu.cpp:536 with :230-235); update_kv appends clusters behind the prompt's."""
    B, H, nc, nprobe = 1, 2, 6, 3
    wb, idx, kv, pool = _wb(B, H, nprobe, nc, nc + 4, 16, 8)
    sizes = np.array([[3, 0, 9, 0, 8, 4]] * H, dtype=np.int32)
    n = int(sizes[0].sum())
    lists = np.zeros((H, nc, 9), dtype=np.int32)
    off = np.concatenate([[0], np.cumsum(sizes[0])])
    for h in range(H):
        for c in range(nc):
            lists[h, c, :sizes[h, c]] = np.arange(off[c], off[c + 1])
    kv["in_k"][:, :n] = torch.randn(H, n, 128).to(torch.bfloat16)
    wb.async_construction(torch.from_numpy(lists), torch.from_numpy(sizes), 0)
    wb.construction_sync()
    idx["searched"][:] = torch.tensor([1, 2, 3])
    wb.batch_access(); wb.sync()
    assert idx["miss_n"].tolist() == [2, 2]                       # cluster 2 only: blocks of 8 and 1
    assert idx["miss_ids"][0, :2].tolist() == [3, 11] and idx["miss_sizes"][0, :2].tolist() == [8, 1]
    # append 4 new clusters of sizes 2,0,5,1 built from 8 new tokens
    new_sizes = np.array([[2, 0, 5, 1]] * H, dtype=np.int32)
    new_lists = np.zeros((H, 4, 5), dtype=np.int32)
    new_lists[:, 0, :2] = [0, 1]; new_lists[:, 2, :5] = [2, 3, 4, 5, 6]; new_lists[:, 3, :1] = [7]
    uk = torch.randn(H, 8, 128).to(torch.bfloat16); uv = torch.randn(H, 8, 128).to(torch.bfloat16)
    wb.update_kv(uk, uv, torch.from_numpy(new_lists), torch.from_numpy(new_sizes))
    assert torch.equal(kv["ivf_k"].view(H, -1, 128)[:, n:n + 8], uk)
    idx["searched"][:] = torch.tensor([6, 8, 9])                   # new clusters 0, 2, 3
    wb.batch_access(); wb.sync()
    assert idx["miss_ids"][0, :3].tolist() == [n, n + 2, n + 7]
    assert idx["miss_sizes"][0, :3].tolist() == [2, 5, 1]


def test_bad_arguments_are_rejected():
    from retrievalattention_amd import kernels
    pool = kernels.ThreadPool(1)
    with pytest.raises(ValueError):
        kernels.WaveBufferCPU(1, 1, 128, 0, 8, 4, 4, 4, 4, 1, pool.get())     # nprobe = 0
    wb = kernels.WaveBufferCPU(1, 1, 128, 1, 8, 4, 4, 4, 4, 1, pool.get())
    with pytest.raises(RuntimeError, match="before it was set up"):
        wb.batch_access()


def test_pinned_workers():
    """Worker i bound to core first_core + i (thread_pool.hpp:18-23, 65-66): as many workers report a
    binding as there are cores the process may use among those asked for; the pool then works as usual."""
    import os
    from retrievalattention_amd import kernels
    allowed = os.sched_getaffinity(0)
    pool = kernels.ThreadPool(3, first_core=0)
    assert pool.pinned_workers == len(allowed & {0, 1, 2})
    assert kernels.ThreadPool(2).pinned_workers == 0
    wb = kernels.WaveBufferCPU(1, 1, 128, 1, 8, 4, 4, 4, 4, 2, pool.get())
    del wb, pool


@pytest.mark.parametrize("ncl,nprobe,capacity,buffer_size,steps,seed", [
    (200, 12, 60, 48, 80, 0),        # constant eviction pressure, several probes per step
    (60, 8, 10, 64, 120, 1),         # a cache smaller than one step's hits: hits of the current step are evicted
    (300, 20, 40, 30, 60, 2),        # buffer cut-off and admission prefix
    (40, 1, 24, 16, 250, 3),         # one probe per step
    (500, 30, 4000, 400, 30, 4),     # no eviction at all
    (30, 6, 0, 64, 20, 5),           # no cache
])
def test_device_manager_model_follows_the_reference_policy(ncl, nprobe, capacity, buffer_size, steps, seed):
    """DeviceLruModel (what the device-side manager is compared with, list by list) keeps the reference's
    policy: over random probe traces its hit, miss and admission lists and the set of resident clusters after
    every step equal those of LruModel, which is pinned by the reference's own BufferManager build; only the
    block id values differ (the two hand out free ids in different orders; the map must stay a bijection)."""
    import random
    from oracle.wavebuf import DeviceLruModel
    from tests.parity import BlockIdMap
    rnd = random.Random(seed)
    sizes = [rnd.choice([0, 1, 7, 8, 9, 16, 23]) if rnd.random() < 0.3 else rnd.randint(1, 30) for _ in range(ncl)]
    dev_m, ref_m, ids_map = DeviceLruModel(sizes, 8, capacity, buffer_size), LruModel(sizes, 8, capacity, buffer_size), BlockIdMap()
    hot = rnd.sample(range(ncl), min(ncl, 3 * nprobe))
    evictions = evicted_hits = 0
    for step in range(steps):
        ids = rnd.sample(hot if rnd.random() < 0.7 else range(ncl), nprobe)
        before = set(ref_m.resident)
        hit_r, miss_r = ref_m.access(ids)
        hit_keys = list(ref_m.hit_keys)
        upd_r = ref_m.update()
        gone = before - set(ref_m.resident)
        evictions += len(gone)
        evicted_hits += len(gone & set(hit_keys))
        hit_d, miss_d, upd_d = dev_m.step(ids)
        assert miss_d == miss_r
        assert [(ids_map.to_ref(b), s, o) for b, s, o in hit_d] == hit_r
        ids_map.retain({b for v in ref_m.resident.values() for b in v} - {b for b, _, _ in upd_r})
        assert len(upd_d) == len(upd_r)
        for (bd, _, _), (br, _, _) in zip(upd_d, upd_r):
            ids_map.bind(bd, br)
        assert [(ids_map.to_ref(b), s, o) for b, s, o in upd_d] == upd_r
        assert set(dev_m.blocks) == set(ref_m.resident)
        used = [b for v in dev_m.blocks.values() for b in v]
        assert len(set(used)) == len(used) and not set(used) & set(dev_m.free) and len(used) + len(dev_m.free) == capacity
    if seed in (0, 1, 3):
        assert evictions > 0
    if seed == 1:
        assert evicted_hits > 0
