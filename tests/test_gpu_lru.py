"""Device-side block cache manager against its Python restatement (oracle.wavebuf.DeviceLruModel), and
against the restatement of the reference's manager (oracle.wavebuf.LruModel) where the two policies coincide."""
import random

import pytest
import torch

from oracle.wavebuf import DeviceLruModel, LruModel
from tests.parity import BlockIdMap

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("ncl,nprobe,capacity,buffer_size,steps,seed", [
    (200, 12, 60, 48, 40, 0),        # constant eviction pressure
    (3840, 69, 600, 552, 25, 1),     # config-4 sizes: 5 % cache
    (300, 20, 40, 30, 30, 2),        # buffer cut-off and admissions cut short
    (2500, 40, 4000, 400, 12, 3),    # cache larger than everything requested: no eviction
    (300, 20, 0, 160, 6, 4),         # a cache without blocks (throughput_eval/test.py:77): all misses, none admitted
    (20000, 1500, 9000, 12000, 6, 5),   # probe lists past 1023 ranks (four ranks per thread)
    (40000, 3000, 2000, 20000, 5, 6),   #   with the buffer cut-off and admissions cut short
])
def test_lists_match_the_model_step_by_step(dev, ncl, nprobe, capacity, buffer_size, steps, seed):
    from retrievalattention_amd import kernels
    BG, block = 3, 8
    rnd = random.Random(seed)
    sizes = [[rnd.choice([0, 1, 7, 8, 9, 16, 23, 40]) if rnd.random() < 0.3 else rnd.randint(1, 30) for _ in range(ncl)]
             for _ in range(BG)]
    models = [DeviceLruModel(s, block, capacity, buffer_size) for s in sizes]
    sz = torch.tensor(sizes, dtype=torch.int32, device=dev)
    st = (torch.cumsum(sz.long(), 1) - sz.long()).to(torch.int32)
    lru = kernels.DeviceLru(BG, ncl + 7, int(((sz + block - 1) // block).sum(1).max()) + 5, capacity, buffer_size, block,
                            dev)
    lru.set_sizes(sz)
    lists = [torch.full((BG, buffer_size), -7, dtype=torch.int32, device=dev) if i % 4 != 3
             else torch.zeros(BG, dtype=torch.int32, device=dev) for i in range(12)]
    hot = [rnd.sample(range(ncl), min(ncl, 3 * nprobe)) for _ in range(BG)]
    for step in range(steps):
        ids = []
        for g in range(BG):   # mostly a hot set (hits), some fresh ids (misses), now and then an invalid id
            pool = hot[g] if rnd.random() < 0.8 else list(range(ncl))
            row = rnd.sample(pool, nprobe)
            if rnd.random() < 0.2:
                row[rnd.randrange(nprobe)] = ncl + 3
            ids.append(row)
        t = torch.tensor(ids, dtype=torch.int32, device=dev)
        lru.access_update(t, sz, st, lists)
        torch.cuda.synchronize()
        host = [x.cpu() for x in lists]
        for g in range(BG):
            hit, miss, upd = models[g].step(ids[g])
            for k, ref in enumerate((hit, miss, upd)):
                a, b, c, n = host[4 * k:4 * k + 4]
                assert int(n[g]) == len(ref), (step, g, k)
                got = list(zip(a[g, :len(ref)].tolist(), b[g, :len(ref)].tolist(), c[g, :len(ref)].tolist()))
                if k == 2:   # update lists are (buffer offset, size, cache block id); the model gives (id, size, offset)
                    got = [(z, y, x) for x, y, z in got]
                assert got == ref, (step, g, k)
            assert int(lru.free_count[g]) == len(models[g].free)
            assert lru.free_list[g, :len(models[g].free)].tolist() == models[g].free
            stamp = lru.stamp[g, :ncl].cpu()
            assert [int(x) for x in stamp] == models[g].stamp
            order = lru.order[g, :ncl].cpu()
            assert all(int(order[c]) == models[g].sub[c] for c in models[g].blocks)
    assert capacity == 0 or any(len(m.blocks) > 0 for m in models)


@pytest.mark.parametrize("ncl,nprobe,capacity,steps,seed", [(40, 1, 24, 250, 0), (300, 1, 64, 250, 1), (200, 12, 60, 80, 2),
                                                           (60, 8, 10, 120, 3), (3000, 150, 900, 40, 4)])
def test_lists_equal_the_reference_policy(dev, ncl, nprobe, capacity, steps, seed):
    """The kernel's hit / miss / admission lists and its evictions equal those of the reference's manager
    (LruModel, itself checked against the reference's own BufferManager build) over random probe traces: one
    probe per step, several probes with eviction pressure, a cache smaller than one step's hits (hits of the
    current step are evicted), a config-4-like size.  Block id values aside: an id map is kept and must stay
    a bijection."""
    from retrievalattention_amd import kernels
    BG, block, buffer_size = 2, 8, max(16, 4 * nprobe)
    rnd = random.Random(seed)
    sizes = [[rnd.randint(0, 30) for _ in range(ncl)] for _ in range(BG)]
    refs = [LruModel(s, block, capacity, buffer_size) for s in sizes]
    maps = [BlockIdMap() for _ in range(BG)]
    sz = torch.tensor(sizes, dtype=torch.int32, device=dev)
    st = (torch.cumsum(sz.long(), 1) - sz.long()).to(torch.int32)
    lru = kernels.DeviceLru(BG, ncl, int(((sz + block - 1) // block).sum(1).max()) + 1, capacity, buffer_size, block, dev)
    lru.set_sizes(sz)
    lists = [torch.full((BG, buffer_size), -7, dtype=torch.int32, device=dev) if i % 4 != 3
             else torch.zeros(BG, dtype=torch.int32, device=dev) for i in range(12)]
    hot = [rnd.sample(range(ncl), max(2, min(ncl, 3 * nprobe), ncl // 3 if nprobe == 1 else 0)) for _ in range(BG)]
    evictions = 0
    for step in range(steps):
        ids = [rnd.sample(hot[g] if rnd.random() < 0.6 else range(ncl), nprobe) for g in range(BG)]
        lru.access_update(torch.tensor(ids, dtype=torch.int32, device=dev), sz, st, lists)
        torch.cuda.synchronize()
        host = [x.cpu() for x in lists]
        for g in range(BG):
            before = set(refs[g].resident)
            hit, miss = refs[g].access(ids[g])
            upd = refs[g].update()
            evictions += len(before - set(refs[g].resident))
            lists_g = []
            for k, ref in enumerate((hit, miss, upd)):
                a, b, c, n = host[4 * k:4 * k + 4]
                assert int(n[g]) == len(ref), (step, g, k)
                got = list(zip(a[g, :len(ref)].tolist(), b[g, :len(ref)].tolist(), c[g, :len(ref)].tolist()))
                lists_g.append([(z, y, x) for x, y, z in got] if k == 2 else got)
            # hits: block ids through the map (a hit of this step may be evicted by the same step's admission)
            assert [(maps[g].to_ref(x), y, z) for x, y, z in lists_g[0]] == hit, (step, g, 0)
            assert lists_g[1] == miss, (step, g, 1)      # misses: host rows, no block ids involved
            # blocks of clusters evicted in this step go back to the free list and may be handed out again at once
            maps[g].retain({b for ids_c in refs[g].resident.values() for b in ids_c} - {b for b, _, _ in upd})
            for (bg, _, _), (br, _, _) in zip(lists_g[2], upd):     # admission hands out ids: the map learns them
                maps[g].bind(bg, br)
            assert [(maps[g].to_ref(x), y, z) for x, y, z in lists_g[2]] == upd, (step, g, 2)
            # the same clusters are resident: evictions happened in the same order
            resident = set(torch.nonzero(lru.stamp[g, :ncl]).flatten().tolist())
            assert resident == set(refs[g].resident), (step, g)
    assert evictions > 0


def test_row_table_for_attention_in_place(dev):
    """With a row table the manager lists no hits for copying and writes, for every retrieved token in
    rank order, its row in a tensor that holds the cache blocks followed by the staged misses."""
    from retrievalattention_amd import kernels
    BG, block, ncl, nprobe, capacity, buffer_size = 2, 8, 500, 30, 150, 120
    rnd = random.Random(9)
    sizes = [[rnd.randint(0, 45) for _ in range(ncl)] for _ in range(BG)]
    stage0 = capacity * block
    models = [DeviceLruModel(s, block, capacity, buffer_size, stage_row0=stage0) for s in sizes]
    sz = torch.tensor(sizes, dtype=torch.int32, device=dev)
    st = (torch.cumsum(sz.long(), 1) - sz.long()).to(torch.int32)
    lru = kernels.DeviceLru(BG, ncl, int(((sz + block - 1) // block).sum(1).max()), capacity, buffer_size, block, dev)
    lru.set_sizes(sz)
    lists = [torch.zeros((BG, buffer_size), dtype=torch.int32, device=dev) if i % 4 != 3
             else torch.zeros(BG, dtype=torch.int32, device=dev) for i in range(12)]
    row_src = torch.full((BG, buffer_size * block), -1, dtype=torch.int32, device=dev)
    meta = torch.zeros(BG, 4, dtype=torch.int32, device=dev)
    hot = [rnd.sample(range(ncl), 60) for _ in range(BG)]
    for step in range(25):
        ids = [rnd.sample(hot[g] if rnd.random() < 0.7 else range(ncl), nprobe) for g in range(BG)]
        lru.access_update(torch.tensor(ids, dtype=torch.int32, device=dev), sz, st, lists, row_src=row_src,
                          stage_row0=stage0, meta=meta)
        torch.cuda.synchronize()
        for g in range(BG):
            hit, miss, upd = models[g].step(ids[g])
            rows = models[g].rows
            assert int(meta[g, 1]) == len(rows) and int(meta[g, 2]) == len(hit) + len(miss)
            assert row_src[g, :len(rows)].tolist() == rows
            assert int(lists[3][g]) == 0 and int(lists[7][g]) == len(miss) and int(lists[11][g]) == len(upd)
            assert lru.free_list[g, :len(models[g].free)].tolist() == models[g].free
    assert any(any(r < stage0 for r in m.rows) for m in models) and any(any(r >= stage0 for r in m.rows) for m in models)


def test_bad_arguments(dev):
    from retrievalattention_amd import _lib
    l = _lib.lib()
    z = torch.zeros(64, dtype=torch.int32, device=dev)
    p = z.data_ptr()
    ptrs = [p] * 12
    assert l.ri_lru_access_update(p, p, p, 8, p, 9, p, p, 8, p, 8, p, p, p, *ptrs, None, 0, 0, None, 1, 4097, 8, 4, 4, 8, None) == -1   # np too large
    assert l.ri_lru_access_update(p, p, p, 4, p, 9, p, p, 8, p, 8, p, p, p, *ptrs, None, 0, 0, None, 1, 2, 8, 4, 4, 8, None) == -1      # stride < ncl
    assert l.ri_lru_access_update(None, p, p, 8, p, 9, p, p, 8, p, 8, p, p, p, *ptrs, None, 0, 0, None, 1, 2, 8, 4, 4, 8, None) == -1
