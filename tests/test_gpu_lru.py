"""Device-side block cache manager against its Python restatement (oracle.wavebuf.DeviceLruModel)."""
import random

import pytest
import torch

from oracle.wavebuf import DeviceLruModel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("ncl,nprobe,capacity,buffer_size,steps,seed", [
    (200, 12, 60, 48, 40, 0),        # constant eviction pressure
    (3840, 69, 600, 552, 25, 1),     # config-4 sizes: 5 % cache
    (300, 20, 40, 30, 30, 2),        # buffer cut-off and admissions cut short
    (2500, 40, 4000, 400, 12, 3),    # cache larger than everything requested: no eviction
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
    assert any(len(m.blocks) > 0 for m in models)


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
    assert l.ri_lru_access_update(p, p, p, 8, p, 9, p, 8, p, 8, p, p, p, *ptrs, None, 0, 0, None, 1, 1024, 8, 4, 4, 8, None) == -1   # np too large
    assert l.ri_lru_access_update(p, p, p, 4, p, 9, p, 8, p, 8, p, p, p, *ptrs, None, 0, 0, None, 1, 2, 8, 4, 4, 8, None) == -1      # stride < ncl
    assert l.ri_lru_access_update(None, p, p, 8, p, 9, p, 8, p, 8, p, p, p, *ptrs, None, 0, 0, None, 1, 2, 8, 4, 4, 8, None) == -1
