"""The reference's own host wave buffer (compiled by oracle/build_ref.py into oracle/_ref/) beside the
list model of oracle/wavebuf.py and the library's host manager: same K/V re-organisation, same
hit/miss/update lists step by step (wave_buffer_cpu.cpp:102-257, 513-630).

Block id values are the one thing that may differ: the reference takes free ids from an unordered_set
(:153-156), the library and the model from a stack.  Everything else is compared exactly: which clusters
hit and miss, the host rows of the misses, block sizes and offsets, which clusters are admitted, which
stay resident, and that each implementation's hit ids are the ids it handed out at admission.
Probed clusters are never empty here: for an empty cluster the reference emits one block of stale size
(:230-235 with BlockNum = 0), which the library deliberately does not reproduce."""
import glob
import importlib.util
import os

import numpy as np
import pytest
import torch

from oracle.wavebuf import LruModel
from tests.test_wavebuf import _wb

_REF_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref")


def _ref_module():
    hits = glob.glob(os.path.join(_REF_DIR, "WaveBufferRef*.so"))
    if not hits:
        pytest.skip("oracle/_ref is not built (python oracle/build_ref.py needs the reference tree)")
    spec = importlib.util.spec_from_file_location("WaveBufferRef", hits[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _clustering(rng, H, nc, n):
    """Random clustering without empty clusters: (dense lists [H, nc, max], sizes [H, nc])."""
    a = np.stack([np.concatenate([np.arange(nc), rng.integers(0, nc, n - nc)]) for _ in range(H)])
    for h in range(H):
        rng.shuffle(a[h])
    sizes = np.stack([np.bincount(a[h], minlength=nc) for h in range(H)]).astype(np.int32)
    lists = np.zeros((H, nc, int(sizes.max())), dtype=np.int32)
    for h in range(H):
        order = np.argsort(a[h], kind="stable")
        off = np.concatenate([[0], np.cumsum(sizes[h])])
        for c in range(nc):
            lists[h, c, :sizes[h, c]] = order[off[c]:off[c + 1]]
    return lists, sizes


def test_construction_matches_the_reference():
    ref = _ref_module()
    rng = np.random.default_rng(5)
    B, H, nc, n = 2, 3, 24, 500
    mine = _wb(B, H, 4, nc, nc, 64, 16, in_len=n)
    theirs = _wb(B, H, 4, nc, nc, 64, 16, in_len=n, mod=ref)
    for b in range(B):
        lists, sizes = _clustering(rng, H, nc, n)
        k = torch.randn(H, n, 128).to(torch.bfloat16)
        v = torch.randn(H, n, 128).to(torch.bfloat16)
        for wb, idx, kv, pool in (mine, theirs):
            kv["in_k"].copy_(k); kv["in_v"].copy_(v)
            wb.async_construction(torch.from_numpy(lists), torch.from_numpy(sizes), b)
            wb.construction_sync()
    for name in ("ivf_k", "ivf_v"):
        a = mine[2][name].view(B * H, -1, 128)[:, :n]
        r = theirs[2][name].view(B * H, -1, 128)[:, :n]
        assert torch.equal(a.view(torch.int16), r.view(torch.int16))


@pytest.mark.parametrize("capacity,buffer_size,seed", [(40, 64, 0), (12, 64, 1), (200, 12, 2), (6, 64, 3)])
def test_lru_lists_match_the_reference(capacity, buffer_size, seed):
    ref = _ref_module()
    rng = np.random.default_rng(seed)
    B, H, nc, n, nprobe = 1, 4, 40, 900, 6
    BG = B * H
    lists, sizes = _clustering(rng, H, nc, n)
    impls = {}
    for name, mod in (("lib", None), ("ref", ref)):
        wb, idx, kv, pool = _wb(B, H, nprobe, nc, nc, buffer_size, capacity, in_len=n, mod=mod)
        wb.async_construction(torch.from_numpy(lists), torch.from_numpy(sizes), 0)
        wb.construction_sync()
        impls[name] = (wb, idx, kv, pool)
    models = [LruModel(sizes[g], 8, capacity, buffer_size) for g in range(BG)]
    start = np.concatenate([np.zeros((BG, 1), dtype=np.int64), np.cumsum(sizes, 1)[:, :-1]], 1)
    row_to_cluster = [{int(start[g, c]): c for c in range(nc)} for g in range(BG)]
    owner = {name: [dict() for _ in range(BG)] for name in impls}     # block id -> cluster, per implementation
    hot = [rng.choice(nc, 10, replace=False) for _ in range(BG)]
    for step in range(60):
        probes = np.stack([rng.choice(hot[g], nprobe, replace=False) if rng.random() < 0.7
                           else rng.choice(nc, nprobe, replace=False) for g in range(BG)])
        got = {}
        for name, (wb, idx, kv, pool) in impls.items():
            idx["searched"].copy_(torch.from_numpy(probes.astype(np.int64)))
            wb.batch_access()
            wb.sync()
            got[name] = {k: t.clone() for k, t in idx.items()}
        for g in range(BG):
            hit, miss = models[g].access(probes[g].tolist())
            model_hit_clusters = [c for c in models[g].hit_keys for _ in range(models[g].nblk[c])]
            upd = models[g].update()
            for name in impls:
                o = got[name]
                nh, nm, nu = int(o["hit_n"][g]), int(o["miss_n"][g]), int(o["upd_n"][g])
                col = lambda key, k: o[key][g, :k].tolist()
                # misses: host row, size, offset -- exact
                assert list(zip(col("miss_ids", nm), col("miss_sizes", nm), col("miss_cum", nm))) == \
                    [tuple(e) for e in miss], (name, step, g)
                # hits: sizes and offsets exact; ids are the ones this implementation handed out
                assert list(zip(col("hit_sizes", nh), col("hit_cum", nh))) == [(s, c) for _, s, c in hit], (name, step, g)
                assert [owner[name][g][b] for b in col("hit_ids", nh)] == model_hit_clusters, (name, step, g)
                # updates: sizes and buffer offsets exact, ids free and unique
                assert list(zip(col("upd_sizes", nu), col("upd_buf", nu))) == [(s, off) for _, s, off in upd], (name, step, g)
                ids = col("upd_cache", nu)
                assert len(set(ids)) == nu and all(0 <= b < capacity for b in ids)
                # bookkeeping of who owns which block: admitted clusters are the first misses, in order
                admitted, k = [], 0
                miss_clusters = [row_to_cluster[g][r] for r, _, c in miss if r in row_to_cluster[g]]
                while k < nu:
                    c = miss_clusters[len(admitted)]
                    admitted.append(c)
                    k += models[g].nblk[c]
                assert k == nu
                resident_now = set(models[g].resident)
                new_owner = {b: c for b, c in owner[name][g].items() if c in resident_now and c not in admitted}
                k = 0
                for c in admitted:
                    for b in ids[k:k + models[g].nblk[c]]:
                        assert b not in new_owner, (name, step, g)      # a handed-out block was free
                        new_owner[b] = c
                    k += models[g].nblk[c]
                owner[name][g] = new_owner
                assert set(new_owner.values()) == resident_now, (name, step, g)
