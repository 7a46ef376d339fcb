"""Known-answer cases of tests/golden/known_answers.json (worked out by hand from the rules of the
reference's code, see tests/golden/make_known_answers.py) against the CPU restatement (no GPU needed)
and against the library through its C entry points (GPU)."""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import attention, kmeans as okm, scoring
from oracle.wavebuf import LruModel

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")) as f:
    KA = json.load(f)


def _dense(rows, dim=128, dtype=torch.bfloat16):
    t = torch.zeros(len(rows), dim, dtype=torch.float32)
    for i, r in enumerate(rows):
        for k, v in r.items():
            t[i, int(k)] = v
    return t.to(dtype)


def _kmeans_inputs():
    c = KA["kmeans"]
    return c, _dense(c["keys"])[None].contiguous(), _dense(c["values"])[None].contiguous()


def _check_kmeans(c, cent, vsum, clusters, size, assign=None):
    assert size.tolist() == c["cluster_size"]
    for i, members in enumerate(c["clusters"]):
        assert clusters[i, :len(members)].tolist() == members
    assert torch.equal(cent.float(), _dense(c["centroids"]).float())
    assert torch.equal(vsum.float(), _dense(c["value_sum"]).float())
    if assign is not None:
        assert list(assign) == c["assign"]


def _scoring_inputs(c):
    q = torch.zeros(1, c["gs"], 128)
    q[:, :, c["q_coord"]] = c["q_amp"]
    return q.to(torch.bfloat16), _dense(c["cent"])[None].contiguous()


def _selection_inputs():
    c = KA["selection"]
    q = torch.zeros(1, c["gs"], 128)
    q[:, :, 0] = c["q_amp"]
    cent = torch.zeros(1, c["nc"], 128)
    cent[0, :, 0] = torch.tensor(c["amps"])
    size = torch.tensor([c["sizes"]], dtype=torch.int32)
    return c, q.to(torch.bfloat16), cent.to(torch.bfloat16), size


def _attention_inputs(c):
    """One group, 4 query heads along coordinate 10, every key along coordinate 20: all logits 0."""
    n = len(c["values"])
    q = torch.zeros(1, 4, 128)
    q[:, :, 10] = 1.5
    k = torch.zeros(1, n, 128)
    k[:, :, 20] = 2.0
    v = _dense(c["values"])[None]
    w = None if c["weights"] is None else torch.tensor([c["weights"]]).to(torch.bfloat16)
    po = pl = None
    if "previous_out" in c:
        po = _dense([c["previous_out"]] * 4)[None]
        pl = torch.full((1, 4), c["previous_lse"], dtype=torch.float32)
    out = _dense([c["out"]] * 4).float()
    return q.to(torch.bfloat16), k.to(torch.bfloat16), v.contiguous(), w, po, pl, out


# ------------------------------------------------------------------ CPU restatement

@pytest.mark.parametrize("case", KA["init_indices"], ids=lambda c: f"{c['n_tokens']}x{c['n_centroids']}")
def test_oracle_init_indices(case):
    idx = okm.init_indices(case["n_tokens"], case["n_centroids"]).tolist()
    assert idx[:4] == case["first"] and idx[-2:] == case["last"] and sum(idx) == case["sum"]


@pytest.mark.parametrize("segments,iters", [(1, 3), (2, 3), (1, 10)])
def test_oracle_kmeans_hand_case(segments, iters):
    c, keys, vals = _kmeans_inputs()
    assert okm.init_indices(c["n_tokens"], c["n_centroids"]).tolist() == c["init"]
    cent, vsum, clusters, size, assign = okm.segment_k_means(keys, vals, c["n_centroids"], iters, segments)
    _check_kmeans(c, cent[0], vsum[0], clusters[0], size[0], assign[0])


@pytest.mark.parametrize("case", KA["scoring"], ids=lambda c: c["name"])
def test_oracle_scoring_exact_cases(case):
    q, cent = _scoring_inputs(case)
    _, _, _, soft = scoring.batch_gemm_softmax(q, cent)
    assert torch.allclose(soft[0].float(), torch.tensor(case["softmax"]), atol=1e-6, rtol=0)
    dist = scoring.dist_from_softmax(soft)
    assert torch.allclose(dist[0].float(), torch.tensor(case["dist"]), atol=1e-6, rtol=0)


def test_oracle_selection_ties_and_masked_clusters():
    c, q, cent, size = _selection_inputs()
    _, _, _, soft = scoring.batch_gemm_softmax(q, cent)
    ret, est = scoring.select(scoring.dist_from_softmax(soft, size == 0), c["nprobe"], c["es"])
    assert ret[0].tolist() == c["ret"] and sorted(est[0].tolist()) == sorted(c["est"])


def test_oracle_layout_cutoff():
    c = KA["layout"]
    kept, offs = scoring.retrieval_layout(torch.tensor([c["ret"]]), torch.tensor([c["cluster_size"]]),
                                          c["page"], c["max_pages"])
    assert int(kept[0]) == c["kept"]
    assert offs[0, :c["kept"] + 1].tolist() == c["token_offsets"] and int(offs[0, -1]) == c["tokens"]


def test_oracle_lru_trace():
    c = KA["lru"]
    m = LruModel(c["sizes"], c["block"], c["capacity"], c["buffer_size"])
    for s in c["steps"]:
        hit, miss = m.access(s["ids"])
        assert [list(e) for e in hit] == s["hit"] and [list(e) for e in miss] == s["miss"]
        assert [list(e) for e in m.update()] == s["update"]
        assert {str(k): v for k, v in m.resident.items()} == s["resident"]


@pytest.mark.parametrize("case", KA["attention"], ids=lambda c: c["name"])
def test_oracle_attention_rational_cases(case):
    q, k, v, w, po, pl, out = _attention_inputs(case)
    o, lse = attention.weighted_flash_decoding(q, k, v, w, po, pl)
    assert torch.equal(o[0].float(), out)
    assert torch.allclose(lse, torch.full_like(lse, case["lse"]), atol=1e-6)


def test_host_wave_buffer_lru_trace():
    """The host-side block cache manager of the library (no GPU involved) on the hand-followed trace."""
    from retrievalattention_amd import kernels
    c = KA["lru"]
    nc, nprobe, bs = len(c["sizes"]), max(len(s["ids"]) for s in c["steps"]), c["buffer_size"]
    pool = kernels.ThreadPool(2)
    wb = kernels.WaveBufferCPU(1, 1, 128, nprobe, c["block"], nc, nc, bs, c["capacity"], 2, pool.get())
    z = lambda *s: torch.zeros(s, dtype=torch.int32)
    idx = dict(hit_ids=z(1, bs), hit_sizes=z(1, bs), hit_cum=z(1, bs), hit_n=z(1),
               miss_ids=z(1, bs), miss_sizes=z(1, bs), miss_cum=z(1, bs), miss_n=z(1),
               upd_buf=z(1, bs), upd_sizes=z(1, bs), upd_cache=z(1, bs), upd_n=z(1),
               searched=torch.zeros(1, nprobe, dtype=torch.int64))
    wb.set_indices(*idx.values())
    n = sum(c["sizes"])
    kv = [torch.zeros(1, 1, 64, 128, dtype=torch.bfloat16), torch.zeros(1, 1, 64, 128, dtype=torch.bfloat16),
          torch.zeros(1, 64, 128, dtype=torch.bfloat16), torch.zeros(1, 64, 128, dtype=torch.bfloat16)]
    wb.set_kv(*kv)
    lists = np.zeros((1, nc, max(c["sizes"])), dtype=np.int32)
    row = 0
    for i, s in enumerate(c["sizes"]):
        lists[0, i, :s] = np.arange(row, row + s)
        row += s
    assert row == n
    wb.async_construction(torch.from_numpy(lists), torch.tensor([c["sizes"]], dtype=torch.int32), 0)
    wb.construction_sync()
    for s in c["steps"]:
        assert len(s["ids"]) == nprobe   # the host manager walks exactly nprobe ids per group
        idx["searched"][0] = torch.tensor(s["ids"])
        wb.batch_access()
        wb.sync()
        nh, nm, nu = int(idx["hit_n"][0]), int(idx["miss_n"][0]), int(idx["upd_n"][0])
        got = lambda a, b, d, k: [list(e) for e in zip(idx[a][0, :k].tolist(), idx[b][0, :k].tolist(), idx[d][0, :k].tolist())]
        assert got("hit_ids", "hit_sizes", "hit_cum", nh) == s["hit"]
        assert got("miss_ids", "miss_sizes", "miss_cum", nm) == s["miss"]
        assert got("upd_cache", "upd_sizes", "upd_buf", nu) == s["update"]


# ------------------------------------------------------------------ the library on the GPU

@pytest.mark.gpu
@pytest.mark.parametrize("case", KA["init_indices"], ids=lambda c: f"{c['n_tokens']}x{c['n_centroids']}")
def test_gpu_init_indices(dev, case):
    from retrievalattention_amd.cache_hub.kmeans import init_centroid_indices
    idx = init_centroid_indices(case["n_tokens"], case["n_centroids"], dev).cpu().tolist()
    assert idx[:4] == case["first"] and idx[-2:] == case["last"] and sum(idx) == case["sum"]


@pytest.mark.gpu
@pytest.mark.parametrize("segments,iters", [(1, 2), (1, 3), (1, 10)])   # (a segment needs a multiple of 32 centroids)
def test_gpu_kmeans_hand_case(dev, segments, iters):
    from retrievalattention_amd.cache_hub.kmeans import segment_k_means
    c, keys, vals = _kmeans_inputs()
    cent, vsum, clusters, size = segment_k_means(keys.to(dev), vals.to(dev), c["n_centroids"], iters, segments)
    torch.cuda.synchronize()
    _check_kmeans(c, cent[0].cpu(), vsum[0].cpu(), clusters[0].cpu(), size[0].cpu())


@pytest.mark.gpu
@pytest.mark.parametrize("case", KA["scoring"], ids=lambda c: c["name"])
def test_gpu_scoring_exact_cases(dev, case):
    from retrievalattention_amd import kernels
    q, cent = _scoring_inputs(case)
    gs, nc = case["gs"], case["nc"]
    D = torch.zeros(1, gs, nc, dtype=torch.bfloat16, device=dev)
    S = torch.zeros_like(D)
    norm = torch.zeros(1, gs, 1, dtype=torch.float32, device=dev)
    ssum = torch.zeros_like(norm)
    kernels.batch_gemm_softmax(q.to(dev), cent.to(dev), D, norm, ssum, S, 1, gs, nc, 128, 1 / math.sqrt(128), 0)
    torch.cuda.synchronize()
    assert torch.allclose(S[0].cpu().float(), torch.tensor(case["softmax"]), atol=1e-6, rtol=0)


@pytest.mark.gpu
def test_gpu_selection_and_layout(dev):
    """Ties by ascending id, masked clusters last, page cut-off and rank tables on the hand cases."""
    from retrievalattention_amd import kernels
    c, q, cent, size = _selection_inputs()
    nc, nprobe, es = c["nc"], c["nprobe"], c["es"]
    start = (torch.cumsum(size, 1) - size).to(torch.int32)

    def run(q, cent, size, start, nprobe, es, page, max_pages):
        logits = torch.empty(1, q.shape[1], cent.shape[1], dtype=torch.float32, device=dev)
        ret = torch.empty(1, nprobe, dtype=torch.int32, device=dev)
        est = torch.empty(1, max(es, 1), dtype=torch.int32, device=dev)
        off = torch.empty(1, nprobe + 1, dtype=torch.int32, device=dev)
        rst = torch.empty(1, nprobe, dtype=torch.int32, device=dev)
        meta = torch.empty(1, 4, dtype=torch.int32, device=dev)
        kernels.score_select(q.to(dev), cent.to(dev), (size == 0).to(torch.uint8).to(dev), size.to(dev), start.to(dev),
                             logits, None, None, ret, est if es else None, off, None, meta, nprobe, es, page,
                             max_pages, 1 / math.sqrt(128), ret_start=rst)
        torch.cuda.synchronize()
        return ret.cpu()[0].tolist(), est.cpu()[0, :es].tolist(), off.cpu()[0].tolist(), rst.cpu()[0].tolist(), meta.cpu()[0].tolist()

    ret, est, off, rst, meta = run(q, cent, size, start, nprobe, es, 8, 64)
    assert ret == c["ret"] and sorted(est) == sorted(c["est"])
    assert rst == [int(start[0, i]) for i in ret]

    # layout: scores that put the clusters in the hand case's rank order (amplitude falls with rank)
    L = KA["layout"]
    n = 8
    amps = [0.0] * n
    for r, cl in enumerate(L["ret"]):
        amps[cl] = 4.0 - 0.5 * r
    cent2 = torch.zeros(1, n, 128)
    cent2[0, :, 0] = torch.tensor(amps)
    size2 = torch.tensor([L["cluster_size"] + [1, 1, 1]], dtype=torch.int32)
    start2 = (torch.cumsum(size2, 1) - size2).to(torch.int32)
    # the empty cluster of the hand case must stay in the probe list: leave it unmasked by passing
    # a mask of zeros (the cut-off rule is about pages, not about the mask)
    logits = torch.empty(1, 4, n, dtype=torch.float32, device=dev)
    np_ = len(L["ret"])
    ret_t = torch.empty(1, np_, dtype=torch.int32, device=dev)
    off_t = torch.empty(1, np_ + 1, dtype=torch.int32, device=dev)
    rst_t = torch.empty(1, np_, dtype=torch.int32, device=dev)
    meta_t = torch.empty(1, 4, dtype=torch.int32, device=dev)
    kernels.score_select(q.to(dev), cent2.to(torch.bfloat16).to(dev), torch.zeros(1, n, dtype=torch.uint8, device=dev),
                         size2.to(dev), start2.to(dev), logits, None, None, ret_t, None, off_t, None, meta_t, np_, 0,
                         L["page"], L["max_pages"], 1 / math.sqrt(128), ret_start=rst_t)
    torch.cuda.synchronize()
    assert ret_t.cpu()[0].tolist() == L["ret"]
    assert off_t.cpu()[0, :L["kept"] + 1].tolist() == L["token_offsets"]
    assert meta_t.cpu()[0, 0].item() == L["kept"] and meta_t.cpu()[0, 1].item() == L["tokens"]


@pytest.mark.gpu
@pytest.mark.parametrize("case", KA["attention"], ids=lambda c: c["name"])
def test_gpu_attention_rational_cases(dev, case):
    from retrievalattention_amd import kernels
    q, k, v, w, po, pl, out = _attention_inputs(case)
    n = k.shape[1]
    o, lse = kernels.weighted_flash_decoding(
        q.view(1, 1, 4, 128).to(dev), k.view(1, n, 1, 128).to(dev), v.view(1, n, 1, 128).to(dev),
        None if w is None else w.view(1, 1, 1, n).to(dev),
        previous_out=None if po is None else po.view(1, 1, 4, 128).to(dev),
        previous_lse=None if pl is None else pl.to(dev), return_softmax_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(o.cpu().view(4, 128).float(), out)
    assert torch.allclose(lse.cpu(), torch.full((1, 4), case["lse"]), atol=1e-5)
