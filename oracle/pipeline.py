"""Prefill wrapper and one decode step of retroinfer_cache, restated with the oracle's parts
(cache_hub/retroinfer_cache.py:384-436 prefill, :549-697 compute)."""
import math

import numpy as np
import torch

from . import attention, kmeans, scoring


def prefill_index(keys, values, n_centroids, n_segment, num_iters=10):
    """keys/values [H, N, D] bf16: the clustered tokens of one sequence.
    Returns dict(centroids, value_sum, mask, size_bf16, size, lists, assign) per head
    (retroinfer_cache.py:416-436: centre by the bf16 mean, cluster, add the mean back)."""
    mean_key = torch.mean(keys, dim=1, keepdim=True)
    cent, vsum, clusters, csize, assign = kmeans.segment_k_means(keys - mean_key, values, n_centroids,
                                                                 num_iters, n_segment)
    return dict(centroids=cent + mean_key, value_sum=vsum, mask=csize == 0, size_bf16=csize.to(keys.dtype),
                size=csize, lists=clusters, assign=assign)


def cluster_store(keys, values, lists, size):
    """Cluster-contiguous K/V of one head (wave_buffer_cpu.cpp:545-567) and cluster start rows."""
    order = np.concatenate([lists[c, :int(size[c])] for c in range(lists.shape[0])] + [np.zeros(0, np.int64)])
    order = torch.from_numpy(order.astype(np.int64))
    start = torch.cumsum(size.long(), 0) - size.long()
    return keys[order], values[order], start


def decode_step(q, steady_k, steady_v, static_len, centroids, value_sum, mask, size_i32, size_bf16, store_k,
                store_v, start, nprobe, es, page, max_pages, logits=None, zone_logits=None):
    """One layer's decode attention for all groups.
    q [BG, gs, D]; steady_* [BG, >=static_len, D]; centroids/value_sum [BG, nc, D]; mask, size_* [BG, nc];
    store_* list of per-group [rows, D]; start [BG, nc].  `logits` lets a test substitute the scores the
    kernels produced.  `zone_logits`: scores of another (predicted) query that choose the zones while the
    estimation zone is still scored by q (next-layer cluster estimation, retroinfer_cache.py:582-617).  Returns (out bf16 [BG, gs, D], aux)."""
    BG, gs, D = q.shape
    scale = 1.0 / math.sqrt(D)
    x = scoring.logits_fp32(q, centroids, scale) if logits is None else logits
    _, _, _, soft = scoring.softmax_from_logits(x if zone_logits is None else zone_logits, q.dtype)
    dist = scoring.dist_from_softmax(soft, mask)
    ret, est = scoring.select(dist, nprobe, es)
    kept, offs = scoring.retrieval_layout(ret, size_i32, page, max_pages)
    out = torch.empty(BG, gs, D, dtype=q.dtype)
    for g in range(BG):
        ks, vs = [steady_k[g, :static_len]], [steady_v[g, :static_len]]
        for c in ret[g, :int(kept[g])]:
            s0, n = int(start[g, c]), int(size_i32[g, c])
            ks.append(store_k[g][s0:s0 + n]); vs.append(store_v[g][s0:s0 + n])
        po = pl = None
        if es > 0:
            eo, el = attention.estimation(x[g:g + 1], est[g:g + 1], value_sum[g:g + 1], size_bf16[g:g + 1])
            po, pl = eo.to(q.dtype), el.float()
        out[g] = attention.weighted_flash_decoding(q[g:g + 1], torch.cat(ks)[None], torch.cat(vs)[None], None,
                                                   po, pl)[0][0]
    return out, dict(dist=dist, ret=ret, est=est, kept=kept, offs=offs, logits=x)
